// Host-logic tests of the slice pipeline (fairring_amd/csrc/pipeline.cc and its
// schedule_*.cc behind the C ABI) on the fake HIP runtime: no GPU, meant to run under
// ThreadSanitizer and AddressSanitizer. Each scenario prints its name and
// aborts on the first failed check.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cmath>
#include <condition_variable>
#include <cstdio>
#include <cstdlib>
#include <chrono>
#include <cstring>
#include <mutex>
#include <random>
#include <string>
#include <thread>
#include <vector>

#include "../../fairring_amd/csrc/ksum_kernels.h"
#include "../../fairring_amd/csrc/layout.h"
#include "../../include/fairring_hip.h"

namespace frg {
long long mixedLoadLaunches();  // of the stand-in for the kernels
}

// The default launch shapes, pinned: 48 MiB up to 2 contributions; 3 contributions
// 12.5 MiB with the kernel's own grid, 20 MiB from 100 MiB per contribution; from 4
// contributions on launches of whole rounds aimed at about 80 MB per launch.
static_assert(frg::defaultLaunchShape(2, 1ll << 30).bytes == 48ll << 20);
static_assert(frg::defaultLaunchShape(2, 1ll << 30).blocksPerCu == 6);
static_assert(frg::defaultLaunchShape(2, 1ll << 20).blocksPerCu == 0);
static_assert(!frg::defaultLaunchShape(2, 1ll << 30).wholeRounds);
static_assert(frg::defaultLaunchShape(3, 1ll << 30).bytes == 20ll << 20);
static_assert(frg::defaultLaunchShape(3, 1ll << 20).bytes == 13107200);
static_assert(!frg::defaultLaunchShape(3, 1ll << 30).wholeRounds);
static_assert(frg::defaultLaunchShape(8, 25ll << 20).bytes == 8ll << 20);
static_assert(frg::defaultLaunchShape(8, 25ll << 20).wholeRounds);
static_assert(frg::defaultLaunchShape(8, 100ll << 20).bytes == 8ll << 20);
static_assert(frg::defaultLaunchShape(8, 100ll << 20).blocksPerCu == 4);
static_assert(frg::defaultLaunchShape(4, 1ll << 30).bytes == 16ll << 20);
static_assert(frg::defaultLaunchShape(5, 1ll << 30).bytes == 12ll << 20);
static_assert(frg::defaultLaunchShape(7, 1ll << 30).bytes == 12ll << 20);
static_assert(frg::defaultLaunchShape(9, 1ll << 20).bytes == 8ll << 20);
static_assert(frg::defaultLaunchShape(12, 1ll << 30).bytes == 8ll << 20);
static_assert(frg::defaultLaunchShape(13, 1ll << 30).bytes == 4ll << 20);
static_assert(frg::defaultLaunchShape(16, 1ll << 30).bytes == 4ll << 20);
static_assert(frg::defaultLaunchShape(64, 1ll << 30).bytes == 4ll << 20);
static_assert(frg::defaultLaunchShape(64, 1ll << 30).wholeRounds);
// the compressed reduction: whole rounds of 2 MiB of wire, about 80 MB per launch; a bucket is one launch
static_assert(frg::defaultCompressedLaunchBytes(8, true, true, 1ll << 30) == 8ll << 20);
static_assert(frg::defaultCompressedLaunchBytes(8, true, true, 12ll << 20) == 16ll << 20);
static_assert(frg::defaultCompressedLaunchBytes(16, true, true, 1ll << 30) == 6ll << 20);
static_assert(frg::defaultCompressedLaunchBytes(32, true, true, 1ll << 30) == 4ll << 20);
static_assert(frg::defaultCompressedLaunchBytes(64, true, true, 1ll << 20) == 2ll << 20);
static_assert(frg::defaultCompressedLaunchBytes(2, true, true, 1ll << 30) == 16ll << 20);

#define CHECK(cond)                                                                  \
  do {                                                                               \
    if (!(cond)) {                                                                   \
      std::fprintf(stderr, "CHECK failed: %s (%s:%d) last error: %s\n", #cond, __FILE__, \
                   __LINE__, frg_last_error());                                      \
      std::abort();                                                                  \
    }                                                                                \
  } while (0)

namespace {

using Vec = std::vector<float>;

std::vector<Vec> randomContribs(int k, int64_t n, unsigned seed) {
  std::mt19937 rng(seed);
  std::normal_distribution<float> d(0.f, 0.01f);
  std::vector<Vec> v(k, Vec(static_cast<size_t>(n)));
  for (auto& c : v) {
    for (auto& x : c) x = d(rng);
  }
  return v;
}

Vec fold(const std::vector<Vec>& c, int scaleMode, float scale, const Vec* carry = nullptr) {
  Vec out(c[0].size());
  for (size_t i = 0; i < out.size(); ++i) {
    auto term = [&](size_t kk) {
      const float x = c[kk][i];
      return scaleMode == FRG_SCALE_PRE_MUL ? x * scale
                                            : (scaleMode == FRG_SCALE_PRE_DIV ? x / scale : x);
    };
    size_t k = 0;
    float acc = carry ? (*carry)[i] : term(k++);
    for (; k < c.size(); ++k) acc = acc + term(k);
    if (scaleMode == FRG_SCALE_MUL) acc = acc * scale;
    if (scaleMode == FRG_SCALE_DIV) acc = acc / scale;
    out[i] = acc;
  }
  return out;
}

bool same(const Vec& a, const Vec& b) {
  return a.size() == b.size() && std::memcmp(a.data(), b.data(), a.size() * 4) == 0;
}

std::vector<const void*> table(const std::vector<Vec>& c) {
  std::vector<const void*> t;
  for (auto& v : c) t.push_back(v.data());
  return t;
}

frg_ctx* makeCtx(int64_t total, int64_t slice, int streams, int64_t launchBytes) {
  frg_options o = {};
  o.max_memory_allocated_in_bytes = total;
  o.slice_size_in_bytes = slice;
  o.num_reduce_streams = streams;
  o.max_launch_bytes = launchBytes;
  frg_ctx* ctx = nullptr;
  CHECK(frg_create(0, &o, &ctx) == FRG_OK);
  return ctx;
}

void scenarioResident() {
  std::puts("resident: slicing, launch splitting, stream rotation");
  for (int streams : {1, 2, 3}) {
    for (int64_t launch : {int64_t(-1), int64_t(1024), int64_t(4096)}) {
      // a chain scratch of one tile (two for three streams, the default for one):
      // the chains below then walk it in several pieces
      if (streams == 1) {
        unsetenv("FAIRRING_CHAIN_SCRATCH_BYTES");
      } else {
        setenv("FAIRRING_CHAIN_SCRATCH_BYTES", streams == 2 ? "4096" : "8192", 1);
      }
      frg_ctx* ctx = makeCtx(16384, 4096, streams, launch);
      unsetenv("FAIRRING_CHAIN_SCRATCH_BYTES");
      auto c = randomContribs(8, 10007, 1);
      Vec out(10007);
      frg_work* w = nullptr;
      auto t = table(c);
      CHECK(frg_allreduce(ctx, out.data(), t.data(), 8, 10007, FRG_F32, FRG_SUM, FRG_SCALE_MUL,
                          0.125f, nullptr, nullptr, nullptr, &w) == FRG_OK);
      CHECK(frg_work_wait(w) == FRG_OK);
      CHECK(frg_work_is_completed(w) == FRG_OK);
      CHECK(same(out, fold(c, FRG_SCALE_MUL, 0.125f)));
      frg_work_release(w);
      // more contributions than one launch takes: chained with carry
      auto big = randomContribs(150, 3001, 2);
      Vec out2(3001);
      auto t2 = table(big);
      CHECK(frg_allreduce(ctx, out2.data(), t2.data(), 150, 3001, FRG_F32, FRG_SUM, FRG_SCALE_DIV,
                          150.f, nullptr, nullptr, nullptr, &w) == FRG_OK);
      CHECK(frg_work_wait(w) == FRG_OK);
      CHECK(same(out2, fold(big, FRG_SCALE_DIV, 150.f)));
      frg_work_release(w);
      // the same reduced in place into contribution 100, which only the second
      // launch of the chain reads: the partial result must not land there early
      Vec want = fold(big, FRG_SCALE_DIV, 150.f);
      CHECK(frg_allreduce(ctx, big[100].data(), t2.data(), 150, 3001, FRG_F32, FRG_SUM,
                          FRG_SCALE_DIV, 150.f, nullptr, nullptr, nullptr, &w) == FRG_OK);
      CHECK(frg_work_wait(w) == FRG_OK);
      CHECK(same(big[100], want));
      frg_work_release(w);
      CHECK(frg_destroy(ctx) == FRG_OK);
    }
  }
}

float widenBf16(uint16_t b) {
  const uint32_t u = static_cast<uint32_t>(b) << 16;
  float f;
  std::memcpy(&f, &u, 4);
  return f;
}

uint16_t narrowBf16(float f) {
  uint32_t u;
  std::memcpy(&u, &f, 4);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0;
  return static_cast<uint16_t>((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}

void scenarioPreScaleAndCompressed() {
  std::puts("pre-scaled chains and the compressed reduction: offsets per element size");
  frg_ctx* ctx = makeCtx(16384, 4096, 2, 1024);
  frg_work* w = nullptr;
  // a pre-scale goes on every launch of a chain, never on the carried term
  auto big = randomContribs(150, 3001, 21);
  Vec out(3001);
  auto t = table(big);
  CHECK(frg_allreduce(ctx, out.data(), t.data(), 150, 3001, FRG_F32, FRG_SUM, FRG_SCALE_PRE_DIV,
                      150.f, nullptr, nullptr, nullptr, &w) == FRG_OK);
  CHECK(frg_work_wait(w) == FRG_OK);
  CHECK(same(out, fold(big, FRG_SCALE_PRE_DIV, 150.f)));
  frg_work_release(w);
  CHECK(frg_allreduce_host(ctx, out.data(), t.data(), 3, 3001, FRG_F32, FRG_SUM,
                           FRG_SCALE_PRE_MUL, .5f, 0, nullptr, nullptr, nullptr,
                           nullptr) == FRG_ERR_UNSUPPORTED);
  // compressed: 5 contributions, the raw fp32 one third in the chain, reduced in place into it;
  // slices are 2048 wire elements, so the fp32 side advances by 8 KiB per slice
  const int64_t n = 10007;
  const int K = 5, rawIndex = 2;
  auto raw = randomContribs(1, n, 22)[0];
  std::vector<std::vector<uint16_t>> peers(K, std::vector<uint16_t>(static_cast<size_t>(n)));
  auto src = randomContribs(K, n, 23);
  for (int k = 0; k < K; ++k) {
    for (int64_t i = 0; i < n; ++i) peers[k][i] = narrowBf16(src[k][i]);
  }
  Vec want(static_cast<size_t>(n));
  for (int64_t i = 0; i < n; ++i) {
    float acc = 0.f;
    for (int k = 0; k < K; ++k) {
      float term = k == rawIndex ? widenBf16(narrowBf16(widenBf16(narrowBf16(raw[i])) * 0.2f))
                                 : widenBf16(peers[k][i]);
      acc = k == 0 ? term : acc + term;
    }
    want[i] = widenBf16(narrowBf16(acc));
  }
  std::vector<const void*> tab;
  for (int k = 0; k < K; ++k) tab.push_back(k == rawIndex ? (const void*)raw.data() : peers[k].data());
  CHECK(frg_allreduce_compressed(ctx, raw.data(), FRG_F32, tab.data(), K, rawIndex, n, FRG_BF16,
                                 FRG_SCALE_MUL, 0.2f, nullptr, nullptr, nullptr, &w) == FRG_OK);
  CHECK(frg_work_wait(w) == FRG_OK);
  CHECK(same(raw, want));
  frg_work_release(w);
  // the same with the raw contribution in four tensors of its own (one of them empty, one of
  // a single element), into a separate bucket: a launch per tensor, same result
  {
    const Vec rawAgain = randomContribs(1, n, 22)[0];
    const int64_t cuts[6] = {0, 4096, 4096, 4097, 9000, n};
    std::vector<Vec> tensors;
    std::vector<frg_segment> segs;
    for (int i = 0; i < 5; ++i) {
      tensors.emplace_back(rawAgain.begin() + cuts[i], rawAgain.begin() + cuts[i + 1]);
    }
    for (const Vec& v : tensors) segs.push_back(frg_segment{v.data(), static_cast<int64_t>(v.size())});
    Vec bucket(static_cast<size_t>(n), -3.f);
    std::vector<const void*> gtab = tab;
    gtab[rawIndex] = nullptr;  // ignored
    frg_progress before = {};
    CHECK(frg_get_progress(ctx, &before) == FRG_OK);
    CHECK(frg_allreduce_compressed_gathered(ctx, bucket.data(), FRG_F32, gtab.data(), K, rawIndex,
                                            segs.data(), 5, n, FRG_BF16, FRG_SCALE_MUL, 0.2f,
                                            nullptr, nullptr, nullptr, &w) == FRG_OK);
    CHECK(frg_work_wait(w) == FRG_OK);
    CHECK(same(bucket, want));
    frg_work_release(w);
    frg_progress after = {};
    CHECK(frg_get_progress(ctx, &after) == FRG_OK);
    // a tensor that starts within a lane's group of 8 elements: tensor by tensor, one launch
    // for each that holds anything
    CHECK(after.launches - before.launches == 4);
    // tensors that start where groups of 8 do (and on 16-byte boundaries): one launch reads
    // all of them through its table
    {
      const int64_t even[5] = {0, 4096, 4104, 9000, n};
      std::vector<Vec> parts;
      std::vector<frg_segment> esegs;
      for (int i = 0; i < 4; ++i) parts.emplace_back(rawAgain.begin() + even[i], rawAgain.begin() + even[i + 1]);
      bool aligned = reinterpret_cast<uintptr_t>(bucket.data()) % 16 == 0;
      for (const Vec& v : parts) {
        esegs.push_back(frg_segment{v.data(), static_cast<int64_t>(v.size())});
        aligned = aligned && reinterpret_cast<uintptr_t>(v.data()) % 16 == 0;
      }
      std::fill(bucket.begin(), bucket.end(), -3.f);
      CHECK(frg_allreduce_compressed_gathered(ctx, bucket.data(), FRG_F32, gtab.data(), K, rawIndex,
                                              esegs.data(), 4, n, FRG_BF16, FRG_SCALE_MUL, 0.2f,
                                              nullptr, nullptr, nullptr, &w) == FRG_OK);
      CHECK(frg_work_wait(w) == FRG_OK);
      CHECK(same(bucket, want));
      frg_work_release(w);
      frg_progress last = {};
      CHECK(frg_get_progress(ctx, &last) == FRG_OK);
      if (aligned) CHECK(last.launches - after.launches == 1);
    }
    // the piecewise contribution is the raw one, and its lengths must add up
    CHECK(frg_allreduce_compressed_gathered(ctx, bucket.data(), FRG_F32, gtab.data(), K, -1,
                                            segs.data(), 5, n, FRG_BF16, 0, 1.f, nullptr, nullptr,
                                            nullptr, nullptr) == FRG_ERR_INVALID);
    CHECK(frg_allreduce_compressed_gathered(ctx, bucket.data(), FRG_F32, gtab.data(), K, rawIndex,
                                            segs.data(), 4, n, FRG_BF16, 0, 1.f, nullptr, nullptr,
                                            nullptr, nullptr) == FRG_ERR_INVALID);
  }
  // under graph capture the pipeline refuses (the one-launch entry points are the ones to capture)
  fake_hip_set_capturing(1);
  CHECK(frg_allreduce(ctx, out.data(), t.data(), 3, 3001, FRG_F32, FRG_SUM, FRG_SCALE_NONE, 1.f,
                      nullptr, nullptr, nullptr, nullptr) == FRG_ERR_UNSUPPORTED);
  CHECK(std::strstr(frg_last_error(), "captured") != nullptr);
  CHECK(frg_allreduce_compressed(ctx, raw.data(), FRG_F32, tab.data(), K, rawIndex, n, FRG_BF16,
                                 FRG_SCALE_MUL, 0.2f, nullptr, nullptr, nullptr,
                                 nullptr) == FRG_ERR_UNSUPPORTED);
  fake_hip_set_capturing(0);
  // contract violations of the compressed entry point
  CHECK(frg_allreduce_compressed(ctx, raw.data(), FRG_F32, tab.data(), K, 7, n, FRG_BF16, 0, 1.f,
                                 nullptr, nullptr, nullptr, nullptr) == FRG_ERR_INVALID);
  CHECK(frg_allreduce_compressed(ctx, raw.data(), FRG_F32, tab.data(), K, rawIndex, n, FRG_F32, 0,
                                 1.f, nullptr, nullptr, nullptr, nullptr) == FRG_ERR_UNSUPPORTED);
  CHECK(frg_allreduce_compressed(ctx, raw.data(), FRG_F64, tab.data(), K, rawIndex, n, FRG_BF16, 0,
                                 1.f, nullptr, nullptr, nullptr, nullptr) == FRG_ERR_UNSUPPORTED);
  CHECK(frg_allreduce_compressed(ctx, raw.data(), FRG_F32, tab.data(), K, rawIndex, n, FRG_BF16,
                                 FRG_SCALE_PRE_MUL, 1.f, nullptr, nullptr, nullptr,
                                 nullptr) == FRG_ERR_INVALID);
  CHECK(frg_destroy(ctx) == FRG_OK);
}

int64_t launchesSoFar(frg_ctx* ctx) {
  frg_progress p = {};
  CHECK(frg_get_progress(ctx, &p) == FRG_OK);
  return p.launches;
}

void scenarioWholeRoundPlan() {
  std::puts("aligned launch plan: whole rounds placed on the output's multiples of a round");
  const int64_t MiB = 1 << 20;
  auto sizes = [](const std::vector<frg::LaunchPart>& v) {
    std::vector<std::vector<int64_t>> out;
    for (auto& p : v) out.push_back({p.bytes, p.blocksPerCu, p.leadBytes});
    return out;
  };
  using P = std::vector<std::vector<int64_t>>;
  // 256 CUs: a round of the 4-blocks-per-CU grid is 4 MiB
  CHECK(frg::alignedRoundBytes(256) == 4 * MiB);
  // a bucket on a multiple of a round: 2 + 2 + 2 rounds, 1 MiB left to the last launch
  CHECK(sizes(frg::planAlignedLaunches(25 * MiB, 0, 8 * MiB, 256)) ==
        (P{{8 * MiB, 4, 0}, {8 * MiB, 4, -1}, {9 * MiB, 4, -1}}));
  CHECK(sizes(frg::planAlignedLaunches(24 * MiB, 0, 8 * MiB, 256)) ==
        (P{{8 * MiB, 4, 0}, {8 * MiB, 4, -1}, {8 * MiB, 4, -1}}));
  // 1 MiB past a multiple: 3 MiB ahead of the first round go to the first launch, five
  // whole rounds follow (2 + 3), 2 MiB behind them go to the last
  CHECK(sizes(frg::planAlignedLaunches(25 * MiB, 3 * MiB, 8 * MiB, 256)) ==
        (P{{11 * MiB, 4, 3 * MiB}, {14 * MiB, 4, -1}}));
  // an odd round goes to the last launch; a lead of less than a tile is like any other
  CHECK(sizes(frg::planAlignedLaunches(28 * MiB + 1536 + 100, 1536, 8 * MiB, 256)) ==
        (P{{8 * MiB + 1536, 4, 1536}, {8 * MiB, 4, -1}, {12 * MiB + 100, 4, -1}}));
  // fewer than two whole rounds: one launch, everything left to the kernel
  CHECK(sizes(frg::planAlignedLaunches(7 * MiB, 0, 8 * MiB, 256)) == (P{{7 * MiB, 0, -1}}));
  CHECK(sizes(frg::planAlignedLaunches(10 * MiB, 3 * MiB, 8 * MiB, 256)) == (P{{10 * MiB, 0, -1}}));
  CHECK(sizes(frg::planAlignedLaunches(0, 0, 8 * MiB, 256)) == (P{{0, 0, -1}}));
  CHECK(sizes(frg::planAlignedLaunches(100, 3000, 8 * MiB, 256)) == (P{{100, 0, -1}}));
  CHECK(sizes(frg::planAlignedLaunches(8 * MiB, 0, 8 * MiB, 256)) == (P{{8 * MiB, 4, 0}}));
  // more contributions aim at one round per launch; few at four
  CHECK(frg::planAlignedLaunches(25 * MiB, 0, 4 * MiB, 256).size() == 6);
  CHECK(sizes(frg::planAlignedLaunches(41 * MiB, 0, 16 * MiB, 256)) ==
        (P{{20 * MiB, 4, 0}, {21 * MiB, 4, -1}}));  // ten rounds as 5 + 5, 1 MiB left over
  // every size: the parts add up, every launch but the last is whole rounds past its lead
  for (int64_t lead : {int64_t(0), int64_t(1536), 3 * MiB + 512}) {
    for (int64_t m = 1; m <= 70; ++m) {
      const int64_t bytes = m * MiB + 12345 * 16;
      const auto plan = frg::planAlignedLaunches(bytes, lead, 8 * MiB, 256);
      int64_t sum = 0;
      for (size_t i = 0; i < plan.size(); ++i) {
        sum += plan[i].bytes;
        if (plan.size() > 1 && i + 1 < plan.size()) {
          CHECK((plan[i].bytes - (i == 0 ? lead : 0)) % (4 * MiB) == 0);
        }
      }
      CHECK(sum == bytes);
    }
  }
  // a whole gradient: 8 MiB launches throughout
  const auto big = frg::planAlignedLaunches(5480000000ll, 0, 8 * MiB, 256);
  int64_t sum = 0;
  for (auto& p : big) sum += p.bytes;
  CHECK(sum == 5480000000ll && big.size() == 653);
  CHECK(big.front().bytes == 8 * MiB && big[big.size() / 2].bytes == 8 * MiB);
  // where the rounds start: at the output's next multiple of a round within its
  // allocation, on the 4 KiB grid of the first contribution
  CHECK(frg::alignedLeadBytes(0, 0x7f0000000000ull, 256) == 0);
  CHECK(frg::alignedLeadBytes(1 * MiB, 0x7f0000100000ull, 256) == 3 * MiB);
  CHECK(frg::alignedLeadBytes(4 * MiB - 1536, 0x7f0000000a00ull, 256) == 1536);
  CHECK(frg::alignedLeadBytes(2 * MiB + 2560, 0x7f0000000a00ull, 256) == 2 * MiB - 2560);
  // the output 512 bytes off the first contribution's 4 KiB grid: the tile grid wins
  CHECK(frg::alignedLeadBytes(1 * MiB + 512, 0x7f0000100000ull, 256) == 3 * MiB - 4096);
  // through the ABI, in elements
  int64_t elems[8];
  int32_t bpc[8];
  int n = 0;
  CHECK(frg_plan_launches(8, 6553600, 4, 0, 0, 1, 256, elems, bpc, 8, &n) == FRG_OK);
  CHECK(n == 3 && elems[0] == 2097152 && elems[1] == 2097152 && elems[2] == 2359296);
  CHECK(bpc[0] == 4 && bpc[2] == 4);
  // a short operation is not aligned unless the caller says that its neighbours are too
  CHECK(frg_plan_launches(8, 6553600, 4, 0, 0, 0, 256, elems, bpc, 8, &n) == FRG_OK);
  CHECK(n == 2 && elems[0] == 3276800 && bpc[0] == 0);
  // 3 MiB short of a multiple, 5 whole rounds: aligning does not pay, two equal launches
  CHECK(frg_plan_launches(8, 6553600, 4, 0x7f0000100000ull, 1 * MiB, 1, 256, elems, bpc, 8,
                          &n) == FRG_OK);
  CHECK(n == 2 && elems[0] == 3276800 && elems[1] == 3276800 && bpc[0] == 0);
  // 1 MiB short of one: it does (the first launch takes that MiB ahead of its rounds)
  CHECK(frg_plan_launches(8, 6553600, 4, 0x7f0000300000ull, 3 * MiB, 1, 256, elems, bpc, 8,
                          &n) == FRG_OK);
  CHECK(n == 3 && elems[0] == 9 * MiB / 4 && elems[1] == 2 * MiB && elems[2] == 2 * MiB);
  // a large operation is aligned wherever it starts
  CHECK(frg_plan_launches(8, 100 << 20, 4, 0x7f0000200000ull, 2 * MiB, 0, 256, elems, bpc, 8,
                          &n) == FRG_OK);
  CHECK(n == 49 && elems[0] == 10 * MiB / 4 && elems[1] == 2 * MiB && bpc[0] == 4);
  // more than 8 contributions far from a multiple: whole rounds from the start
  CHECK(frg_plan_launches(16, 6553600, 4, 0x7f0000200000ull, 2 * MiB, 1, 256, elems, bpc, 8,
                          &n) == FRG_OK);
  CHECK(n == 6 && elems[0] == 1 * MiB && bpc[0] == 4);
  CHECK(frg_plan_launches(2, 100 << 20, 4, 0, 0, 0, 256, elems, bpc, 8, &n) == FRG_OK);  // 400 MiB
  CHECK(n == 8 && elems[0] == 12582912 && bpc[0] == 6);
  CHECK(frg_plan_launches(0, 10, 4, 0, 0, 0, 256, elems, bpc, 8, &n) == FRG_ERR_INVALID);
}

void scenarioLaunchPartition() {
  std::puts("launch partition: sizes cut from the tensor on tile boundaries, 1.5x rule, per slice");
  struct Case {
    int64_t launchBytes, sliceBytes, numel;
    int64_t wantLaunches;
  };
  // 16 KiB launches = 4096 fp32 elements each (a multiple of the 1024-element tile)
  const Case cases[] = {
      {16384, 4096, 4096, 1},          // exactly one launch
      {16384, 4096, 6144, 1},          // 1.5 x the launch size: still one
      {16384, 4096, 6145, 2},          // a little more: 4096 + 2049
      {16384, 4096, 40960 + 100, 10},  // nine of 4096, the last takes 4096 + 100
      {16384, 65536, 40960 + 100, 10},  // the slice size does not matter
      {-1, 4096, 10000, 10},           // one launch per slice: ceil(10000 / 1024)
      {-1, 65536, 10000, 1},
      {6000, 65536, 10000, 10},        // 1496 elements round down to one 1024-element tile: 9 + a rest of 784
  };
  for (const Case& cs : cases) {
    frg_ctx* ctx = makeCtx(2 * cs.sliceBytes, cs.sliceBytes, 2, cs.launchBytes);
    auto c = randomContribs(3, cs.numel, 5);
    Vec out(static_cast<size_t>(cs.numel));
    auto t = table(c);
    frg_work* w = nullptr;
    const int64_t before = launchesSoFar(ctx);
    CHECK(frg_allreduce(ctx, out.data(), t.data(), 3, cs.numel, FRG_F32, FRG_SUM, FRG_SCALE_NONE,
                        1.f, nullptr, nullptr, nullptr, &w) == FRG_OK);
    CHECK(frg_work_wait(w) == FRG_OK);
    CHECK(same(out, fold(c, FRG_SCALE_NONE, 1.f)));
    const int64_t got = launchesSoFar(ctx) - before;
    if (got != cs.wantLaunches) {
      std::fprintf(stderr, "launch bytes %lld, slice %lld, numel %lld: %lld launches, expected %lld\n",
                   (long long)cs.launchBytes, (long long)cs.sliceBytes, (long long)cs.numel,
                   (long long)got, (long long)cs.wantLaunches);
      std::abort();
    }
    frg_work_release(w);
    CHECK(frg_destroy(ctx) == FRG_OK);
  }
}

void scenarioBusyProducer() {
  std::puts("many operations submitted while the producer stream is busy");
  frg_ctx* ctx = makeCtx(2 * 65536, 65536, 2, 32768);
  const int ops = 211;
  std::vector<std::vector<Vec>> inputs;
  std::vector<Vec> outs(ops);
  std::vector<frg_work*> works(ops);
  fake_hip_occupy(nullptr, 100);  // the default stream is busy for a while
  for (int i = 0; i < ops; ++i) {
    const int64_t n = 1000 + 37 * i;
    inputs.push_back(randomContribs(8, n, 100 + i));
    outs[i].assign(static_cast<size_t>(n), -1.f);
    auto t = table(inputs.back());
    CHECK(frg_allreduce(ctx, outs[i].data(), t.data(), 8, n, FRG_F32, FRG_SUM, FRG_SCALE_MUL,
                        0.125f, /*producer=*/nullptr, nullptr, nullptr, &works[i]) == FRG_OK);
  }
  for (int i = 0; i < ops; ++i) {
    CHECK(frg_work_wait(works[i]) == FRG_OK);
    CHECK(same(outs[i], fold(inputs[i], FRG_SCALE_MUL, 0.125f)));
    frg_work_release(works[i]);
  }
  CHECK(frg_synchronize(ctx) == FRG_OK);
  CHECK(frg_destroy(ctx) == FRG_OK);
}

void scenarioWaitGivesUp() {
  std::puts("a wait with a time limit gives up with a report, and can be repeated");
  frg_ctx* ctx = makeCtx(16384, 4096, 2, 1024);
  auto c = randomContribs(4, 5000, 77);
  Vec out(5000);
  auto t = table(c);
  frg_work* w = nullptr;
  CHECK(frg_set_wait_timeout(0.2) == FRG_OK);
  fake_hip_occupy(nullptr, 1500);  // the producer's stream is busy for a while
  CHECK(frg_allreduce(ctx, out.data(), t.data(), 4, 5000, FRG_F32, FRG_SUM, FRG_SCALE_NONE, 1.f,
                      /*producer=*/nullptr, nullptr, nullptr, &w) == FRG_OK);
  CHECK(frg_work_wait(w) == FRG_ERR_NOT_READY);
  CHECK(std::strstr(frg_last_error(), "gave up after") != nullptr);
  CHECK(std::strstr(frg_last_error(), "submitted") != nullptr);
  CHECK(frg_set_wait_timeout(0) == FRG_OK);
  CHECK(frg_work_wait(w) == FRG_OK);
  CHECK(same(out, fold(c, FRG_SCALE_NONE, 1.f)));
  frg_work_release(w);
  CHECK(frg_destroy(ctx) == FRG_OK);
}

void scenarioIdleProducer() {
  std::puts("no event is recorded on a producer stream that has drained");
  frg_ctx* ctx = makeCtx(8192, 4096, 2, 1024);
  auto c = randomContribs(3, 3000, 31);
  Vec out(3000);
  auto t = table(c);
  frg_work* w = nullptr;
  CHECK(hipStreamSynchronize(nullptr) == hipSuccess);
  long records = fake_hip_calls("hipEventRecord");
  CHECK(frg_allreduce(ctx, out.data(), t.data(), 3, 3000, FRG_F32, FRG_SUM, FRG_SCALE_NONE, 1.f,
                      nullptr, nullptr, nullptr, &w) == FRG_OK);
  CHECK(frg_work_wait(w) == FRG_OK);
  CHECK(same(out, fold(c, FRG_SCALE_NONE, 1.f)));
  CHECK(fake_hip_calls("hipEventRecord") == records);
  frg_work_release(w);
  fake_hip_occupy(nullptr, 30);  // busy: the event is recorded and waited for
  records = fake_hip_calls("hipEventRecord");
  CHECK(frg_allreduce(ctx, out.data(), t.data(), 3, 3000, FRG_F32, FRG_SUM, FRG_SCALE_NONE, 1.f,
                      nullptr, nullptr, nullptr, &w) == FRG_OK);
  CHECK(fake_hip_calls("hipEventRecord") >= records + 1);
  CHECK(frg_work_wait(w) == FRG_OK);
  CHECK(fake_hip_calls("hipEventRecord") == records + 1);
  frg_work_release(w);
  // a busy answer is dear: the next 15 operations from that stream record
  // without asking, whatever the stream does meanwhile; then it is asked again
  CHECK(hipStreamSynchronize(nullptr) == hipSuccess);
  for (int i = 0; i < 16; ++i) {
    records = fake_hip_calls("hipEventRecord");
    CHECK(frg_allreduce(ctx, out.data(), t.data(), 3, 3000, FRG_F32, FRG_SUM, FRG_SCALE_NONE, 1.f,
                        nullptr, nullptr, nullptr, &w) == FRG_OK);
    CHECK(frg_work_wait(w) == FRG_OK);
    CHECK(same(out, fold(c, FRG_SCALE_NONE, 1.f)));
    CHECK(fake_hip_calls("hipEventRecord") == records + (i < 15 ? 1 : 0));
    frg_work_release(w);
  }
  CHECK(frg_destroy(ctx) == FRG_OK);
}

std::vector<hipStream_t> streamsOf(frg_ctx* ctx);

// What the completion callback of the scenario below notes down.
struct InlineNote {
  std::thread::id thread;
  void* stream = nullptr;
  int status = -1;
  int calls = 0;
};
void noteDone(void* user, int status, void* lastStream) {
  auto* n = static_cast<InlineNote*>(user);
  n->thread = std::this_thread::get_id();
  n->stream = lastStream;
  n->status = status;
  n->calls += 1;
}

void scenarioSmallOperationsOnTheCallersStream() {
  std::puts("a small operation with nothing in flight runs on the caller's stream");
  setenv("FAIRRING_INLINE_BYTES", "65536", 1);
  frg_ctx* ctx = makeCtx(8192, 4096, 2, 0);
  setenv("FAIRRING_INLINE_BYTES", "0", 1);
  hipStream_t p, q;
  CHECK(hipStreamCreateWithFlags(&p, hipStreamNonBlocking) == hipSuccess);
  CHECK(hipStreamCreateWithFlags(&q, hipStreamNonBlocking) == hipSuccess);
  const int64_t n = 3000;           // 4 x 12,000 B moved: small
  const int64_t big = 20000;        // 4 x 80,000 B: through the pipeline
  auto c = randomContribs(3, big, 70);
  auto t = table(c);
  const long waits = fake_hip_calls("hipStreamWaitEvent");

  // 1. launched by the call itself: the callback has run when it returns, on
  // this thread, naming the caller's stream; no stream waits for another
  {
    Vec out(n, -1.f);
    InlineNote note;
    frg_work* w = nullptr;
    fake_hip_occupy(p, 40);  // the producer is busy: the operation queues up behind it
    CHECK(frg_allreduce(ctx, out.data(), t.data(), 3, n, FRG_F32, FRG_SUM, FRG_SCALE_MUL, 0.5f, p,
                        &noteDone, &note, &w) == FRG_OK);
    CHECK(note.calls == 1 && note.status == FRG_OK && note.stream == p);
    CHECK(note.thread == std::this_thread::get_id());
    CHECK(frg_work_is_completed(w) == FRG_OK);
    CHECK(fake_hip_calls("hipStreamWaitEvent") == waits);
    frg_progress2 pr = {};
    CHECK(frg_get_progress2(ctx, &pr, sizeof(pr)) == FRG_OK);
    CHECK(pr.submitted == 1 && pr.started == 1 && pr.enqueued == 1 && pr.launches == 1);
    // frg_synchronize covers it, without the caller touching its stream
    CHECK(frg_synchronize(ctx) == FRG_OK);
    std::vector<Vec> head = {Vec(c[0].begin(), c[0].begin() + n), Vec(c[1].begin(), c[1].begin() + n),
                             Vec(c[2].begin(), c[2].begin() + n)};
    CHECK(same(out, fold(head, FRG_SCALE_MUL, 0.5f)));
    CHECK(frg_work_wait(w) == FRG_OK);
    frg_work_release(w);
  }

  // 2. its output read by a large operation that comes from another stream
  // while it is still queued behind its producer: that one waits for it
  {
    Vec mid(big, -1.f), out(big, -1.f);
    InlineNote first, second;
    frg_work *w0 = nullptr, *w1 = nullptr;
    fake_hip_occupy(p, 60);
    CHECK(frg_allreduce(ctx, mid.data(), t.data(), 3, n, FRG_F32, FRG_SUM, FRG_SCALE_NONE, 1.f, p,
                        &noteDone, &first, &w0) == FRG_OK);
    CHECK(first.calls == 1 && first.thread == std::this_thread::get_id());
    const void* tab[2] = {mid.data(), c[1].data()};
    CHECK(frg_allreduce(ctx, out.data(), tab, 2, big, FRG_F32, FRG_SUM, FRG_SCALE_NONE, 1.f, q,
                        &noteDone, &second, &w1) == FRG_OK);
    CHECK(frg_work_wait(w1) == FRG_OK);
    CHECK(frg_synchronize(ctx) == FRG_OK);  // the callback follows the mark the wait sees
    CHECK(second.calls == 1 && second.thread != std::this_thread::get_id());
    for (int64_t i = 0; i < n; ++i) {
      CHECK(out[i] == (c[0][i] + c[1][i] + c[2][i]) + c[1][i]);
    }
    frg_work_release(w0);
    frg_work_release(w1);
    CHECK(frg_synchronize(ctx) == FRG_OK);
  }

  // 3. two small in-place operations on one tensor from two streams, the first
  // stream held up: the second follows the first
  {
    Vec own(c[0].begin(), c[0].begin() + n);
    const void* tab[3] = {own.data(), c[1].data(), c[2].data()};
    std::vector<Vec> terms = {own, Vec(c[1].begin(), c[1].begin() + n),
                              Vec(c[2].begin(), c[2].begin() + n)};
    Vec want = fold(terms, FRG_SCALE_MUL, 0.5f);
    terms[0] = want;
    want = fold(terms, FRG_SCALE_MUL, 0.25f);
    frg_work *w0 = nullptr, *w1 = nullptr;
    fake_hip_occupy(p, 60);
    CHECK(frg_allreduce(ctx, own.data(), tab, 3, n, FRG_F32, FRG_SUM, FRG_SCALE_MUL, 0.5f, p,
                        nullptr, nullptr, &w0) == FRG_OK);
    // the reduce streams were found idle for the first and nothing has gone to them since:
    // the second does not ask again
    const long asked = fake_hip_calls("hipStreamQuery");
    CHECK(frg_allreduce(ctx, own.data(), tab, 3, n, FRG_F32, FRG_SUM, FRG_SCALE_MUL, 0.25f, q,
                        nullptr, nullptr, &w1) == FRG_OK);
    CHECK(fake_hip_calls("hipStreamQuery") == asked);
    CHECK(frg_work_wait(w1) == FRG_OK);
    CHECK(same(own, want));
    frg_work_release(w0);
    frg_work_release(w1);
    CHECK(frg_synchronize(ctx) == FRG_OK);
  }

  // 4. with a reduce stream still at work the small operation takes the
  // pipeline (and its place in the order of what shares its memory)
  {
    Vec mid(big, -1.f), out(n, -1.f);
    InlineNote note;
    frg_work *w0 = nullptr, *w1 = nullptr;
    fake_hip_occupy(streamsOf(ctx)[0], 40);
    fake_hip_occupy(streamsOf(ctx)[1], 40);
    CHECK(frg_allreduce(ctx, mid.data(), t.data(), 3, big, FRG_F32, FRG_SUM, FRG_SCALE_NONE, 1.f,
                        p, nullptr, nullptr, &w0) == FRG_OK);
    const void* tab[2] = {mid.data(), c[2].data()};
    CHECK(frg_allreduce(ctx, out.data(), tab, 2, n, FRG_F32, FRG_SUM, FRG_SCALE_NONE, 1.f, q,
                        &noteDone, &note, &w1) == FRG_OK);
    CHECK(frg_work_wait(w1) == FRG_OK);
    CHECK(frg_synchronize(ctx) == FRG_OK);
    CHECK(note.calls == 1 && note.thread != std::this_thread::get_id());
    for (int64_t i = 0; i < n; ++i) {
      CHECK(out[i] == (c[0][i] + c[1][i] + c[2][i]) + c[2][i]);
    }
    frg_work_release(w0);
    frg_work_release(w1);
  }

  // 5. a failure found by the launch is the work's status, as on the command thread
  {
    Vec out(n, -1.f);
    InlineNote note;
    frg_work* w = nullptr;
    CHECK(frg_synchronize(ctx) == FRG_OK);
    // (this build's stand-in for the kernel reduces fp32 only and says so at the launch)
    CHECK(frg_allreduce(ctx, out.data(), t.data(), 3, n / 2, FRG_I32, FRG_SUM, FRG_SCALE_NONE, 1.f,
                        p, &noteDone, &note, &w) == FRG_OK);
    CHECK(note.calls == 1 && note.status == FRG_ERR_UNSUPPORTED);
    CHECK(note.thread == std::this_thread::get_id());
    CHECK(frg_work_wait(w) == FRG_ERR_UNSUPPORTED);
    frg_work_release(w);
    frg_progress2 pr = {};
    CHECK(frg_get_progress2(ctx, &pr, sizeof(pr)) == FRG_OK);
    CHECK(pr.submitted == pr.enqueued && pr.submitted == pr.started);
  }
  CHECK(frg_destroy(ctx) == FRG_OK);
  CHECK(hipStreamDestroy(p) == hipSuccess);
  CHECK(hipStreamDestroy(q) == hipSuccess);
}

void scenarioNullStreamRemembersItsWaits() {
  std::puts("the null stream is told once per reduce stream to wait, not once per operation");
  frg_ctx* ctx = makeCtx(8192, 4096, 2, 0);
  const int64_t n = 3000;
  const int ops = 12;
  std::vector<std::vector<Vec>> c;
  std::vector<Vec> outs(ops, Vec(n, -1.f));
  std::vector<frg_work*> w(ops, nullptr);
  hipStream_t producer;
  CHECK(hipStreamCreateWithFlags(&producer, hipStreamNonBlocking) == hipSuccess);
  fake_hip_occupy(streamsOf(ctx)[0], 40);  // the operations are still queued when they are waited for
  fake_hip_occupy(streamsOf(ctx)[1], 40);
  for (int i = 0; i < ops; ++i) {
    c.push_back(randomContribs(3, n, 80 + i));
    auto t = table(c.back());
    CHECK(frg_allreduce(ctx, outs[i].data(), t.data(), 3, n, FRG_F32, FRG_SUM, FRG_SCALE_NONE, 1.f,
                        producer, nullptr, nullptr, &w[i]) == FRG_OK);
  }
  // (once the command thread has dealt with all of them: an event covers what its stream holds)
  while (frg_work_is_completed(w[ops - 1]) != FRG_OK) std::this_thread::yield();
  const long waits = fake_hip_calls("hipStreamWaitEvent");
  for (int i = 0; i < ops; ++i) CHECK(frg_work_block_stream(w[i], nullptr) == FRG_OK);
  // the first wait on each reduce stream covers the operations behind it too
  const long told = fake_hip_calls("hipStreamWaitEvent") - waits;
  CHECK(told >= 1 && told <= 2);
  CHECK(hipStreamSynchronize(nullptr) == hipSuccess);
  for (int i = 0; i < ops; ++i) CHECK(same(outs[i], fold(c[i], FRG_SCALE_NONE, 1.f)));
  // any other stream is told every time (it may be destroyed and its handle reused)
  hipStream_t consumer;
  CHECK(hipStreamCreateWithFlags(&consumer, hipStreamNonBlocking) == hipSuccess);
  const long before = fake_hip_calls("hipStreamWaitEvent");
  for (int i = 0; i < ops; ++i) CHECK(frg_work_block_stream(w[i], consumer) == FRG_OK);
  CHECK(fake_hip_calls("hipStreamWaitEvent") - before == ops);
  for (frg_work* x : w) frg_work_release(x);
  // an operation that comes later is waited for again
  Vec late(n, -1.f);
  frg_work* wl = nullptr;
  auto t = table(c[0]);
  fake_hip_occupy(streamsOf(ctx)[0], 20);
  fake_hip_occupy(streamsOf(ctx)[1], 20);
  CHECK(frg_allreduce(ctx, late.data(), t.data(), 3, n, FRG_F32, FRG_SUM, FRG_SCALE_NONE, 1.f,
                      producer, nullptr, nullptr, &wl) == FRG_OK);
  const long again = fake_hip_calls("hipStreamWaitEvent");
  CHECK(frg_work_block_stream(wl, nullptr) == FRG_OK);
  CHECK(fake_hip_calls("hipStreamWaitEvent") == again + 1);
  CHECK(hipStreamSynchronize(nullptr) == hipSuccess);
  CHECK(same(late, fold(c[0], FRG_SCALE_NONE, 1.f)));
  frg_work_release(wl);
  CHECK(frg_destroy(ctx) == FRG_OK);
  CHECK(hipStreamDestroy(producer) == hipSuccess);
  CHECK(hipStreamDestroy(consumer) == hipSuccess);
}

// A completion callback that holds the command thread until the test lets go.
struct Gate {
  std::mutex mu;
  std::condition_variable cv;
  bool open = false;
  bool reached = false;
};
void waitAtGate(void* user, int, void*) {
  auto* g = static_cast<Gate*>(user);
  std::unique_lock<std::mutex> lock(g->mu);
  g->reached = true;
  g->cv.notify_all();
  g->cv.wait(lock, [&] { return g->open; });
}
struct Order {
  std::mutex mu;
  std::vector<int> seen;
};
struct OrderNote {
  Order* order;
  int index;
};
void noteOrder(void* user, int status, void*) {
  auto* n = static_cast<OrderNote*>(user);
  std::lock_guard<std::mutex> g(n->order->mu);
  n->order->seen.push_back(status == FRG_OK ? n->index : -1);
}

void scenarioNeighboursRunAsOne() {
  std::puts("operations that are waiting and continue one another run as one");
  const int64_t piece = 3000, pieces = 8;
  for (int variant = 0; variant < 4; ++variant) {
    frg_ctx* ctx = makeCtx(8192, 4096, 2, 0);
    // one tensor per contribution, cut into pieces like a gradient into buckets
    auto c = randomContribs(3, piece * pieces, 90 + variant);
    Vec out(piece * pieces, -1.f);
    Vec own = c[0];
    // hold the command thread in the callback of an operation of its own
    Gate gate;
    auto other = randomContribs(2, 100, 99);
    Vec otherOut(100);
    auto ot = table(other);
    CHECK(frg_allreduce(ctx, otherOut.data(), ot.data(), 2, 100, FRG_F32, FRG_SUM, FRG_SCALE_NONE,
                        1.f, nullptr, &waitAtGate, &gate, nullptr) == FRG_OK);
    {
      std::unique_lock<std::mutex> lock(gate.mu);
      gate.cv.wait(lock, [&] { return gate.reached; });
    }
    frg_progress2 before = {};
    CHECK(frg_get_progress2(ctx, &before, sizeof(before)) == FRG_OK);
    Order order;
    std::vector<OrderNote> notes(pieces);
    std::vector<frg_work*> w(pieces, nullptr);
    for (int i = 0; i < pieces; ++i) {
      // variant 0: from the end of the tensor to its start (DDP's order), a separate output;
      // 1: from start to end, in place into the first contribution; 2: the order changes
      // direction half way; 3: every second piece, then the others (nothing continues anything)
      int at = variant == 1 ? i : pieces - 1 - i;
      if (variant == 2 && i >= 4) at = i - 4;                      // 7 6 5 4, then 0 1 2 3
      if (variant == 3) at = i < 4 ? 2 * i : 2 * (i - 4) + 1;      // 0 2 4 6 1 3 5 7
      const int64_t off = at * piece;
      const void* tab[3] = {variant == 1 ? own.data() + off : c[0].data() + off,
                            c[1].data() + off, c[2].data() + off};
      float* dst = variant == 1 ? own.data() + off : out.data() + off;
      notes[i] = OrderNote{&order, i};
      CHECK(frg_allreduce(ctx, dst, tab, 3, piece, FRG_F32, FRG_SUM, FRG_SCALE_MUL, 0.5f, nullptr,
                          &noteOrder, &notes[i], &w[i]) == FRG_OK);
    }
    {
      std::lock_guard<std::mutex> lock(gate.mu);
      gate.open = true;
    }
    gate.cv.notify_all();
    for (frg_work* x : w) CHECK(frg_work_wait(x) == FRG_OK);
    CHECK(frg_synchronize(ctx) == FRG_OK);
    frg_progress2 after = {};
    CHECK(frg_get_progress2(ctx, &after, sizeof(after)) == FRG_OK);
    CHECK(after.enqueued - before.enqueued == pieces);
    if (variant <= 1) {
      CHECK(after.merged - before.merged == pieces);           // one run of eight
      CHECK(after.launches - before.launches < pieces);        // cut from the joint range
    } else if (variant == 2) {
      CHECK(after.merged - before.merged == pieces);           // two runs of four
    } else {
      CHECK(after.merged == before.merged);
      CHECK(after.launches - before.launches >= pieces);
    }
    const Vec want = fold(c, FRG_SCALE_MUL, 0.5f);
    CHECK(same(variant == 1 ? own : out, want));
    {
      std::lock_guard<std::mutex> g(order.mu);
      CHECK(static_cast<int>(order.seen.size()) == pieces);
      for (int i = 0; i < pieces; ++i) CHECK(order.seen[i] == i);  // callbacks in submission order
    }
    for (frg_work* x : w) frg_work_release(x);
    CHECK(frg_destroy(ctx) == FRG_OK);
  }
  // Two operations that continue one another but each read what the other
  // writes are not one elementwise operation: they stay apart, and in order.
  {
    frg_ctx* ctx = makeCtx(8192, 4096, 2, 0);
    const int64_t n = 2000;
    Vec z(3 * n);
    for (int64_t i = 0; i < 3 * n; ++i) z[i] = static_cast<float>(i % 97) * 0.25f;
    const Vec z0 = z;
    Gate gate;
    auto other = randomContribs(2, 100, 98);
    Vec otherOut(100);
    auto ot = table(other);
    CHECK(frg_allreduce(ctx, otherOut.data(), ot.data(), 2, 100, FRG_F32, FRG_SUM, FRG_SCALE_NONE,
                        1.f, nullptr, &waitAtGate, &gate, nullptr) == FRG_OK);
    {
      std::unique_lock<std::mutex> lock(gate.mu);
      gate.cv.wait(lock, [&] { return gate.reached; });
    }
    frg_progress2 before = {};
    CHECK(frg_get_progress2(ctx, &before, sizeof(before)) == FRG_OK);
    // pieces of n/4 from the top of z[n, 2n) downwards, each written from the piece n below it
    // and added to itself: z[n + j] += z[j]; the four would join into z[n, 2n) += z[0, n),
    // fine; then the same one step further down, z[j] += z[j - ...] is what must not join:
    // here output z[n/2 + ...] reads z[...] that a neighbour writes
    std::vector<frg_work*> w;
    const int64_t q = n / 4;
    for (int i = 0; i < 4; ++i) {
      // output piece [2n - (i+1)q, 2n - iq), contribution one piece lower: [.. - q, ..)
      float* dst = z.data() + 2 * n - (i + 1) * q;
      const void* tab[2] = {dst, dst - q};  // in place, plus the piece directly below
      frg_work* x = nullptr;
      CHECK(frg_allreduce(ctx, dst, tab, 2, q, FRG_F32, FRG_SUM, FRG_SCALE_NONE, 1.f, nullptr,
                          nullptr, nullptr, &x) == FRG_OK);
      w.push_back(x);
    }
    {
      std::lock_guard<std::mutex> lock(gate.mu);
      gate.open = true;
    }
    gate.cv.notify_all();
    for (frg_work* x : w) CHECK(frg_work_wait(x) == FRG_OK);
    frg_progress2 after = {};
    CHECK(frg_get_progress2(ctx, &after, sizeof(after)) == FRG_OK);
    CHECK(after.merged == before.merged);
    // sequentially: piece i adds the ORIGINAL piece below it (that one is updated only later)
    Vec want = z0;
    for (int i = 0; i < 4; ++i) {
      const int64_t lo = 2 * n - (i + 1) * q;
      for (int64_t j = 0; j < q; ++j) want[lo + j] = want[lo + j] + want[lo - q + j];
    }
    CHECK(same(z, want));
    for (frg_work* x : w) frg_work_release(x);
    CHECK(frg_destroy(ctx) == FRG_OK);
  }
  // The same with the contribution four and a half pieces below the output:
  // a run of four neighbours is apart from what it reads, a run of five is not,
  // so the eight waiting operations run as two runs of four.
  {
    frg_ctx* ctx = makeCtx(8192, 4096, 2, 0);
    const int64_t q = 500, count = 8, gap = 9 * q / 2;
    Vec z(gap + count * q);
    for (size_t i = 0; i < z.size(); ++i) z[i] = static_cast<float>(i % 89) * 0.5f;
    const Vec z0 = z;
    Gate gate;
    auto other = randomContribs(2, 100, 97);
    Vec otherOut(100);
    auto ot = table(other);
    CHECK(frg_allreduce(ctx, otherOut.data(), ot.data(), 2, 100, FRG_F32, FRG_SUM, FRG_SCALE_NONE,
                        1.f, nullptr, &waitAtGate, &gate, nullptr) == FRG_OK);
    {
      std::unique_lock<std::mutex> lock(gate.mu);
      gate.cv.wait(lock, [&] { return gate.reached; });
    }
    std::vector<frg_work*> w;
    for (int i = 0; i < count; ++i) {   // from the top down; each adds what lies `gap` below it
      float* dst = z.data() + gap + (count - 1 - i) * q;
      const void* tab[2] = {dst, dst - gap};
      frg_work* x = nullptr;
      CHECK(frg_allreduce(ctx, dst, tab, 2, q, FRG_F32, FRG_SUM, FRG_SCALE_NONE, 1.f, nullptr,
                          nullptr, nullptr, &x) == FRG_OK);
      w.push_back(x);
    }
    {
      std::lock_guard<std::mutex> lock(gate.mu);
      gate.open = true;
    }
    gate.cv.notify_all();
    for (frg_work* x : w) CHECK(frg_work_wait(x) == FRG_OK);
    frg_progress2 after = {};
    CHECK(frg_get_progress2(ctx, &after, sizeof(after)) == FRG_OK);
    CHECK(after.merged == count);
    Vec want = z0;
    for (int i = 0; i < count; ++i) {
      const int64_t lo = gap + (count - 1 - i) * q;
      for (int64_t j = 0; j < q; ++j) want[lo + j] = want[lo + j] + want[lo - gap + j];
    }
    CHECK(same(z, want));
    for (frg_work* x : w) frg_work_release(x);
    CHECK(frg_destroy(ctx) == FRG_OK);
  }
}

void scenarioProducerOrdering() {
  std::puts("the pipeline waits for the producer stream");
  frg_ctx* ctx = makeCtx(8192, 4096, 2, 1024);
  hipStream_t producer;
  CHECK(hipStreamCreateWithFlags(&producer, hipStreamNonBlocking) == hipSuccess);
  const int64_t n = 5000;
  Vec a(n, 0.f), b(n, 0.f), out(n, -1.f);
  // the producer fills a and b late, on its own stream
  fake_hip_occupy(producer, 50);
  Vec srcA(n, 1.5f), srcB(n, 2.5f);
  CHECK(hipMemcpyAsync(a.data(), srcA.data(), n * 4, hipMemcpyHostToDevice, producer) == hipSuccess);
  CHECK(hipMemcpyAsync(b.data(), srcB.data(), n * 4, hipMemcpyHostToDevice, producer) == hipSuccess);
  const void* t[2] = {a.data(), b.data()};
  frg_work* w = nullptr;
  CHECK(frg_allreduce(ctx, out.data(), t, 2, n, FRG_F32, FRG_SUM, FRG_SCALE_NONE, 1.f, producer,
                      nullptr, nullptr, &w) == FRG_OK);
  // a consumer stream ordered after the work without a host wait
  hipStream_t consumer;
  CHECK(hipStreamCreateWithFlags(&consumer, hipStreamNonBlocking) == hipSuccess);
  Vec copy(n, 0.f);
  CHECK(frg_work_block_stream(w, consumer) == FRG_OK);
  CHECK(hipMemcpyAsync(copy.data(), out.data(), n * 4, hipMemcpyDeviceToHost, consumer) == hipSuccess);
  CHECK(hipStreamSynchronize(consumer) == hipSuccess);
  for (float x : copy) CHECK(x == 4.0f);
  frg_work_release(w);
  CHECK(frg_destroy(ctx) == FRG_OK);
}

void scenarioHostStaged() {
  std::puts("host-staged accumulation: slot rotation and reuse");
  for (int slots : {1, 2, 3, 5, 7, 8, 9, 11}) {
    frg_ctx* ctx = makeCtx(4096 * slots, 4096, 0, 0);
    frg_layout l;
    CHECK(frg_get_layout(ctx, &l) == FRG_OK && l.num_staging_slots == slots);
    for (int k : {1, 2, 7, 20}) {
      auto c = randomContribs(k, 2500, 7 * k + slots);  // 3 staged slices of <= 1024 elements
      Vec out(2500, -1.f);
      auto t = table(c);
      frg_work* w = nullptr;
      CHECK(frg_allreduce_host(ctx, out.data(), t.data(), k, 2500, FRG_F32, FRG_SUM,
                               FRG_SCALE_DIV, static_cast<float>(k), /*carry=*/0, nullptr, nullptr,
                               nullptr, &w) == FRG_OK);
      CHECK(frg_work_wait(w) == FRG_OK);
      CHECK(same(out, fold(c, FRG_SCALE_DIV, static_cast<float>(k))));
      frg_work_release(w);
      // carry: the output already holds the first term
      Vec own = c[0];
      std::vector<Vec> rest(c.begin() + 1, c.end());
      auto tr = table(rest);
      CHECK(frg_allreduce_host(ctx, own.data(), tr.data(), k - 1, 2500, FRG_F32, FRG_SUM,
                               FRG_SCALE_DIV, static_cast<float>(k), /*carry=*/1, nullptr, nullptr,
                               nullptr, &w) == FRG_OK);
      CHECK(frg_work_wait(w) == FRG_OK);
      CHECK(same(own, fold(c, FRG_SCALE_DIV, static_cast<float>(k))));
      frg_work_release(w);
    }
    CHECK(frg_destroy(ctx) == FRG_OK);
  }
  // slices of 4 MiB and more: the second staging stream's first batch goes in two halves
  for (int slots : {2, 4}) {
    const int64_t n = (5ll << 20) / 4 + 12345;  // two slices: 4 MiB and a ragged rest
    frg_ctx* ctx = makeCtx((4ll << 20) * slots, 4ll << 20, 0, 0);
    for (int k : {2, 3, 6}) {
      auto c = randomContribs(k, n, 90 + k + slots);
      Vec own = c[0];
      std::vector<Vec> rest(c.begin() + 1, c.end());
      auto tr = table(rest);
      frg_work* w = nullptr;
      CHECK(frg_allreduce_host(ctx, own.data(), tr.data(), k - 1, n, FRG_F32, FRG_SUM,
                               FRG_SCALE_MUL, 0.5f, /*carry=*/1, nullptr, nullptr, nullptr,
                               &w) == FRG_OK);
      CHECK(frg_work_wait(w) == FRG_OK);
      CHECK(same(own, fold(c, FRG_SCALE_MUL, 0.5f)));
      frg_work_release(w);
      Vec out(n, -1.f);
      auto t = table(c);
      CHECK(frg_allreduce_host(ctx, out.data(), t.data(), k, n, FRG_F32, FRG_SUM, FRG_SCALE_NONE,
                               1.f, /*carry=*/0, nullptr, nullptr, nullptr, &w) == FRG_OK);
      CHECK(frg_work_wait(w) == FRG_OK);
      CHECK(same(out, fold(c, FRG_SCALE_NONE, 1.f)));
      frg_work_release(w);
    }
    CHECK(frg_destroy(ctx) == FRG_OK);
  }
}

void scenarioGathered() {
  std::puts("one contribution given piecewise: cut on tiles, packed into segmented launches");
  std::mt19937 rng(321);
  for (int round = 0; round < 6; ++round) {
    const int k = round % 2 == 0 ? 8 : 3;
    const int g = static_cast<int>(rng() % k);
    // segment lengths: big ones (one crosses a launch's 8 MiB), tiny ones, odd ones
    std::vector<int64_t> lens;
    if (round < 2) {
      lens = {2500000, 2048, 2048, 700000, 0, 4096, 1, 3};
    } else if (round == 2) {
      lens = {5000000, 16, 2048, 1200000};  // 23.7 MiB: launches of 8 + 8 + the rest
    } else {
      const int count = 1 + static_cast<int>(rng() % 40);
      for (int i = 0; i < count; ++i) {
        const int kind = static_cast<int>(rng() % 4);
        lens.push_back(kind == 0 ? static_cast<int64_t>(rng() % 9)
                                 : (kind == 1 ? 4 * static_cast<int64_t>(rng() % 3000)
                                              : static_cast<int64_t>(rng() % 50000)));
      }
    }
    int64_t n = 0;
    for (int64_t l : lens) n += l;
    auto c = randomContribs(k, n, 600 + round);
    // the gathered contribution lives in tensors of its own (some start off a 16-byte boundary)
    std::vector<Vec> pieces;
    std::vector<frg_segment> segs;
    int64_t off = 0;
    for (size_t i = 0; i < lens.size(); ++i) {
      const int64_t skew = (round >= 4 && i % 3 == 1) ? 1 : 0;
      Vec v(static_cast<size_t>(lens[i] + skew + 4));
      for (int64_t j = 0; j < lens[i]; ++j) v[static_cast<size_t>(j + skew)] = c[g][static_cast<size_t>(off + j)];
      pieces.push_back(std::move(v));
      off += lens[i];
    }
    for (size_t i = 0; i < lens.size(); ++i) {
      const int64_t skew = (round >= 4 && i % 3 == 1) ? 1 : 0;
      segs.push_back(frg_segment{pieces[i].data() + skew, lens[i]});
    }
    auto t = table(c);
    t[static_cast<size_t>(g)] = nullptr;  // ignored
    frg_ctx* ctx = makeCtx(8192, 4096, 2, 0);
    Vec out(static_cast<size_t>(n), -1.f);
    frg_work* w = nullptr;
    const int mode = round % 3 == 0 ? FRG_SCALE_MUL : (round % 3 == 1 ? FRG_SCALE_PRE_MUL : FRG_SCALE_NONE);
    CHECK(frg_allreduce_gathered(ctx, out.data(), t.data(), k, g, segs.data(),
                                 static_cast<int>(segs.size()), n, FRG_F32, FRG_SUM, mode, 0.125f,
                                 nullptr, nullptr, nullptr, &w) == FRG_OK);
    CHECK(frg_work_wait(w) == FRG_OK);
    CHECK(same(out, fold(c, mode, 0.125f)));
    frg_work_release(w);
    frg_progress2 pr = {};
    CHECK(frg_get_progress2(ctx, &pr, sizeof(pr)) == FRG_OK);
    if (round < 3) CHECK(pr.segmented_launches >= 1);  // the random rounds may hold one tensor only
    if (round == 2) {
      // 2048 + 2048 + 1974 tiles: the first two lie within the first tensor and are plain
      // launches, the third holds the ends of all four
      CHECK(pr.segmented_launches == 1 && pr.launches == 3);
    }
    if (round == 0) {
      // 3.2 M elements of 8 contributions, 12.2 MiB each: a launch of 8 MiB and one with the
      // rest (more than half a launch's worth); the last piece sits 4 bytes off its tensor's
      // position within 16 bytes (a one-element piece lies ahead of it): a plain launch of its own
      CHECK(pr.segmented_launches == 1 && pr.launches == 3);
    }
    // MAX is not the segmented kernel's: every piece as a plain launch, same result as the fold
    Vec mx(static_cast<size_t>(n), -1.f);
    CHECK(frg_allreduce_gathered(ctx, mx.data(), t.data(), k, g, segs.data(),
                                 static_cast<int>(segs.size()), n, FRG_F32, FRG_MAX, FRG_SCALE_NONE,
                                 1.f, nullptr, nullptr, nullptr, &w) == FRG_OK);
    CHECK(frg_work_wait(w) == FRG_OK);
    for (int64_t i = 0; i < n; ++i) {
      float m = c[0][static_cast<size_t>(i)];
      for (int kk = 1; kk < k; ++kk) m = m > c[kk][static_cast<size_t>(i)] ? m : c[kk][static_cast<size_t>(i)];
      CHECK(mx[static_cast<size_t>(i)] == m);
    }
    frg_work_release(w);
    // contract: lengths must add up, the index must be in range, the output no other contribution
    CHECK(frg_allreduce_gathered(ctx, out.data(), t.data(), k, g, segs.data(),
                                 static_cast<int>(segs.size()), n + 1, FRG_F32, FRG_SUM, 0, 1.f,
                                 nullptr, nullptr, nullptr, nullptr) == FRG_ERR_INVALID);
    CHECK(frg_allreduce_gathered(ctx, out.data(), t.data(), k, k, segs.data(),
                                 static_cast<int>(segs.size()), n, FRG_F32, FRG_SUM, 0, 1.f,
                                 nullptr, nullptr, nullptr, nullptr) == FRG_ERR_INVALID);
    if (n > 0) {
      auto alias = t;
      alias[static_cast<size_t>((g + 1) % k)] = out.data();
      CHECK(frg_allreduce_gathered(ctx, out.data(), alias.data(), k, g, segs.data(),
                                   static_cast<int>(segs.size()), n, FRG_F32, FRG_SUM, 0, 1.f,
                                   nullptr, nullptr, nullptr, nullptr) == FRG_ERR_INVALID);
    }
    CHECK(frg_destroy(ctx) == FRG_OK);
  }
}

bool gSharedHwQueues = false;

// Streams of a context as the ABI hands them out (reduce streams first).
std::vector<hipStream_t> streamsOf(frg_ctx* ctx) {
  void* raw[16];
  int n = 0;
  CHECK(frg_get_streams(ctx, raw, 16, &n) == FRG_OK);
  std::vector<hipStream_t> v;
  for (int i = 0; i < n && i < 16; ++i) v.push_back(static_cast<hipStream_t>(raw[i]));
  return v;
}

// Which launches are asked to mix the loads of a lane's two vectors: those of
// operations whose contributions lie close to one another.
void scenarioMixedLoadsRule() {
  auto at = [](uint64_t a) { return reinterpret_cast<const void*>(a); };
  const uint64_t MiBs = 1ull << 20, base = 0x7f0000000000ull;
  {
    const void* p[8];
    for (int k = 0; k < 8; ++k) p[k] = at(base + k * 26 * MiBs);
    CHECK(frg::closelySpaced(p, 8));  // a bucket's tensors, allocated one by one
    for (int k = 0; k < 8; ++k) p[k] = at(base + k * 5480000000ull);
    CHECK(!frg::closelySpaced(p, 8));  // the tensors of a whole gradient
    for (int k = 1; k < 8; ++k) p[k] = at(base + k * 26 * MiBs);
    p[0] = at(base + 40000 * MiBs);
    CHECK(frg::closelySpaced(p, 8));  // the bucket far from its peers' copies, those side by side
    p[3] = p[0];
    CHECK(frg::closelySpaced(p, 8));  // an address twice (in place) counts once
    CHECK(!frg::closelySpaced(p, 1));
    const void* two[2] = {at(base), at(base + 512 * MiBs)};
    CHECK(frg::closelySpaced(two, 2));
    two[1] = at(base + 1024 * MiBs);
    CHECK(!frg::closelySpaced(two, 2));
    const void* same[2] = {at(base), at(base)};
    CHECK(!frg::closelySpaced(same, 2));
  }
  // through the pipeline: host buffers lie megabytes apart
  frg_options o = {};
  o.max_memory_allocated_in_bytes = 2 << 20;
  o.slice_size_in_bytes = 1 << 20;
  frg_ctx* ctx = nullptr;
  CHECK(frg_create(0, &o, &ctx) == FRG_OK);
  const int64_t n = 300000;
  std::vector<std::vector<float>> x(4, std::vector<float>(n, 1.0f));
  std::vector<float> out(n, 0.0f);
  const void* t[4] = {x[0].data(), x[1].data(), x[2].data(), x[3].data()};
  const long long before = frg::mixedLoadLaunches();
  frg_work* w = nullptr;
  CHECK(frg_allreduce(ctx, out.data(), t, 4, n, FRG_F32, FRG_SUM, FRG_SCALE_NONE, 1.0f, nullptr,
                      nullptr, nullptr, &w) == FRG_OK);
  CHECK(frg_work_wait(w) == FRG_OK);
  frg_work_release(w);
  frg_progress pr = {};
  CHECK(frg_get_progress(ctx, &pr) == FRG_OK);
  CHECK(frg::mixedLoadLaunches() - before >= 1);
  for (int64_t i = 0; i < n; i += 9973) CHECK(out[static_cast<size_t>(i)] == 4.0f);
  CHECK(frg_destroy(ctx) == FRG_OK);
}

void scenarioStreamsAreReused() {
  std::puts("contexts created one after the other run on the same streams");
  frg_ctx* a = makeCtx(8192, 4096, 2, 0);
  const std::vector<hipStream_t> first = streamsOf(a);
  CHECK(first.size() == 2);
  CHECK(frg_destroy(a) == FRG_OK);
  const long created = fake_hip_calls("hipStreamCreateWithFlags");
  frg_ctx* b = makeCtx(8192, 4096, 2, 0);
  CHECK(streamsOf(b) == first);                       // handed back, handed out again
  frg_ctx* c = makeCtx(8192, 4096, 2, 0);             // while b lives: streams of its own
  const std::vector<hipStream_t> other = streamsOf(c);
  CHECK(other.size() == 2 && other[0] != first[0] && other[0] != first[1] &&
        other[1] != first[0] && other[1] != first[1]);
  CHECK(frg_destroy(b) == FRG_OK);
  CHECK(frg_destroy(c) == FRG_OK);
  frg_ctx* d = makeCtx(8192, 4096, 3, 0);             // three: the oldest idle ones first
  const std::vector<hipStream_t> three = streamsOf(d);
  CHECK(three.size() == 3 && three[0] == first[0] && three[1] == first[1]);
  CHECK(frg_destroy(d) == FRG_OK);
  CHECK(fake_hip_calls("hipStreamCreateWithFlags") <= created + 2);
}

void scenarioOrderBetweenOperations() {
  std::puts("operations that share memory keep their order across the reduce streams");
  // bucket-sized operations alternate between the two reduce streams; the first
  // stream is held up, so whatever is not ordered after it runs too early
  const int64_t n = 3000;
  for (int round = 0; round < 3; ++round) {
    frg_ctx* ctx = makeCtx(8192, 4096, 2, 0);
    CHECK(streamsOf(ctx).size() == 2);  // no copy streams until something is staged
    hipStream_t s0 = streamsOf(ctx)[0];
    auto c = randomContribs(4, n, 40 + round);
    auto t = table(c);
    Vec own = c[0];
    std::vector<const void*> tab = t;
    tab[0] = own.data();
    frg_work* w[3] = {nullptr, nullptr, nullptr};
    fake_hip_occupy(s0, 60);
    std::printf("  shared tensor, case %d\n", round);
    if (round == 0) {
      // three in-place reductions of the same tensor, none waited for (a scale
      // of its own each, so that their order shows in the result)
      Vec want = own;
      const float scales[3] = {0.5f, 0.25f, 2.0f};
      for (int i = 0; i < 3; ++i) {
        std::vector<Vec> terms = {want, c[1], c[2], c[3]};
        want = fold(terms, FRG_SCALE_MUL, scales[i]);
        CHECK(frg_allreduce(ctx, own.data(), tab.data(), 4, n, FRG_F32, FRG_SUM, FRG_SCALE_MUL,
                            scales[i], nullptr, nullptr, nullptr, &w[i]) == FRG_OK);
      }
      CHECK(frg_work_wait(w[2]) == FRG_OK);  // the last one covers the others
      CHECK(same(own, want));
    } else if (round == 1) {
      // the output of one operation is a contribution of the next (a
      // reduce-scatter's output fed to an allreduce)
      Vec mid(n, -1.f), out(n, -1.f);
      CHECK(frg_allreduce(ctx, mid.data(), t.data(), 4, n, FRG_F32, FRG_SUM, FRG_SCALE_NONE, 1.f,
                          nullptr, nullptr, nullptr, &w[0]) == FRG_OK);
      const void* second[2] = {mid.data(), c[1].data()};
      CHECK(frg_allreduce(ctx, out.data(), second, 2, n, FRG_F32, FRG_SUM, FRG_SCALE_NONE, 1.f,
                          nullptr, nullptr, nullptr, &w[1]) == FRG_OK);
      CHECK(frg_work_wait(w[1]) == FRG_OK);
      std::vector<Vec> terms = {fold(c, FRG_SCALE_NONE, 1.f), c[1]};
      CHECK(same(out, fold(terms, FRG_SCALE_NONE, 1.f)));
    } else {
      // write after read: the second operation overwrites a contribution of the first
      Vec out(n, -1.f);
      const Vec want = fold(c, FRG_SCALE_NONE, 1.f);
      CHECK(frg_allreduce(ctx, out.data(), t.data(), 4, n, FRG_F32, FRG_SUM, FRG_SCALE_NONE, 1.f,
                          nullptr, nullptr, nullptr, &w[0]) == FRG_OK);
      const void* second[2] = {c[1].data(), c[2].data()};
      CHECK(frg_allreduce(ctx, c[3].data(), second, 2, n, FRG_F32, FRG_SUM, FRG_SCALE_NONE, 1.f,
                          nullptr, nullptr, nullptr, &w[1]) == FRG_OK);
      CHECK(frg_work_wait(w[0]) == FRG_OK);
      CHECK(frg_work_wait(w[1]) == FRG_OK);
      CHECK(same(out, want));
    }
    for (frg_work* x : w) {
      if (x) frg_work_release(x);
    }
    CHECK(frg_destroy(ctx) == FRG_OK);
  }
  // independent buckets are not ordered against each other: with the first
  // stream held up, the bucket on the second stream finishes first
  {
    frg_ctx* ctx = makeCtx(8192, 4096, 2, 0);
    hipStream_t s0 = streamsOf(ctx)[0];
    auto a = randomContribs(3, n, 50), b = randomContribs(3, n, 51);
    Vec outA(n), outB(n);
    auto ta = table(a), tb = table(b);
    frg_work *wa = nullptr, *wb = nullptr;
    fake_hip_occupy(s0, 300);
    std::puts("  independent buckets");
    CHECK(frg_allreduce(ctx, outA.data(), ta.data(), 3, n, FRG_F32, FRG_SUM, FRG_SCALE_NONE, 1.f,
                        nullptr, nullptr, nullptr, &wa) == FRG_OK);
    CHECK(frg_allreduce(ctx, outB.data(), tb.data(), 3, n, FRG_F32, FRG_SUM, FRG_SCALE_NONE, 1.f,
                        nullptr, nullptr, nullptr, &wb) == FRG_OK);
    CHECK(frg_work_wait(wb) == FRG_OK);
    CHECK(same(outB, fold(b, FRG_SCALE_NONE, 1.f)));
    // the first stream is still held up (streams that share a hardware queue
    // cannot overtake each other, so this only holds with a queue per stream)
    if (!gSharedHwQueues) CHECK(hipStreamQuery(s0) == hipErrorNotReady);
    CHECK(frg_work_wait(wa) == FRG_OK);
    CHECK(same(outA, fold(a, FRG_SCALE_NONE, 1.f)));
    frg_work_release(wa);
    frg_work_release(wb);
    // many independent buckets: the bookkeeping stays bounded (a forced join now and then)
    std::puts("  many independent buckets");
    std::vector<Vec> outs(200, Vec(256));
    auto small = randomContribs(2, 256, 52);
    auto ts = table(small);
    for (auto& o : outs) {
      CHECK(frg_allreduce(ctx, o.data(), ts.data(), 2, 256, FRG_F32, FRG_SUM, FRG_SCALE_NONE, 1.f,
                          nullptr, nullptr, nullptr, nullptr) == FRG_OK);
    }
    CHECK(frg_synchronize(ctx) == FRG_OK);
    for (auto& o : outs) CHECK(same(o, fold(small, FRG_SCALE_NONE, 1.f)));
    CHECK(frg_destroy(ctx) == FRG_OK);
  }
  // a resident operation followed by a host-staged one into the same tensor, and back
  {
    frg_ctx* ctx = makeCtx(2 * 4096, 4096, 2, 0);
    auto c = randomContribs(3, n, 53);
    auto t = table(c);
    Vec out(n, -1.f);
    hipStream_t s1 = streamsOf(ctx)[1];
    std::puts("  resident, host-staged, resident on one tensor");
    CHECK(frg_allreduce(ctx, out.data(), t.data(), 3, 16, FRG_F32, FRG_SUM, FRG_SCALE_NONE, 1.f,
                        nullptr, nullptr, nullptr, nullptr) == FRG_OK);  // takes stream 0
    fake_hip_occupy(s1, 60);
    CHECK(frg_allreduce(ctx, out.data(), t.data(), 3, n, FRG_F32, FRG_SUM, FRG_SCALE_NONE, 1.f,
                        nullptr, nullptr, nullptr, nullptr) == FRG_OK);  // stream 1, held up
    // `out` now is the first term; the staged copies must not overtake the operation before
    CHECK(frg_allreduce_host(ctx, out.data(), t.data(), 3, n, FRG_F32, FRG_SUM, FRG_SCALE_NONE,
                             1.f, /*carry=*/1, nullptr, nullptr, nullptr, nullptr) == FRG_OK);
    frg_work* w = nullptr;
    const void* again[2] = {out.data(), c[0].data()};
    Vec out2(n, -1.f);
    CHECK(frg_allreduce(ctx, out2.data(), again, 2, n, FRG_F32, FRG_SUM, FRG_SCALE_NONE, 1.f,
                        nullptr, nullptr, nullptr, &w) == FRG_OK);
    CHECK(frg_work_wait(w) == FRG_OK);
    CHECK(streamsOf(ctx).size() == 3);  // the staging stream exists once something was staged
    const Vec first = fold(c, FRG_SCALE_NONE, 1.f);
    const Vec staged = fold(c, FRG_SCALE_NONE, 1.f, &first);
    CHECK(same(out, staged));
    std::vector<Vec> terms = {staged, c[0]};
    CHECK(same(out2, fold(terms, FRG_SCALE_NONE, 1.f)));
    frg_work_release(w);
    CHECK(frg_destroy(ctx) == FRG_OK);
  }
}

void scenarioRandomDependentOperations() {
  std::puts("random sequences of operations over shared buffers equal their sequential execution");
  for (unsigned seed = 0; seed < 6; ++seed) {
    std::mt19937 rng(7000 + seed);
    const int nbuf = 4;
    const int64_t size = 6000;
    const int streams = 2 + static_cast<int>(seed % 2);
    frg_ctx* ctx = makeCtx(8192, 4096, streams, seed % 3 == 0 ? 0 : 2048);
    const std::vector<hipStream_t> ss = streamsOf(ctx);
    auto bufs = randomContribs(nbuf, size, 8000 + seed);
    auto shadow = bufs;
    std::uniform_int_distribution<int> pickBuf(0, nbuf - 1), pickK(2, 5), pickDelay(0, 3);
    std::vector<std::vector<const void*>> tables;  // kept alive until the operations have run
    for (int op = 0; op < 60; ++op) {
      const int64_t n = 200 + static_cast<int64_t>(rng() % 1500);
      const int ob = pickBuf(rng);
      const int64_t olo = static_cast<int64_t>(rng() % static_cast<unsigned>(size - n));
      const int k = pickK(rng);
      std::vector<std::pair<int, int64_t>> terms;
      for (int t = 0; t < k; ++t) {
        if (rng() % 4 == 0) {
          terms.emplace_back(ob, olo);  // in place
          continue;
        }
        for (;;) {
          const int cb = pickBuf(rng);
          const int64_t clo = static_cast<int64_t>(rng() % static_cast<unsigned>(size - n));
          if (cb != ob || clo + n <= olo || olo + n <= clo) {
            terms.emplace_back(cb, clo);
            break;
          }
        }
      }
      // hold one of the streams up now and then, so that an unordered operation runs too early
      if (pickDelay(rng) == 0) fake_hip_occupy(ss[rng() % ss.size()], 2);
      std::vector<const void*> tab;
      for (auto& t : terms) tab.push_back(bufs[t.first].data() + t.second);
      tables.push_back(tab);
      CHECK(frg_allreduce(ctx, bufs[ob].data() + olo, tables.back().data(), k, n, FRG_F32, FRG_SUM,
                          FRG_SCALE_MUL, 0.5f, nullptr, nullptr, nullptr, nullptr) == FRG_OK);
      Vec acc(shadow[terms[0].first].begin() + terms[0].second,
              shadow[terms[0].first].begin() + terms[0].second + n);
      for (size_t t = 1; t < terms.size(); ++t) {
        for (int64_t i = 0; i < n; ++i) acc[i] = acc[i] + shadow[terms[t].first][terms[t].second + i];
      }
      for (int64_t i = 0; i < n; ++i) shadow[ob][olo + i] = acc[i] * 0.5f;
    }
    CHECK(frg_synchronize(ctx) == FRG_OK);
    for (int b = 0; b < nbuf; ++b) CHECK(same(bufs[b], shadow[b]));
    CHECK(frg_destroy(ctx) == FRG_OK);
  }
}

// What the c10d extension does around the ABI, with a mutex standing in for
// Python's global lock: the caller holds it except inside the calls that let go
// of it (submitting, waiting); the completion callback, on the command thread,
// takes it briefly (it drops tensor references). 15 peers in host memory staged
// through 2 slots, the rank's own term already in `out`, several operations,
// each waited for through its callback alone.
std::mutex gInterpreterLock;

struct GroupPending {
  std::atomic<int> done{0};
  std::atomic<void*> stream{nullptr};
};

void onGroupDone(void* user, int status, void* lastStream) {
  auto* p = static_cast<GroupPending*>(user);
  CHECK(status == FRG_OK);
  {
    std::lock_guard<std::mutex> g(gInterpreterLock);  // "drop the tensor references"
    p->stream = lastStream;
  }
  p->done = 1;
}

void scenarioProcessGroupShaped() {
  std::puts("process-group-shaped: staged peers, callback that takes the interpreter lock");
  frg_ctx* ctx = makeCtx(2 * 4096, 4096, 2, 0);
  hipStream_t callerStream;
  CHECK(hipStreamCreateWithFlags(&callerStream, hipStreamNonBlocking) == hipSuccess);
  std::unique_lock<std::mutex> gil(gInterpreterLock);
  const int ops = 8;
  for (int i = 0; i < ops; ++i) {
    const int64_t n = 2500 + 13 * i;
    auto all = randomContribs(16, n, 400 + i);
    Vec out = all[0];
    std::vector<Vec> rest(all.begin() + 1, all.end());
    auto tr = table(rest);
    GroupPending pending;
    fake_hip_occupy(i % 2 ? callerStream : nullptr, 2);  // the producer is still busy
    gil.unlock();  // the binding lets go of the lock around the call
    CHECK(frg_allreduce_host(ctx, out.data(), tr.data(), 15, n, FRG_F32, FRG_SUM, FRG_SCALE_MUL,
                             1.f / 16, /*carry=*/1, i % 2 ? callerStream : nullptr, &onGroupDone,
                             &pending, nullptr) == FRG_OK);
    gil.lock();
    gil.unlock();  // Work.wait lets go of it as well
    while (pending.done.load() == 0) std::this_thread::yield();
    gil.lock();
    CHECK(hipStreamSynchronize(static_cast<hipStream_t>(pending.stream.load())) == hipSuccess);
    CHECK(same(out, fold(all, FRG_SCALE_MUL, 1.f / 16)));
  }
  gil.unlock();
  CHECK(frg_destroy(ctx) == FRG_OK);
}

void scenarioBlockStreamGivesUp() {
  std::puts("blocking a stream on an operation gives up like a wait does");
  frg_ctx* ctx = makeCtx(16384, 4096, 2, 1024);
  auto c = randomContribs(4, 5000, 78);
  Vec out(5000);
  auto t = table(c);
  // hold the command thread up: it queries and waits on the producer's event,
  // then launches, only after a stalled operation ahead of it is through
  hipStream_t consumer;
  CHECK(hipStreamCreateWithFlags(&consumer, hipStreamNonBlocking) == hipSuccess);
  CHECK(frg_set_wait_timeout(0.2) == FRG_OK);
  std::atomic<int> release{0};
  struct Held {
    std::atomic<int>* release;
  } held{&release};
  // an operation whose completion callback blocks the command thread for a while
  auto blocker = [](void* user, int, void*) {
    auto* h = static_cast<Held*>(user);
    while (h->release->load() == 0) std::this_thread::sleep_for(std::chrono::milliseconds(1));
  };
  Vec out0(5000);
  CHECK(frg_allreduce(ctx, out0.data(), t.data(), 4, 5000, FRG_F32, FRG_SUM, FRG_SCALE_NONE, 1.f,
                      nullptr, blocker, &held, nullptr) == FRG_OK);
  frg_work* w = nullptr;
  CHECK(frg_allreduce(ctx, out.data(), t.data(), 4, 5000, FRG_F32, FRG_SUM, FRG_SCALE_NONE, 1.f,
                      nullptr, nullptr, nullptr, &w) == FRG_OK);
  CHECK(frg_work_block_stream(w, consumer) == FRG_ERR_NOT_READY);
  CHECK(std::strstr(frg_last_error(), "gave up after") != nullptr);
  release = 1;
  CHECK(frg_set_wait_timeout(0) == FRG_OK);
  CHECK(frg_work_block_stream(w, consumer) == FRG_OK);
  CHECK(hipStreamSynchronize(consumer) == hipSuccess);
  CHECK(same(out, fold(c, FRG_SCALE_NONE, 1.f)));
  frg_work_release(w);
  CHECK(frg_destroy(ctx) == FRG_OK);
}

struct CallbackState {
  std::atomic<int> calls{0};
  std::atomic<int> status{-1};
  std::atomic<void*> stream{nullptr};
};

void onDone(void* user, int status, void* lastStream) {
  auto* s = static_cast<CallbackState*>(user);
  s->status = status;
  s->stream = lastStream;
  s->calls++;
}

void scenarioCallback() {
  std::puts("completion callback: once per operation, ordered on the last stream");
  frg_ctx* ctx = makeCtx(8192, 4096, 3, 512);
  auto c = randomContribs(4, 9001, 5);
  Vec out(9001, -1.f);
  auto t = table(c);
  CallbackState st;
  CHECK(frg_allreduce(ctx, out.data(), t.data(), 4, 9001, FRG_F32, FRG_SUM, FRG_SCALE_NONE, 1.f,
                      nullptr, &onDone, &st, nullptr) == FRG_OK);
  while (st.calls.load() == 0) std::this_thread::yield();
  CHECK(st.status.load() == FRG_OK && st.stream.load() != nullptr);
  // everything the operation launched is ordered before the end of that one stream
  CHECK(hipStreamSynchronize(static_cast<hipStream_t>(st.stream.load())) == hipSuccess);
  CHECK(same(out, fold(c, FRG_SCALE_NONE, 1.f)));
  CHECK(frg_synchronize(ctx) == FRG_OK);
  CHECK(st.calls.load() == 1);
  CHECK(frg_destroy(ctx) == FRG_OK);

  // the same through the host-staged path as a process group drives it: the
  // rank's own term already in `out`, 15 peers staged through 2 slots, several
  // operations in flight, completion known through the callback alone
  ctx = makeCtx(2 * 4096, 4096, 0, 0);
  const int ops = 6;
  std::vector<std::vector<Vec>> all, rests(ops);
  std::vector<Vec> outs(ops);
  std::vector<CallbackState> sts(ops);
  for (int i = 0; i < ops; ++i) {
    const int64_t n = 5000 + 11 * i;
    all.push_back(randomContribs(16, n, 300 + i));
    outs[i] = all[i][0];
    rests[i].assign(all[i].begin() + 1, all[i].end());
    auto tr = table(rests[i]);
    CHECK(frg_allreduce_host(ctx, outs[i].data(), tr.data(), 15, n, FRG_F32, FRG_SUM,
                             FRG_SCALE_NONE, 1.f, /*carry=*/1, nullptr, &onDone, &sts[i],
                             nullptr) == FRG_OK);
  }
  for (int i = 0; i < ops; ++i) {
    while (sts[i].calls.load() == 0) std::this_thread::yield();
    CHECK(sts[i].status.load() == FRG_OK);
    CHECK(hipStreamSynchronize(static_cast<hipStream_t>(sts[i].stream.load())) == hipSuccess);
    CHECK(same(outs[i], fold(all[i], FRG_SCALE_NONE, 1.f)));
  }
  CHECK(frg_synchronize(ctx) == FRG_OK);
  CHECK(frg_destroy(ctx) == FRG_OK);
}

void scenarioErrors() {
  std::puts("error paths: injected HIP failures, contract violations");
  frg_ctx* ctx = makeCtx(8192, 4096, 2, 0);
  auto c = randomContribs(3, 3000, 9);
  Vec out(3000);
  auto t = table(c);
  frg_work* w = nullptr;
  // a copy fails while the command thread enqueues: the work reports it, the context lives on
  fake_hip_fail_call("hipMemcpyAsync", 2);
  CallbackState st;
  CHECK(frg_allreduce_host(ctx, out.data(), t.data(), 3, 3000, FRG_F32, FRG_SUM, FRG_SCALE_NONE,
                           1.f, 0, nullptr, &onDone, &st, &w) == FRG_OK);
  CHECK(frg_work_wait(w) == FRG_ERR_HIP);
  CHECK(std::strstr(frg_last_error(), "HIP error") != nullptr);
  while (st.calls.load() == 0) std::this_thread::yield();
  CHECK(st.status.load() == FRG_ERR_HIP);
  frg_work_release(w);
  CHECK(frg_allreduce_host(ctx, out.data(), t.data(), 3, 3000, FRG_F32, FRG_SUM, FRG_SCALE_NONE,
                           1.f, 0, nullptr, nullptr, nullptr, &w) == FRG_OK);
  CHECK(frg_work_wait(w) == FRG_OK);
  CHECK(same(out, fold(c, FRG_SCALE_NONE, 1.f)));
  frg_work_release(w);
  // recording the initial event fails on the caller's thread: the call itself reports it
  // (the producer's stream must be busy: nothing is recorded on a stream that has drained)
  fake_hip_occupy(nullptr, 50);
  fake_hip_fail_call("hipEventRecord", 1);
  CHECK(frg_allreduce(ctx, out.data(), t.data(), 3, 3000, FRG_F32, FRG_SUM, FRG_SCALE_NONE, 1.f,
                      nullptr, nullptr, nullptr, &w) == FRG_ERR_HIP);
  CHECK(w == nullptr);
  // contract violations
  CHECK(frg_allreduce(ctx, out.data(), t.data(), 0, 3000, FRG_F32, FRG_SUM, 0, 1.f, nullptr,
                      nullptr, nullptr, nullptr) == FRG_ERR_INVALID);
  CHECK(frg_allreduce(ctx, out.data(), t.data(), 3, 3000, 42, FRG_SUM, 0, 1.f, nullptr, nullptr,
                      nullptr, nullptr) == FRG_ERR_UNSUPPORTED);
  CHECK(frg_allreduce(ctx, out.data(), t.data(), 3, 3000, FRG_F32, 5, 0, 1.f, nullptr, nullptr,
                      nullptr, nullptr) == FRG_ERR_UNSUPPORTED);
  CHECK(frg_allreduce(ctx, out.data(), t.data(), 3, 3000, FRG_F32, FRG_MAX, FRG_SCALE_MUL, .5f,
                      nullptr, nullptr, nullptr, nullptr) == FRG_ERR_INVALID);
  CHECK(frg_allreduce(ctx, nullptr, t.data(), 3, 3000, FRG_F32, FRG_SUM, 0, 1.f, nullptr,
                      nullptr, nullptr, nullptr) == FRG_ERR_INVALID);
  CHECK(frg_allreduce(ctx, out.data(), t.data(), 3, 0, FRG_F32, FRG_SUM, 0, 1.f, nullptr, nullptr,
                      nullptr, &w) == FRG_OK);  // empty: completes, nothing launched
  CHECK(frg_work_wait(w) == FRG_OK);
  frg_work_release(w);
  CHECK(frg_destroy(ctx) == FRG_OK);
  // creation failures
  frg_options o = {};
  o.max_memory_allocated_in_bytes = 1000;
  o.slice_size_in_bytes = 4096;
  frg_ctx* bad = nullptr;
  CHECK(frg_create(0, &o, &bad) == FRG_ERR_LAYOUT && bad == nullptr);
  o.max_memory_allocated_in_bytes = 8192;
  fake_hip_fail_call("hipMalloc", 1);
  CHECK(frg_create(0, &o, &bad) == FRG_ERR_HIP && bad == nullptr);
  // a failure after the staging pool exists: released once, nothing else left behind
  fake_hip_fail_call("hipMalloc", 2);  // the chain scratch
  CHECK(frg_create(0, &o, &bad) == FRG_ERR_HIP && bad == nullptr);
  CHECK(frg_create(7, &o, &bad) == FRG_ERR_INVALID);
}

void scenarioProfiling() {
  std::puts("profile marks and per-launch records");
  frg_ctx* ctx = makeCtx(8192, 4096, 2, 1024);
  auto c = randomContribs(8, 4096, 3);
  Vec out(4096);
  auto t = table(c);
  CHECK(frg_profile_mark(ctx) == FRG_OK);
  for (int i = 0; i < 3; ++i) {
    CHECK(frg_allreduce(ctx, out.data(), t.data(), 8, 4096, FRG_F32, FRG_SUM, 0, 1.f, nullptr,
                        nullptr, nullptr, nullptr) == FRG_OK);
  }
  CHECK(frg_profile_mark(ctx) == FRG_OK);
  frg_launch_record recs[64];
  int n = 0;
  CHECK(frg_launch_records(ctx, recs, 64, &n) == FRG_OK);
  CHECK(n == 2);  // one region, two reduce streams
  int64_t launches = 0, elems = 0;
  for (int i = 0; i < n; ++i) {
    CHECK(recs[i].end_ms >= recs[i].begin_ms && recs[i].num_contributions == 8);
    launches += recs[i].launches;
    elems += recs[i].numel;
  }
  CHECK(launches == 3 * 16 && elems == 3 * 4096);  // 4 slices x 4 launches of 256 elements
  CHECK(frg_set_profiling(ctx, 1) == FRG_OK);
  CHECK(frg_allreduce(ctx, out.data(), t.data(), 8, 4096, FRG_F32, FRG_SUM, 0, 1.f, nullptr,
                      nullptr, nullptr, nullptr) == FRG_OK);
  float ms[64];
  CHECK(frg_kernel_times(ctx, ms, 64, &n) == FRG_OK && n == 16);
  for (int i = 0; i < n; ++i) CHECK(ms[i] >= 0.f);
  CHECK(frg_set_profiling(ctx, 0) == FRG_OK);
  CHECK(frg_destroy(ctx) == FRG_OK);
}

void scenarioDestroyWithPendingWork() {
  std::puts("destroy drains what was submitted");
  frg_ctx* ctx = makeCtx(8192, 4096, 2, 1024);
  auto c = randomContribs(8, 50000, 11);
  Vec out(50000, -1.f);
  auto t = table(c);
  fake_hip_occupy(nullptr, 30);
  frg_work* w = nullptr;
  CHECK(frg_allreduce(ctx, out.data(), t.data(), 8, 50000, FRG_F32, FRG_SUM, 0, 1.f, nullptr,
                      nullptr, nullptr, &w) == FRG_OK);
  CHECK(frg_destroy(ctx) == FRG_OK);  // no wait before it
  CHECK(same(out, fold(c, FRG_SCALE_NONE, 1.f)));
  CHECK(frg_work_wait(w) == FRG_OK);  // the handle outlives the context
  frg_work_release(w);
}

void concurrentSubmitters(frg_ctx* ctx);

void scenarioConcurrentSubmitters() {
  std::puts("several threads submit to one context");
  concurrentSubmitters(makeCtx(8192, 4096, 2, 1024));
  // the same with the library's own partition, small operations on the callers'
  // streams and neighbours joined: whatever path an operation takes
  setenv("FAIRRING_INLINE_BYTES", "65536", 1);
  frg_ctx* ctx = makeCtx(8192, 4096, 2, 0);
  setenv("FAIRRING_INLINE_BYTES", "0", 1);
  concurrentSubmitters(ctx);
}

void concurrentSubmitters(frg_ctx* ctx) {
  std::vector<std::thread> threads;
  std::atomic<int> ok{0};
  for (int tix = 0; tix < 4; ++tix) {
    threads.emplace_back([ctx, tix, &ok] {
      for (int i = 0; i < 25; ++i) {
        auto c = randomContribs(3, 2000 + i, 1000 * tix + i);
        Vec out(c[0].size());
        auto t = table(c);
        frg_work* w = nullptr;
        CHECK(frg_allreduce(ctx, out.data(), t.data(), 3, static_cast<int64_t>(out.size()),
                            FRG_F32, FRG_SUM, 0, 1.f, nullptr, nullptr, nullptr, &w) == FRG_OK);
        CHECK(frg_work_wait(w) == FRG_OK);
        CHECK(same(out, fold(c, FRG_SCALE_NONE, 1.f)));
        frg_work_release(w);
        ok++;
      }
    });
  }
  for (auto& th : threads) th.join();
  CHECK(ok.load() == 100);
  CHECK(frg_destroy(ctx) == FRG_OK);
}

// Ends the process when a scenario stops making progress, with its name, so
// that a cycle of waits shows as a failure rather than as a run that never ends.
std::atomic<long> gScenarioTicks{0};
const char* volatile gScenarioName = "start-up";

int gStallLimitSeconds = 150;

void watchdog() {
  long seen = -1;
  int stale = 0;
  for (;;) {
    std::this_thread::sleep_for(std::chrono::seconds(1));
    const long now = gScenarioTicks.load();
    stale = now == seen ? stale + 1 : 0;
    seen = now;
    if (stale > gStallLimitSeconds) {
      std::fprintf(stderr, "no progress for %d s in scenario: %s\n", gStallLimitSeconds,
                   gScenarioName);
      std::abort();
    }
  }
}

void runAll() {
  struct Scenario {
    const char* name;
    void (*fn)();
  };
  const Scenario all[] = {
      {"resident", scenarioResident},
      {"aligned launch plan", scenarioWholeRoundPlan},
      {"launch partition", scenarioLaunchPartition},
      {"pre-scale and compressed", scenarioPreScaleAndCompressed},
      {"busy producer", scenarioBusyProducer},
      {"wait gives up", scenarioWaitGivesUp},
      {"block stream gives up", scenarioBlockStreamGivesUp},
      {"idle producer", scenarioIdleProducer},
      {"neighbours run as one", scenarioNeighboursRunAsOne},
      {"the null stream remembers its waits", scenarioNullStreamRemembersItsWaits},
      {"small operations on the caller's stream", scenarioSmallOperationsOnTheCallersStream},
      {"producer ordering", scenarioProducerOrdering},
      {"mixed loads rule", scenarioMixedLoadsRule},
      {"streams are reused", scenarioStreamsAreReused},
      {"order between operations", scenarioOrderBetweenOperations},
      {"random dependent operations", scenarioRandomDependentOperations},
      {"host staged", scenarioHostStaged},
      {"gathered contribution", scenarioGathered},
      {"callback", scenarioCallback},
      {"process-group-shaped", scenarioProcessGroupShaped},
      {"errors", scenarioErrors},
      {"profiling", scenarioProfiling},
      {"destroy with pending work", scenarioDestroyWithPendingWork},
      {"concurrent submitters", scenarioConcurrentSubmitters},
  };
  for (const Scenario& sc : all) {
    gScenarioName = sc.name;
    gScenarioTicks++;
    sc.fn();
    gScenarioTicks++;
  }
}

}  // namespace

// With the argument "latest-record-waits" every scenario runs on a runtime whose
// stream waits bind to the record their event holds when the wait packet is
// executed (not what HIP does): what the pipeline makes of that shows how much
// it leans on re-recording an event while a wait on it is pending.
int main(int argc, char** argv) {
  std::setvbuf(stdout, nullptr, _IOLBF, 0);  // a run that is aborted still shows how far it got
  // every scenario but the one about them sends its small operations through the pipeline
  setenv("FAIRRING_INLINE_BYTES", "0", 1);
  if (const char* limit = std::getenv("HOST_TEST_STALL_SECONDS")) gStallLimitSeconds = std::atoi(limit);
  if (argc > 1 && std::string(argv[1]) == "latest-record-waits") {
    std::puts("== stream waits bind to their event's latest record");
    fake_hip_set_latest_record_waits(1);
  }
  std::thread(watchdog).detach();
  // HOST_TEST_TOPOLOGY = "own", "4" or "1" runs one of the three topologies only
  // (the slow sanitizer builds do: a data race does not depend on the topology).
  const char* only = std::getenv("HOST_TEST_TOPOLOGY");
  const std::string topology = only != nullptr ? only : "";
  if (topology.empty() || topology == "own") {
    std::puts("== every stream on a queue of its own");
    runAll();
  }
  // The shape of a GPU process with fewer hardware queues than streams: the
  // null stream, the reduce and copy streams of every context and the callers'
  // side streams multiplexed onto 4 in-order queues, where a wait packet holds
  // up whatever sits behind it.
  if (topology.empty() || topology == "4") {
    std::puts("== all streams on 4 shared in-order hardware queues");
    fake_hip_set_hw_queues(4);
    gSharedHwQueues = true;
    runAll();
  }
  if (topology.empty() || topology == "1") {
    fake_hip_set_hw_queues(1);
    gSharedHwQueues = true;
    std::puts("== all streams on 1 shared in-order hardware queue");
    runAll();
  }
  std::puts("ALL HOST SCENARIOS PASSED");
  return 0;
}
