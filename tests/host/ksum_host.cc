// Test build only: stands in for fairring_amd/csrc/ksum_kernels.hip when the
// pipeline is compiled against the fake HIP runtime. The "kernel" is a plain
// fp32 fold run as one unit of work on the fake stream, so the choreography
// around it (ordering, slot reuse, carry chains) decides whether results come
// out right. fp32 only, plus a bf16 stand-in of the reduction with compression
// folded in.
#include <hip/hip_runtime.h>

#include <atomic>

#include <cstring>
#include <vector>

#include "../../fairring_amd/csrc/ksum_kernels.h"
#include "../../include/fairring_hip.h"

namespace frg {

int64_t elementSize(int dtype) {
  switch (dtype) {
    case FRG_F32:
    case FRG_I32:
      return 4;
    case FRG_BF16:
    case FRG_F16:
      return 2;
    case FRG_F64:
    case FRG_I64:
      return 8;
    case FRG_U8:
    case FRG_I8:
      return 1;
    default:
      return 0;
  }
}

bool isFloating(int dtype) {
  return dtype == FRG_F32 || dtype == FRG_BF16 || dtype == FRG_F16 || dtype == FRG_F64;
}

void setTuning(int) {}

void setXcdChunkShift(int) {}
void setMixedLoads(int) {}

int computeUnits(int) { return 4; }  // what the stand-in runtime reports

void prepareStaticScratch(int) {}  // device code: not part of the host build

namespace {

struct Job {
  float* out;
  const float* carrySrc;
  std::vector<const float*> in;
  int64_t n;
  int op;
  int scaleMode;
  float scale;
  bool carry;
};

void runJob(void* p) {
  Job* j = static_cast<Job*>(p);
  for (int64_t i = 0; i < j->n; ++i) {
    const bool preMul = j->scaleMode == FRG_SCALE_PRE_MUL, preDiv = j->scaleMode == FRG_SCALE_PRE_DIV;
    auto term = [&](size_t kk) {
      const float x = j->in[kk][i];
      return preMul ? x * j->scale : (preDiv ? x / j->scale : x);
    };
    size_t k = 0;
    float acc = j->carry ? j->carrySrc[i] : term(k++);
    for (; k < j->in.size(); ++k) {
      const float b = term(k);
      if (j->op == FRG_SUM) {
        acc = acc + b;
      } else {
        acc = (acc != acc) ? acc : ((b != b) ? b : (acc > b ? acc : b));
      }
    }
    if (j->scaleMode == FRG_SCALE_MUL) acc = acc * j->scale;
    if (j->scaleMode == FRG_SCALE_DIV) acc = acc / j->scale;
    j->out[i] = acc;
  }
  delete j;
}

// bf16 helpers of the compressed stand-in
float widen(uint16_t b) {
  const uint32_t u = static_cast<uint32_t>(b) << 16;
  float f;
  std::memcpy(&f, &u, 4);
  return f;
}

uint16_t narrow(float f) {
  uint32_t u;
  std::memcpy(&u, &f, 4);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0;
  return static_cast<uint16_t>((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}

struct CompressedJob {
  void* out;
  bool out32;
  std::vector<const void*> in;
  int rawIndex;
  int64_t n;
  int scaleMode;
  float scale;
  std::vector<RawPiece> pieces;  // the raw term in tensors of its own, when given
};

// the raw term of element i
float rawAt(const CompressedJob* j, int64_t i) {
  if (j->pieces.empty()) return static_cast<const float*>(j->in[static_cast<size_t>(j->rawIndex)])[i];
  size_t s = 0;
  while (s + 1 < j->pieces.size() && i >= j->pieces[s + 1].off) ++s;
  return static_cast<const float*>(j->pieces[s].ptr)[i - j->pieces[s].off];
}

void runCompressedJob(void* p) {
  CompressedJob* j = static_cast<CompressedJob*>(p);
  for (int64_t i = 0; i < j->n; ++i) {
    float acc = 0.0f;
    for (size_t k = 0; k < j->in.size(); ++k) {
      float t;
      if (static_cast<int>(k) == j->rawIndex) {
        t = widen(narrow(rawAt(j, i)));
        if (j->scaleMode == FRG_SCALE_MUL) t = widen(narrow(t * j->scale));
        if (j->scaleMode == FRG_SCALE_DIV) t = widen(narrow(t / j->scale));
      } else {
        t = widen(static_cast<const uint16_t*>(j->in[k])[i]);
      }
      acc = k == 0 ? t : acc + t;
    }
    if (j->out32) {
      static_cast<float*>(j->out)[i] = widen(narrow(acc));
    } else {
      static_cast<uint16_t*>(j->out)[i] = narrow(acc);
    }
  }
  delete j;
}

}  // namespace

int launchCompressedReduce(const CompressedArgs& a, hipStream_t stream, std::string* err) {
  auto fail = [&](int code, const char* msg) {
    if (err) *err = msg;
    return code;
  };
  if (a.wire_dtype != FRG_BF16) return fail(FRG_ERR_UNSUPPORTED, "host test build: bf16 wire only");
  if (a.K < 1 || a.K > kMaxContribsPerLaunch) return fail(FRG_ERR_INVALID, "K out of range");
  if (a.n == 0) return FRG_OK;
  if (a.num_raw_pieces > kMaxRawPiecesPerLaunch) return fail(FRG_ERR_INVALID, "too many raw pieces");
  CompressedJob* j = new CompressedJob{a.out, a.out_dtype == FRG_F32, {}, a.raw_index,
                                       a.n,   a.scale_mode,          a.scale, {}};
  for (int k = 0; k < a.K; ++k) j->in.push_back(a.contribs[k]);
  for (int i = 0; i < a.num_raw_pieces; ++i) j->pieces.push_back(a.raw_pieces[i]);
  fake_hip_enqueue(stream, &runCompressedJob, j);
  return FRG_OK;
}

// the real rule's core: every tensor starts where a group of 8 elements does, on a 16-byte boundary
bool rawPiecesVectorize(const void* out, int, const void* const*, int, int, const RawPiece* pieces,
                        int count, int64_t) {
  if (count < 1 || count > kMaxRawPiecesPerLaunch) return false;
  if (reinterpret_cast<uintptr_t>(out) % 16 != 0) return false;
  for (int i = 0; i < count; ++i) {
    if (pieces[i].off % 8 != 0 || reinterpret_cast<uintptr_t>(pieces[i].ptr) % 16 != 0) return false;
  }
  return true;
}

int launchReduce(const ReduceArgs& a, hipStream_t stream, std::string* err);

// Launches that asked for the mixed loads (the tests read it).
std::atomic<long long> gMixedLoadLaunches{0};
long long mixedLoadLaunches() { return gMixedLoadLaunches.load(); }

// The segmented launch: every piece as a unit of work of its own, in order (the
// packing into launches and the cuts on tiles are the pipeline's and are what is
// under test; the real kernel's limits are checked here as it checks them).
int launchSegmented(const SegmentedArgs& a, hipStream_t stream, std::string* err) {
  auto fail = [&](int code, const char* msg) {
    if (err) *err = msg;
    return code;
  };
  if (!segmentedKind(a.K, a.dtype, FRG_SUM, false)) return fail(FRG_ERR_UNSUPPORTED, "not a segmented kind");
  if (a.numPieces < 0 || a.numPieces > maxSegmentsPerLaunch(a.K)) return fail(FRG_ERR_INVALID, "too many pieces");
  for (int i = 0; i < a.numPieces; ++i) {
    const SegPiece& pc = a.pieces[i];
    if (pc.n == 0) continue;
    if (!segmentable(pc.out, pc.contribs, a.K, elementSize(a.dtype))) {
      return fail(FRG_ERR_INVALID, "piece not congruent modulo 16");
    }
    ReduceArgs r;
    r.out = pc.out;
    r.contribs = pc.contribs;
    r.K = a.K;
    r.n = pc.n;
    r.dtype = a.dtype;
    r.op = FRG_SUM;
    r.scale_mode = a.scale_mode;
    r.scale = a.scale;
    const int rc = launchReduce(r, stream, err);
    if (rc != FRG_OK) return rc;
  }
  return FRG_OK;
}

int launchReduce(const ReduceArgs& a, hipStream_t stream, std::string* err) {
  auto fail = [&](int code, const char* msg) {
    if (err) *err = msg;
    return code;
  };
  if (a.dtype != FRG_F32) return fail(FRG_ERR_UNSUPPORTED, "host test build reduces fp32 only");
  if (a.op != FRG_SUM && a.op != FRG_MAX) return fail(FRG_ERR_UNSUPPORTED, "unsupported op");
  if (a.K < 1 || a.K > kMaxContribsPerLaunch) return fail(FRG_ERR_INVALID, "K out of range");
  if (a.n < 0) return fail(FRG_ERR_INVALID, "negative element count");
  if (a.n == 0) return FRG_OK;
  if (a.out == nullptr || a.contribs == nullptr) return fail(FRG_ERR_INVALID, "null pointer");
  Job* j = new Job{static_cast<float*>(a.out),
                   static_cast<const float*>(a.carry_src ? a.carry_src : a.out),
                   {},
                   a.n,
                   a.op,
                   a.scale_mode,
                   a.scale,
                   a.carry};
  for (int k = 0; k < a.K; ++k) j->in.push_back(static_cast<const float*>(a.contribs[k]));
  if (a.mixed_loads) gMixedLoadLaunches.fetch_add(1);
  if (a.startEvent) hipEventRecord(a.startEvent, stream);
  fake_hip_enqueue(stream, &runJob, j);
  if (a.stopEvent) hipEventRecord(a.stopEvent, stream);
  return FRG_OK;
}

}  // namespace frg
