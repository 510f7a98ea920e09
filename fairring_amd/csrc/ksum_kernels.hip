// K-way elementwise reduction of gradient slices for MI355X (gfx950, CDNA4).
//
// Stands in for the two places where the reference reduces a slice:
//   * doReduction, fairring/device.cc:108-131: at::sum_out / at::amax_out over
//     dim 0 of operand[K, n] (server-side accumulation of per-machine shards);
//   * the arithmetic inside ncclReduceScatter, fairring/device.cc:33-70 (the
//     local reduction over the devices of a machine).
//
// The work is HBM-bound (K reads + 1 write per element, K-1 adds), so the
// kernel is a pure streaming design: every lane owns one 16-byte vector per
// contribution, all K loads are issued before the first add so K x 16 B per
// lane are in flight, the adds run strictly in contribution order in fp32
// registers, the optional post-scale and the bf16 rounding are fused into the
// store, and nothing goes through LDS. Addresses are a uniform 64-bit base
// (SGPRs) plus a 32-bit lane offset, so a wave's load covers 1 KiB of
// consecutive bytes. Loads and stores are non-temporal: no byte is reused.
//
// Bit-exactness rules: no FMA contraction, no reassociation, no packed-fp32
// instructions (build flags), IEEE division for FRG_SCALE_DIV, fp32 denormals
// kept.

#include "ksum_kernels.h"

#include <hip/hip_ext.h>
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdlib>

#include "../../include/fairring_hip.h"
#include "device_traits.h"

namespace frg {
namespace {

// log2 of the tiles in a row that the blocks of one XCD take (0: every eighth tile).
int gXcdChunkShift = 6;

// Which launches take the mixed form of the main loop (reduceTileMixed): -1 those
// whose ReduceArgs ask for it, 0 none, 1 every launch that has the form.
int gMixedLoads = -1;

bool wantsMixedLoads(const ReduceArgs& a) {
  return gMixedLoads < 0 ? a.mixed_loads : gMixedLoads > 0;
}

// Loads N contributions [k0, k0+N) at (base + lane), then folds them into acc
// in index order. `first` makes contribution k0 initialise acc instead. With a
// pre-scale (`pre` = FRG_SCALE_PRE_MUL / FRG_SCALE_PRE_DIV) every term is
// scaled and rounded to the storage type before it is folded in.
template <typename TR, int OP, int N, typename PT>
__device__ __forceinline__ void foldChunk(typename TR::acc_t (&acc)[TR::kLanes], const PT& in,
                                          int k0, int64_t elemBase,
                                          unsigned int laneBytes, bool first, int pre,
                                          typename TR::acc_t preScale) {
  using vec_t = typename TR::vec_t;
  using elem_t = typename TR::elem_t;
  vec_t v[N];
#pragma unroll
  for (int k = 0; k < N; ++k) {
    // uniform 64-bit base + 32-bit byte offset of the lane
    const char* b = reinterpret_cast<const char*>(
        static_cast<const elem_t*>(in.p[k0 + k]) + elemBase);
    v[k] = ldStream(reinterpret_cast<const vec_t*>(b + laneBytes));
  }
#pragma unroll
  for (int k = 0; k < N; ++k) {
    typename TR::acc_t f[TR::kLanes];
    TR::unpack(v[k], f);
    if constexpr (TR::kFloating) {
      if (pre == FRG_SCALE_PRE_MUL) {
#pragma unroll
        for (int j = 0; j < TR::kLanes; ++j) f[j] = TR::roundStorage(f[j] * preScale);
      } else if (pre == FRG_SCALE_PRE_DIV) {
#pragma unroll
        for (int j = 0; j < TR::kLanes; ++j) f[j] = TR::roundStorage(f[j] / preScale);
      }
    }
    if (k == 0 && first) {
#pragma unroll
      for (int j = 0; j < TR::kLanes; ++j) acc[j] = f[j];
    } else {
#pragma unroll
      for (int j = 0; j < TR::kLanes; ++j) acc[j] = combine<OP>(acc[j], f[j]);
    }
  }
}

// SC values of the variants that scale every term before the fold; they are
// compiled apart so that the multiply / IEEE division per term does not weigh
// on the plain variants.
constexpr int kPreMul = -2;
constexpr int kPreDiv = -3;
// SC value of the variant of the 2-byte floating types that can take the
// carried-in term from, and leave its result in, a buffer of fp32 accumulators
// (accFlags): a chain of launches over more contributions than one launch
// takes then rounds once, at its end, like a single launch. Any scale mode.
constexpr int kAccIo = -4;
constexpr int kCarryIsAcc = 1;
constexpr int kOutIsAcc = 2;

// One vector of the output: out = scale(carry? (+) in[0] (+) ... (+) in[K-1]).
// SC >= 0 fixes the scale mode at compile time and rules out a carry: the hot
// variants then hold nothing but loads, adds, one multiply and the store (a
// third of the code, which matters when a launch lasts 10 us and every CU
// starts it with a cold instruction cache).
template <typename TR, int OP, int KT, int SC, typename PT>
__device__ __forceinline__ void reduceOne(typename TR::elem_t* out,
                                          const PT& in, int K,
                                          const typename TR::elem_t* carrySrc,
                                          int scaleMode, float scale, int accFlags,
                                          int64_t elemBase, unsigned int lane) {
  if (SC >= 0) {
    carrySrc = nullptr;
    scaleMode = SC;
  }
  using vec_t = typename TR::vec_t;
  const unsigned int laneBytes = lane * static_cast<unsigned int>(sizeof(vec_t));
  vec_t* o = reinterpret_cast<vec_t*>(reinterpret_cast<char*>(out + elemBase) + laneBytes);
  typename TR::acc_t acc[TR::kLanes];
  bool first = true;
  constexpr int preC = SC == kPreMul ? FRG_SCALE_PRE_MUL : (SC == kPreDiv ? FRG_SCALE_PRE_DIV : 0);
  const int pre = SC == kAccIo ? (scaleMode >= FRG_SCALE_PRE_MUL ? scaleMode : 0) : preC;
  const typename TR::acc_t preScale = static_cast<typename TR::acc_t>(scale);
  vec_t c;
  const bool carry = carrySrc != nullptr;
  // the carried-in term (normally `out` itself): issued before the contribution
  // loads, consumed first
  bool carryLoaded = false;
  if constexpr (SC == kAccIo) {
    if (carry && (accFlags & kCarryIsAcc)) {
      using Side = Fp32Side<TR::kLanes>;
      const typename Side::regs_t r =
          Side::load(reinterpret_cast<const float*>(carrySrc) + elemBase, lane);
      Side::unpack(r, acc);
      first = false;
      carryLoaded = true;
    }
  }
  if (carry && !carryLoaded) {
    c = *reinterpret_cast<const vec_t*>(reinterpret_cast<const char*>(carrySrc + elemBase) +
                                        laneBytes);
  }
  if (KT > 0) {
    if (carry && !carryLoaded) {
      TR::unpack(c, acc);
      first = false;
    }
    foldChunk<TR, OP, (KT > 0 ? KT : 1)>(acc, in, 0, elemBase, laneBytes, first, pre, preScale);
  } else {
    if (carry && !carryLoaded) {
      TR::unpack(c, acc);
      first = false;
    }
    int k = 0;
    for (; k + kChunk <= K; k += kChunk) {
      foldChunk<TR, OP, kChunk>(acc, in, k, elemBase, laneBytes, first, pre, preScale);
      first = false;
    }
    // what is left (1..7 contributions) is loaded in one go as well
    switch (K - k) {
      case 7: foldChunk<TR, OP, 7>(acc, in, k, elemBase, laneBytes, first, pre, preScale); break;
      case 6: foldChunk<TR, OP, 6>(acc, in, k, elemBase, laneBytes, first, pre, preScale); break;
      case 5: foldChunk<TR, OP, 5>(acc, in, k, elemBase, laneBytes, first, pre, preScale); break;
      case 4: foldChunk<TR, OP, 4>(acc, in, k, elemBase, laneBytes, first, pre, preScale); break;
      case 3: foldChunk<TR, OP, 3>(acc, in, k, elemBase, laneBytes, first, pre, preScale); break;
      case 2: foldChunk<TR, OP, 2>(acc, in, k, elemBase, laneBytes, first, pre, preScale); break;
      case 1: foldChunk<TR, OP, 1>(acc, in, k, elemBase, laneBytes, first, pre, preScale); break;
      default: break;
    }
  }
  if constexpr (SC == kAccIo) {
    if (accFlags & kOutIsAcc) {
      // parked unrounded and unscaled for the next launch of the chain
      Fp32Side<TR::kLanes>::store(reinterpret_cast<float*>(out) + elemBase, lane, acc);
      return;
    }
  }
  if constexpr (TR::kFloating && preC == 0) {
    if (OP == FRG_SUM) {
      // in the accumulator's precision: fp32, or fp64 for fp64 data
      const typename TR::acc_t sc = static_cast<typename TR::acc_t>(scale);
      if (scaleMode == FRG_SCALE_MUL) {
#pragma unroll
        for (int j = 0; j < TR::kLanes; ++j) acc[j] = acc[j] * sc;
      } else if (scaleMode == FRG_SCALE_DIV) {
#pragma unroll
        for (int j = 0; j < TR::kLanes; ++j) acc[j] = acc[j] / sc;
      }
    }
  }
  stStream(TR::pack(acc), o);
}

// A lane's two vectors of a tile (kUnroll = 2; they lie 2 KiB apart) reduced
// together, with the loads of both mixed: a first batch of KT loads takes the
// lower half of the contributions at the first vector and the upper half at
// the second, a second batch, issued once the first has landed, the rest. So
// the loads a wave has in flight at any one time do not all sit at the same
// position within 4 KiB. That matters when the contributions do: a bucket's
// tensors that are allocations of their own all start their allocation, and
// run through memory in step. The fold of each vector is still contribution 0
// to KT-1 in order; all loads come before both stores, so an output that is one
// of the contributions is read before it is written, as in reduceOne.
template <typename TR, int KT, int SC>
__device__ __forceinline__ void reduceTileMixed(typename TR::elem_t* out, const Ptrs<KT>& in,
                                                float scale, int64_t elemBase, unsigned int tid) {
  static_assert(kUnroll == 2 && KT >= 2 && KT % 2 == 0, "two vectors per lane, halves of KT");
  using vec_t = typename TR::vec_t;
  using elem_t = typename TR::elem_t;
  using acc_t = typename TR::acc_t;
  constexpr int H = KT / 2;
  const unsigned int laneBytes[2] = {tid * static_cast<unsigned int>(sizeof(vec_t)),
                                     (tid + kBlock) * static_cast<unsigned int>(sizeof(vec_t))};
  auto ld = [&](int k, int u) {
    const char* p = reinterpret_cast<const char*>(static_cast<const elem_t*>(in.p[k]) + elemBase);
    const vec_t v = ldStream(reinterpret_cast<const vec_t*>(p + laneBytes[u]));
    asm volatile("" ::: "memory");  // the loads stay in the order written
    return v;
  };
  vec_t v0[KT], v1[KT];  // the lane's first and second vector of every contribution
#pragma unroll
  for (int k = 0; k < H; ++k) v0[k] = ld(k, 0);
#pragma unroll
  for (int k = H; k < KT; ++k) v1[k] = ld(k, 1);
  // The second batch only when the first has landed: KT loads per wave in
  // flight, as in the loop that takes one vector after the other (with all 2 KT
  // issued at once the 8-way fp32 sum lost 1.5 to 2 %).
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
  for (int k = 0; k < H; ++k) {
    v0[H + k] = ld(H + k, 0);
    v1[k] = ld(k, 1);
  }
  const acc_t sc = static_cast<acc_t>(scale);
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    acc_t acc[TR::kLanes];
#pragma unroll
    for (int k = 0; k < KT; ++k) {
      acc_t f[TR::kLanes];
      TR::unpack(u == 0 ? v0[k] : v1[k], f);
      if constexpr (TR::kFloating && SC == kPreMul) {
        // every term scaled and rounded to the storage type first, as in foldChunk
#pragma unroll
        for (int j = 0; j < TR::kLanes; ++j) f[j] = TR::roundStorage(f[j] * sc);
      }
#pragma unroll
      for (int j = 0; j < TR::kLanes; ++j) acc[j] = k == 0 ? f[j] : combine<FRG_SUM>(acc[j], f[j]);
    }
    if constexpr (TR::kFloating && SC == FRG_SCALE_MUL) {
#pragma unroll
      for (int j = 0; j < TR::kLanes; ++j) acc[j] = acc[j] * sc;
    }
    stStream(TR::pack(acc),
             reinterpret_cast<vec_t*>(reinterpret_cast<char*>(out + elemBase) + laneBytes[u]));
  }
}

// Whether a variant of the body kernel has the mixed form of its main loop.
template <typename TR, int OP, int KT, int SC>
constexpr bool kHasMixedLoads = OP == FRG_SUM && KT >= 2 && KT % 2 == 0 && kUnroll == 2 &&
                                (SC == FRG_SCALE_NONE || SC == FRG_SCALE_MUL ||
                                 (SC == kPreMul && TR::kFloating));

// Body kernel. The slice is [head scalars][nvec vectors][tail scalars], where
// `head` brings every pointer to a 16-byte boundary. The first `lead` vectors
// are dealt in pieces of their own, so that the tiles start on a 4 KiB
// boundary of the first contribution (or where the caller wants its rounds to
// start, ReduceArgs::lead_bytes): a wave's load then covers eight
// whole 128-byte lines instead of straddling nine (measured on MI355X, 8-way
// fp32: 6,465 GB/s from a 4 KiB boundary, 5,940 from 16 bytes past one). Full tiles of
// kBlock*kUnroll vectors are dealt to the blocks round-robin for as many whole
// rounds as there are. What is left (fewer tiles than blocks) is dealt in
// pieces of kBlock vectors, again from block 0 upwards: the hardware places
// blocks on CUs round-robin, so spreading the remainder over twice as many
// blocks in half-size pieces evens out the work per CU, and the launch does not
// end on a few CUs finishing a whole extra tile.
// MIXED: the whole tiles go through reduceTileMixed (a variant of its own, so
// that neither form carries the other's code).
template <typename TRV, typename TRS, int OP, int KT, int SC, bool MIXED = false>
__global__ void __launch_bounds__(kBlock)
    ksumKernel(typename TRV::elem_t* out, Ptrs<KT> in, int K,
               const typename TRV::elem_t* carrySrc,
               int scaleMode, float scale, int accFlags, int64_t head, int lead, int64_t nvec,
               int64_t tail, int64_t roundTiles, int64_t pieces, int chunkShift) {
  // roundTiles (tiles in whole rounds of the grid) and pieces (remainder pieces
  // of kBlock * FRG_REMAINDER_PIECE_UNROLL vectors) come from the host: a
  // 64-bit division by the grid size at the top of every wave is a third of a
  // microsecond that a 10 us launch does not have.
  constexpr int64_t kTile = static_cast<int64_t>(kBlock) * kUnroll;
  const int64_t grid = gridDim.x;
  const int64_t bodyBase = head + static_cast<int64_t>(lead) * TRV::kLanes;  // first tile's element
  const int64_t bodyVecs = nvec - lead;
  for (int64_t t0 = blockIdx.x; t0 < roundTiles; t0 += grid) {
    // Which tile the block takes in this round. The hardware deals blocks to
    // the 8 XCDs in turn, so with tile = block index every XCD reads every
    // eighth 4 KiB tile. Rotating the low three bits of the index up by
    // chunkShift gives the blocks of one XCD runs of 2^chunkShift consecutive
    // tiles instead (256 KiB at 6), while all blocks together still sweep the
    // same narrow front: measured on MI355X in a bare launch loop, 8-way fp32 on
    // two streams, 6,645 GB/s against 6,570 for launches of two rounds (runs of
    // 16 KiB to 128 KiB and of 512 KiB and more are no better than none). A
    // permutation within every aligned group of 8 << chunkShift tiles, whatever
    // the grid.
    int64_t t = t0;
    if (chunkShift > 0) {
      const int64_t low = (int64_t{1} << chunkShift) - 1;
      t = ((t0 >> (3 + chunkShift)) << (3 + chunkShift)) | ((t0 & 7) << chunkShift) |
          ((t0 >> 3) & low);
    }
    const int64_t elemBase = bodyBase + t * kTile * TRV::kLanes;
    if constexpr (SC == kAccIo) {
      // the largest body (every scale mode, both kinds of carry and output) and
      // the rarest: its two vectors per lane go one after the other
      for (int u = 0; u < kUnroll; ++u) {
        reduceOne<TRV, OP, KT, SC>(out, in, K, carrySrc, scaleMode, scale, accFlags, elemBase,
                                   threadIdx.x + u * kBlock);
      }
    } else if constexpr (MIXED) {
      reduceTileMixed<TRV, KT, SC>(out, in, scale, elemBase, threadIdx.x);
    } else {
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        reduceOne<TRV, OP, KT, SC>(out, in, K, carrySrc, scaleMode, scale, accFlags, elemBase,
                                   threadIdx.x + u * kBlock);
      }
    }
  }
  // remainder: pieces of kBlock * kPiece vectors, the last one possibly partial
  const int64_t restBase = roundTiles * kTile;
  constexpr int kPiece = FRG_REMAINDER_PIECE_UNROLL;  // vectors per lane in a remainder piece
  constexpr int64_t pieceVecs = static_cast<int64_t>(kBlock) * kPiece;
  for (int64_t p = blockIdx.x; p < pieces; p += grid) {
    const int64_t v0 = restBase + p * pieceVecs;
#pragma unroll
    for (int u = 0; u < kPiece; ++u) {
      const unsigned int lane = threadIdx.x + u * kBlock;
      if (v0 + lane < bodyVecs) {
        reduceOne<TRV, OP, KT, SC>(out, in, K, carrySrc, scaleMode, scale, accFlags,
                               bodyBase + v0 * TRV::kLanes, lane);
      }
    }
  }
  // the vectors ahead of the first tile, in pieces like the remainder's, dealt
  // from the last block downwards (the remainder's go from block 0 upwards, and
  // block 0 has the edges). Fewer than a tile when they only bring the tiles to a
  // 4 KiB boundary; up to a round when the caller starts the rounds further in.
  const int64_t leadPieces = (static_cast<int64_t>(lead) + pieceVecs - 1) / pieceVecs;
  for (int64_t p = grid - 1 - blockIdx.x; p < leadPieces; p += grid) {
    const int64_t v0 = p * pieceVecs;
#pragma unroll
    for (int u = 0; u < kPiece; ++u) {
      const unsigned int lane = threadIdx.x + u * kBlock;
      if (v0 + lane < lead) {
        reduceOne<TRV, OP, KT, SC>(out, in, K, carrySrc, scaleMode, scale, accFlags,
                                   head + v0 * TRV::kLanes, lane);
      }
    }
  }
  // ragged edges: at most kLanes-1 scalars on each side, done by block 0
  if (blockIdx.x == 0 && threadIdx.x < head + tail) {
    const int64_t e = threadIdx.x < head
                          ? static_cast<int64_t>(threadIdx.x)
                          : head + nvec * TRV::kLanes + (threadIdx.x - head);
    reduceOne<TRS, OP, KT, SC>(out, in, K, carrySrc, scaleMode, scale, accFlags, e, 0u);
  }
}

// Vectors between the first vector of a slice and the next 4 KiB boundary of
// its first contribution (0 for the element-wise variants and for slices that
// end before the boundary).
template <typename TRV>
int leadVectors(const void* firstContrib, int64_t head, int64_t nvec, int64_t leadBytesHint) {
  if (sizeof(typename TRV::vec_t) != 16) return 0;
  if (leadBytesHint >= 0) {
    // the caller's choice, counted from the first byte of the slice
    const int64_t headBytes = head * static_cast<int64_t>(sizeof(typename TRV::elem_t));
    const int64_t lead = leadBytesHint > headBytes ? (leadBytesHint - headBytes) / 16 : 0;
    return lead < nvec && lead < (int64_t{1} << 30) ? static_cast<int>(lead) : 0;
  }
  const uintptr_t first = reinterpret_cast<uintptr_t>(firstContrib) +
                          static_cast<uintptr_t>(head) * sizeof(typename TRV::elem_t);
  const int64_t lead = static_cast<int64_t>(((kLaunchAlignBytes - (first & (kLaunchAlignBytes - 1))) &
                                             (kLaunchAlignBytes - 1)) / 16);
  return lead < nvec ? static_cast<int>(lead) : 0;
}

template <typename TRV, typename TRS, int OP, int KT, int SC = -1>
hipError_t launchVariant(const ReduceArgs& a, int64_t head, int64_t nvec,
                         int64_t tail, int numCus, hipStream_t stream) {
  Ptrs<KT> tab;
  for (int k = 0; k < a.K; ++k) tab.p[k] = a.contribs[k];
  for (int k = a.K; k < (KT > 0 ? KT : kMaxContribsPerLaunch); ++k) {
    tab.p[k] = a.contribs[0];
  }
  // Measured with 12.5 MiB launches alternating over two streams: the 8-way
  // fp32 variant gains 1.3 % from 3 blocks per CU over 2 (6,342 vs 6,263 GB/s,
  // medians of 4 alternating runs); for every other count of contributions and
  // for the 2-byte types the rule of planGrid is at least as good.
  // (bf16, 25 MiB buckets, 12.5 MiB launches: 5,896 GB/s with 2 blocks per CU,
  // 6,078 with 3, 6,068 with 4.)
  constexpr bool kEightWayGradient = sizeof(typename TRV::elem_t) <= 4 && TRV::kFloating && KT == 8;
  // The pre-scaled sums of the 2-byte types round every term to the storage
  // type before the fold: four times the arithmetic of the plain sum, and with
  // one wave per SIMD nothing overlaps it with the loads. A third block per CU
  // does (bf16, 8-way: 6,340 vs 6,050 GB/s; fp16: 6,330 vs 6,270).
  constexpr bool kPreScaledHalf =
      (SC == kPreMul || SC == kPreDiv) && sizeof(typename TRV::elem_t) == 2 && TRV::kFloating;
  // More than 8 contributions are loaded 8 at a time: several dependent load
  // phases per tile, which more resident waves hide (K = 16: 6,604 GB/s with 4
  // blocks per CU against 6,229 with 2, launches of one round either way).
  const int manyWay = KT == 0 && a.K > kChunk ? 4 : 0;
  const int lead = leadVectors<TRV>(a.contribs[0], head, nvec, a.lead_bytes);
  const int hint = a.blocks_per_cu > 0 ? a.blocks_per_cu
                                       : (kEightWayGradient || kPreScaledHalf ? 3 : manyWay);
  const GridPlan plan = planGrid(nvec - lead, a.K, numCus, hint);
  const int64_t grid = plan.grid, roundTiles = plan.roundTiles, pieces = plan.pieces;
  // Runs of 64 tiles (256 KiB) per XCD where the rounds are whole groups of 512
  // tiles, from 8 contributions on (8-way fp32 in one context on the same
  // buffers, runs on / off: 6,683-6,703 against 6,666-6,678 GB/s; bf16 +0.7 %;
  // 2 and 4 contributions lose 0.3 to 0.5 %).
  const int chunkShift = (gXcdChunkShift > 0 && a.K >= 8 && grid % 8 == 0 &&
                          roundTiles % (int64_t{8} << gXcdChunkShift) == 0 && roundTiles > 0)
                             ? gXcdChunkShift
                             : 0;
  using elem_t = typename TRV::elem_t;
  const elem_t* carrySrc =
      !a.carry ? nullptr
               : static_cast<const elem_t*>(a.carry_src != nullptr ? a.carry_src : a.out);
  const int accFlags = (a.carry && a.carry_acc ? kCarryIsAcc : 0) | (a.out_acc ? kOutIsAcc : 0);
  auto launch = [&](auto kernel) {
    if (a.startEvent != nullptr || a.stopEvent != nullptr) {
      // Timed launch: the events take the dispatch's own begin/end timestamps.
      hipExtLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(grid)), dim3(kBlock), 0, stream,
                            a.startEvent, a.stopEvent, 0, static_cast<typename TRV::elem_t*>(a.out),
                            tab, a.K, carrySrc, a.scale_mode, a.scale, accFlags, head, lead, nvec,
                            tail, roundTiles, pieces, chunkShift);
    } else {
      hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(grid)), dim3(kBlock), 0, stream,
                         static_cast<typename TRV::elem_t*>(a.out), tab, a.K, carrySrc,
                         a.scale_mode, a.scale, accFlags, head, lead, nvec, tail, roundTiles, pieces,
                         chunkShift);
    }
  };
  bool mixed = false;
  if constexpr (kHasMixedLoads<TRV, OP, KT, SC>) mixed = wantsMixedLoads(a) && !a.carry;
  if constexpr (kHasMixedLoads<TRV, OP, KT, SC>) {
    if (mixed) launch(&ksumKernel<TRV, TRS, OP, KT, SC, true>);
  }
  if (!mixed) launch(&ksumKernel<TRV, TRS, OP, KT, SC, false>);
  return hipGetLastError();
}

// ---- one launch over several pieces -------------------------------------------

// The pieces of a segmented launch, by value in the kernel arguments (2.4 KiB):
// per piece the output, the contributions, the split of its length into [head
// scalars][lead vectors][tiles][tail scalars] and where its tiles start in the
// launch's tile count. `lead` vectors bring the tiles of a piece to a 4 KiB
// boundary of its output.
template <int KC, int S>
struct SegTable {
  void* out[S];
  const void* in[S][KC];
  long long tileBegin[S + 1];
  long long nvec[S];
  int lead[S];
  short head[S];
  short tail[S];
  int nseg;
};

// A row of the table, indexed like Ptrs.
struct SegRow {
  const void* const* p;
};

// Every block walks the launch's tiles blockIdx, blockIdx + grid, ...: the
// piece a tile belongs to is found by walking the prefix sums (tiles ascend,
// so the walk never restarts; all of it uniform, in scalar registers), the
// piece's pointers are read from the kernel arguments, and the tile is reduced
// exactly as ksumKernel does it. A piece's first tile (its lead) and its last
// may be partial. The scalars at the ends of piece e are done by block e.
template <typename TRV, typename TRS, int KT, int SC, int KC, int S>
__global__ void __launch_bounds__(kBlock)
    ksumSegmentedKernel(const SegTable<KC, S> tab, int K, int scaleMode, float scale) {
  using elem_t = typename TRV::elem_t;
  constexpr long long kTile = static_cast<long long>(kBlock) * kUnroll;
  const long long total = tab.tileBegin[tab.nseg];
  int s = 0;
  for (long long t = blockIdx.x; t < total; t += gridDim.x) {
    while (t >= tab.tileBegin[s + 1]) ++s;
    const long long lt = t - tab.tileBegin[s];
    const long long lead = tab.lead[s];
    const long long nvec = tab.nvec[s];
    long long v0, count;
    if (lead > 0) {
      v0 = lt == 0 ? 0 : lead + (lt - 1) * kTile;
      count = lt == 0 ? lead : nvec - v0;
    } else {
      v0 = lt * kTile;
      count = nvec - v0;
    }
    const int64_t elemBase = tab.head[s] + v0 * TRV::kLanes;
    const SegRow row{tab.in[s]};
    elem_t* out = static_cast<elem_t*>(tab.out[s]);
    if (count >= kTile) {
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        reduceOne<TRV, FRG_SUM, KT, SC>(out, row, K, static_cast<const elem_t*>(nullptr), scaleMode,
                                        scale, 0, elemBase, threadIdx.x + u * kBlock);
      }
    } else {
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        const unsigned int lane = threadIdx.x + u * kBlock;
        if (lane < count) {
          reduceOne<TRV, FRG_SUM, KT, SC>(out, row, K, static_cast<const elem_t*>(nullptr),
                                          scaleMode, scale, 0, elemBase, lane);
        }
      }
    }
  }
  for (int e = blockIdx.x; e < tab.nseg; e += gridDim.x) {
    const int head = tab.head[e], tail = tab.tail[e];
    if (static_cast<int>(threadIdx.x) < head + tail) {
      const int64_t i = static_cast<int>(threadIdx.x) < head
                            ? static_cast<int64_t>(threadIdx.x)
                            : head + tab.nvec[e] * TRV::kLanes + (threadIdx.x - head);
      const SegRow row{tab.in[e]};
      reduceOne<TRS, FRG_SUM, KT, SC>(static_cast<elem_t*>(tab.out[e]), row, K,
                                      static_cast<const elem_t*>(nullptr), scaleMode, scale, 0, i, 0u);
    }
  }
}

static_assert(static_cast<int64_t>(kBlock) * kUnroll == kSegmentTileVectors, "the tile of the kernels");

// KT > 0: the number of contributions, fixed at compile time. KT == 0: any
// number up to KCAP (8 or 16), which sizes the table's rows and with them the
// number of pieces it holds: maxSegmentsPerLaunch(KCAP), which for every K is
// what maxSegmentsPerLaunch(K) promises the callers.
template <typename TRV, typename TRS, int KT, int SC, int KCAP = kMaxSegmentContribs>
hipError_t launchSegmentedVariant(const SegmentedArgs& a, int numCus, hipStream_t stream) {
  constexpr int KC = KT > 0 ? KT : KCAP;
  constexpr int S = maxSegmentsPerLaunch(KC);
  using Table = SegTable<KC, S>;
  static_assert(sizeof(Table) <= 3072, "the table travels in the kernel arguments");
  if (a.K > KC) return hipErrorInvalidValue;
  Table tab = {};
  const int64_t elsize = static_cast<int64_t>(sizeof(typename TRV::elem_t));
  long long tiles = 0;
  int nseg = 0;
  for (int i = 0; i < a.numPieces; ++i) {
    const SegPiece& pc = a.pieces[i];
    if (pc.n <= 0) continue;
    if (nseg == S) return hipErrorInvalidValue;  // more pieces than the table holds
    const PieceSplit sp = splitPiece(pc.out, pc.n, elsize);
    tab.out[nseg] = pc.out;
    for (int k = 0; k < KC; ++k) tab.in[nseg][k] = pc.contribs[k < a.K ? k : 0];
    tab.tileBegin[nseg] = tiles;
    tab.nvec[nseg] = sp.nvec;
    tab.lead[nseg] = static_cast<int>(sp.lead);
    tab.head[nseg] = static_cast<short>(sp.head);
    tab.tail[nseg] = static_cast<short>(sp.tail);
    tiles += sp.tiles;
    ++nseg;
  }
  if (nseg == 0) return hipSuccess;
  for (int i = nseg; i <= S; ++i) tab.tileBegin[i] = tiles;
  tab.nseg = nseg;
  const int blocksPerCu = a.blocks_per_cu > 0 ? a.blocks_per_cu : 4;
  long long grid = static_cast<long long>(numCus) * blocksPerCu;
  if (grid > tiles) grid = tiles;
  if (grid < nseg) grid = nseg;  // a block per piece for the scalars at its ends
  if (a.startEvent != nullptr || a.stopEvent != nullptr) {
    hipExtLaunchKernelGGL((ksumSegmentedKernel<TRV, TRS, KT, SC, KC, S>),
                          dim3(static_cast<unsigned>(grid)), dim3(kBlock), 0, stream, a.startEvent,
                          a.stopEvent, 0, tab, a.K, a.scale_mode, a.scale);
  } else {
    hipLaunchKernelGGL((ksumSegmentedKernel<TRV, TRS, KT, SC, KC, S>),
                       dim3(static_cast<unsigned>(grid)), dim3(kBlock), 0, stream, tab, a.K,
                       a.scale_mode, a.scale);
  }
  return hipGetLastError();
}

// The gradient shapes (2, 4 or 8 contributions; no scale, the multiply by 1/K
// on the store, or every term times 1/K) as compile-time variants, like the
// plain kernel's; everything else through the runtime-K body.
template <typename TRV, typename TRS>
hipError_t dispatchSegmented(const SegmentedArgs& a, int numCus, hipStream_t stream) {
#define FRG_SEG_CASE(KK, MODE, SCV)                                                    \
  if (a.K == KK && a.scale_mode == MODE) {                                             \
    return launchSegmentedVariant<TRV, TRS, KK, SCV>(a, numCus, stream);               \
  }
  FRG_SEG_CASE(8, FRG_SCALE_NONE, FRG_SCALE_NONE)
  FRG_SEG_CASE(8, FRG_SCALE_MUL, FRG_SCALE_MUL)
  FRG_SEG_CASE(8, FRG_SCALE_PRE_MUL, kPreMul)
  FRG_SEG_CASE(4, FRG_SCALE_NONE, FRG_SCALE_NONE)
  FRG_SEG_CASE(4, FRG_SCALE_MUL, FRG_SCALE_MUL)
  FRG_SEG_CASE(4, FRG_SCALE_PRE_MUL, kPreMul)
  FRG_SEG_CASE(2, FRG_SCALE_NONE, FRG_SCALE_NONE)
  FRG_SEG_CASE(2, FRG_SCALE_MUL, FRG_SCALE_MUL)
  FRG_SEG_CASE(2, FRG_SCALE_PRE_MUL, kPreMul)
#undef FRG_SEG_CASE
  // any other K or scale: the number of contributions at run time, in a table
  // with rows of 8 (24 pieces) or of 16 (12 pieces)
  const bool narrow = a.K <= 8;
  if (a.scale_mode == FRG_SCALE_PRE_MUL) {
    return narrow ? launchSegmentedVariant<TRV, TRS, 0, kPreMul, 8>(a, numCus, stream)
                  : launchSegmentedVariant<TRV, TRS, 0, kPreMul, 16>(a, numCus, stream);
  }
  if (a.scale_mode == FRG_SCALE_PRE_DIV) {
    return narrow ? launchSegmentedVariant<TRV, TRS, 0, kPreDiv, 8>(a, numCus, stream)
                  : launchSegmentedVariant<TRV, TRS, 0, kPreDiv, 16>(a, numCus, stream);
  }
  return narrow ? launchSegmentedVariant<TRV, TRS, 0, -1, 8>(a, numCus, stream)
                : launchSegmentedVariant<TRV, TRS, 0, -1, 16>(a, numCus, stream);
}

// FAST: also instantiate the compile-time-K variants (the gradient types);
// the other types run the runtime-K variant for every K.
template <typename TRV, typename TRS, bool FAST>
hipError_t dispatchK(const ReduceArgs& a, int64_t head, int64_t nvec,
                     int64_t tail, int numCus, hipStream_t stream) {
  if (a.op == FRG_MAX) {
    return launchVariant<TRV, TRS, FRG_MAX, 0>(a, head, nvec, tail, numCus, stream);
  }
  if ((a.carry && a.carry_acc) || a.out_acc) {
    if constexpr (TRV::kFloating && sizeof(typename TRV::elem_t) == 2) {
      return launchVariant<TRV, TRS, FRG_SUM, 0, kAccIo>(a, head, nvec, tail, numCus, stream);
    } else {
      return hipErrorInvalidValue;  // ruled out by launchReduce
    }
  }
  if constexpr (FAST) {
    // the gradient shapes: 2, 4 or 8 contributions, nothing carried in, no
    // scale or the multiply by 1/K
    if (!a.carry && (a.scale_mode == FRG_SCALE_NONE || a.scale_mode == FRG_SCALE_MUL)) {
      const bool mul = a.scale_mode == FRG_SCALE_MUL;
#define FRG_FAST_CASE(KK)                                                                       \
  case KK:                                                                                       \
    return mul ? launchVariant<TRV, TRS, FRG_SUM, KK, FRG_SCALE_MUL>(a, head, nvec, tail, numCus, \
                                                                     stream)                      \
               : launchVariant<TRV, TRS, FRG_SUM, KK, FRG_SCALE_NONE>(a, head, nvec, tail,       \
                                                                      numCus, stream);
      switch (a.K) {
        FRG_FAST_CASE(2)
        FRG_FAST_CASE(4)
        FRG_FAST_CASE(8)
        default:
          break;
      }
#undef FRG_FAST_CASE
    }
  }
  if constexpr (FAST) {
    // DDP's pre-division hook at the gradient shapes: every term times 1/K
    if (!a.carry && a.scale_mode == FRG_SCALE_PRE_MUL) {
      switch (a.K) {
        case 2:
          return launchVariant<TRV, TRS, FRG_SUM, 2, kPreMul>(a, head, nvec, tail, numCus, stream);
        case 4:
          return launchVariant<TRV, TRS, FRG_SUM, 4, kPreMul>(a, head, nvec, tail, numCus, stream);
        case 8:
          return launchVariant<TRV, TRS, FRG_SUM, 8, kPreMul>(a, head, nvec, tail, numCus, stream);
        default:
          break;
      }
    }
  }
  if (a.scale_mode >= FRG_SCALE_PRE_MUL) {
    if constexpr (TRV::kFloating) {
      return a.scale_mode == FRG_SCALE_PRE_MUL
                 ? launchVariant<TRV, TRS, FRG_SUM, 0, kPreMul>(a, head, nvec, tail, numCus, stream)
                 : launchVariant<TRV, TRS, FRG_SUM, 0, kPreDiv>(a, head, nvec, tail, numCus, stream);
    }
  }
  return launchVariant<TRV, TRS, FRG_SUM, 0>(a, head, nvec, tail, numCus, stream);
}

// Vector variant when the pointers allow it (nvec > 0), else the element-wise
// one: pointers that disagree modulo 16, or a slice shorter than a vector.
template <typename TRV, typename TRS, bool FAST>
hipError_t dispatchType(const ReduceArgs& a, int64_t head, int64_t nvec, int64_t tail,
                        int numCus, hipStream_t stream) {
  if (nvec > 0) return dispatchK<TRV, TRS, FAST>(a, head, nvec, tail, numCus, stream);
  return dispatchK<TRS, TRS, false>(a, 0, a.n, 0, numCus, stream);
}

}  // namespace

int computeUnits(int device) {
  // asked on every launch: a relaxed load once the device is known (two threads
  // that ask first at the same time both ask the runtime and store the same answer)
  static std::atomic<int> cusOf[64];
  std::atomic<int>& slot = cusOf[device & 63];
  int cus = slot.load(std::memory_order_relaxed);
  if (cus == 0) {
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) !=
            hipSuccess ||
        cus <= 0) {
      (void)hipGetLastError();
      cus = 256;
    }
    slot.store(cus, std::memory_order_relaxed);
  }
  return cus;
}

static int gBlocksPerCu = 0;  // 0 = derive from the number of loads per lane

GridPlan planGrid(int64_t nvec, int numContribs, int numCus, int blocksPerCuHint) {
  constexpr int64_t kTile = static_cast<int64_t>(kBlock) * kUnroll;
  const int64_t ntiles = (nvec + kTile - 1) / kTile;
  int blocksPerCu = gBlocksPerCu > 0 ? gBlocksPerCu : blocksPerCuHint;
  if (blocksPerCu <= 0) {
    const int perLane = (numContribs < kChunk ? numContribs : kChunk) * kUnroll;
    blocksPerCu = FRG_LOADS_PER_CU / perLane;
    if (blocksPerCu < 1) blocksPerCu = 1;
    if (blocksPerCu > 8) blocksPerCu = 8;  // a plain copy (K = 1) peaks at 8, not 16
  }
  // Persistent grid: a whole number of blocks per CU. The hardware deals blocks
  // to CUs round-robin, every block gets the same share of tiles, and a CU that
  // hosts one block more than its neighbours becomes the straggler the whole
  // launch waits for; measured on MI355X, 520 blocks are 15 % slower than 512.
  const int64_t cap = static_cast<int64_t>(numCus) * blocksPerCu;
  GridPlan plan;
  plan.grid = ntiles < cap ? ntiles : cap;
  if (plan.grid < 1) plan.grid = 1;
  plan.roundTiles = (nvec / kTile / plan.grid) * plan.grid;
  constexpr int64_t kPieceVecs = static_cast<int64_t>(kBlock) * FRG_REMAINDER_PIECE_UNROLL;
  plan.pieces = (nvec - plan.roundTiles * kTile + kPieceVecs - 1) / kPieceVecs;
  return plan;
}

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

void setTuning(int blocksPerCu) { gBlocksPerCu = blocksPerCu > 0 ? blocksPerCu : 0; }

void setXcdChunkShift(int shift) { gXcdChunkShift = shift >= 0 && shift <= 12 ? shift : 0; }
void setMixedLoads(int mode) { gMixedLoads = mode < 0 ? -1 : (mode > 0 ? 1 : 0); }
int xcdChunkShift() { return gXcdChunkShift; }

int launchSegmented(const SegmentedArgs& a, hipStream_t stream, std::string* err) {
  auto fail = [&](int code, const std::string& msg) {
    if (err) *err = msg;
    return code;
  };
  const int64_t elsize = elementSize(a.dtype);
  if (!segmentedKind(a.K, a.dtype, FRG_SUM, false)) {
    return fail(FRG_ERR_UNSUPPORTED, "a segmented launch takes a SUM of fp32, bf16 or fp16 with "
                                     "up to 16 contributions");
  }
  if (a.scale_mode < FRG_SCALE_NONE || a.scale_mode > FRG_SCALE_PRE_DIV) {
    return fail(FRG_ERR_INVALID, "bad scale mode");
  }
  if (a.numPieces < 0 || a.numPieces > maxSegmentsPerLaunch(a.K) ||
      (a.numPieces > 0 && a.pieces == nullptr)) {
    return fail(FRG_ERR_INVALID, "a segmented launch takes up to " +
                                     std::to_string(maxSegmentsPerLaunch(a.K)) + " pieces");
  }
  for (int i = 0; i < a.numPieces; ++i) {
    const SegPiece& pc = a.pieces[i];
    if (pc.n < 0) return fail(FRG_ERR_INVALID, "negative element count");
    if (pc.n == 0) continue;
    if (pc.out == nullptr || pc.contribs == nullptr) return fail(FRG_ERR_INVALID, "null piece");
    const uintptr_t o = reinterpret_cast<uintptr_t>(pc.out);
    const uintptr_t bytes = static_cast<uintptr_t>(pc.n) * static_cast<uintptr_t>(elsize);
    for (int k = 0; k < a.K; ++k) {
      const uintptr_t p = reinterpret_cast<uintptr_t>(pc.contribs[k]);
      if (p == 0) return fail(FRG_ERR_INVALID, "null contribution " + std::to_string(k));
      if (p != o && p < o + bytes && o < p + bytes) {
        return fail(FRG_ERR_INVALID, "output partially overlaps contribution " + std::to_string(k));
      }
    }
    if (!segmentable(pc.out, pc.contribs, a.K, elsize)) {
      return fail(FRG_ERR_INVALID, "the pointers of a piece of a segmented launch must agree "
                                   "modulo 16 bytes");
    }
  }
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return fail(FRG_ERR_HIP, "hipGetDevice failed");
  const int numCus = computeUnits(device);
  hipError_t e = hipErrorInvalidValue;
  switch (a.dtype) {
    case FRG_F32:
      e = dispatchSegmented<F32Vec, F32Scalar>(a, numCus, stream);
      break;
    case FRG_BF16:
      e = dispatchSegmented<Bf16Vec, Bf16Scalar>(a, numCus, stream);
      break;
    case FRG_F16:
      e = dispatchSegmented<F16Vec, F16Scalar>(a, numCus, stream);
      break;
    default:
      break;
  }
  if (e != hipSuccess) {
    return fail(FRG_ERR_HIP, std::string("kernel launch failed: ") + hipGetErrorString(e));
  }
  return FRG_OK;
}

int launchReduce(const ReduceArgs& a, hipStream_t stream, std::string* err) {
  auto fail = [&](int code, const std::string& msg) {
    if (err) *err = msg;
    return code;
  };
  const int64_t elsize = elementSize(a.dtype);
  if (elsize == 0) {
    return fail(FRG_ERR_UNSUPPORTED, "unsupported dtype " + std::to_string(a.dtype));
  }
  if (a.op != FRG_SUM && a.op != FRG_MAX) {
    return fail(FRG_ERR_UNSUPPORTED,
                "unsupported reduce op " + std::to_string(a.op) + " (only SUM and MAX)");
  }
  if (a.K < 1 || a.K > kMaxContribsPerLaunch) {
    return fail(FRG_ERR_INVALID, "K must be in [1, 64] per launch, got " + std::to_string(a.K));
  }
  if (a.n < 0) return fail(FRG_ERR_INVALID, "negative element count");
  if (a.scale_mode < FRG_SCALE_NONE || a.scale_mode > FRG_SCALE_PRE_DIV) {
    return fail(FRG_ERR_INVALID, "bad scale mode");
  }
  if (a.op == FRG_MAX && a.scale_mode != FRG_SCALE_NONE) {
    return fail(FRG_ERR_INVALID, "MAX takes no scale");
  }
  if (a.scale_mode != FRG_SCALE_NONE && !isFloating(a.dtype)) {
    return fail(FRG_ERR_INVALID, "integer types take no scale");
  }
  if (a.contribs == nullptr) return fail(FRG_ERR_INVALID, "null contribution table");
  if (a.n == 0) return FRG_OK;  // device.cc:120-122
  if (a.out == nullptr) return fail(FRG_ERR_INVALID, "null output");

  const bool carryAcc = a.carry && a.carry_acc;
  if (carryAcc || a.out_acc) {
    if ((a.dtype != FRG_BF16 && a.dtype != FRG_F16) || a.op != FRG_SUM) {
      return fail(FRG_ERR_INVALID, "fp32 accumulator buffers go with a SUM of bf16 or fp16");
    }
    if (carryAcc && a.carry_src == nullptr) {
      return fail(FRG_ERR_INVALID, "null accumulator buffer to carry from");
    }
  }
  const int lanes = static_cast<int>(16 / elsize);
  const uintptr_t o = reinterpret_cast<uintptr_t>(a.out);
  const uintptr_t outElsize = a.out_acc ? 4 : static_cast<uintptr_t>(elsize);
  const uintptr_t outBytes = static_cast<uintptr_t>(a.n) * outElsize;
  const uintptr_t bytes = static_cast<uintptr_t>(a.n) * elsize;
  if (o % outElsize != 0) return fail(FRG_ERR_INVALID, "output not element-aligned");
  // Position within 16 bytes that every pointer of the storage type must share
  // for the vector variant; fp32 accumulator buffers (of a 2-byte type) must
  // reach a 16-byte boundary after the same number of head elements.
  const uintptr_t ref = a.out_acc ? (reinterpret_cast<uintptr_t>(a.contribs[0]) & 15) : (o & 15);
  const uintptr_t headElems = ((16 - ref) & 15) / static_cast<uintptr_t>(elsize);
  bool congruent = true;
  auto accCongruent = [&](uintptr_t p) { return ((p + 4 * headElems) & 15) == 0; };
  if (a.out_acc && !accCongruent(o)) congruent = false;
  for (int k = 0; k < a.K; ++k) {
    const uintptr_t p = reinterpret_cast<uintptr_t>(a.contribs[k]);
    if (p == 0) return fail(FRG_ERR_INVALID, "null contribution " + std::to_string(k));
    if (p % elsize != 0) {
      return fail(FRG_ERR_INVALID, "contribution " + std::to_string(k) + " not element-aligned");
    }
    const bool inPlace = p == o && !a.out_acc;
    if (!inPlace && p < o + outBytes && o < p + bytes) {
      return fail(FRG_ERR_INVALID,
                  "output partially overlaps contribution " + std::to_string(k));
    }
    if ((p & 15) != ref) congruent = false;
  }
  if (a.carry && a.carry_src != nullptr && a.carry_src != a.out) {
    const uintptr_t c = reinterpret_cast<uintptr_t>(a.carry_src);
    const uintptr_t cElsize = carryAcc ? 4 : static_cast<uintptr_t>(elsize);
    if (c % cElsize != 0) return fail(FRG_ERR_INVALID, "carried-in term not element-aligned");
    if (c < o + outBytes && o < c + static_cast<uintptr_t>(a.n) * cElsize) {
      return fail(FRG_ERR_INVALID, "output partially overlaps the carried-in term");
    }
    if (carryAcc ? !accCongruent(c) : (c & 15) != ref) congruent = false;
  } else if (a.carry && carryAcc != a.out_acc) {
    // carried from `out` itself: both sides of one buffer must be of one kind
    return fail(FRG_ERR_INVALID, "the carried-in term and the output share a buffer but not a type");
  }

  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) {
    return fail(FRG_ERR_HIP, "hipGetDevice failed");
  }
  const int numCus = computeUnits(device);

  int64_t head = 0, nvec = 0, tail = 0;
  if (congruent) {
    head = static_cast<int64_t>(headElems);
    if (head > a.n) head = a.n;
    nvec = (a.n - head) / lanes;
    tail = a.n - head - nvec * lanes;
  }
  hipError_t e = hipErrorInvalidValue;
  switch (a.dtype) {
    case FRG_F32:
      e = dispatchType<F32Vec, F32Scalar, true>(a, head, nvec, tail, numCus, stream);
      break;
    case FRG_BF16:
      e = dispatchType<Bf16Vec, Bf16Scalar, true>(a, head, nvec, tail, numCus, stream);
      break;
    case FRG_F16:
      e = dispatchType<F16Vec, F16Scalar, true>(a, head, nvec, tail, numCus, stream);
      break;
    case FRG_F64:
      e = dispatchType<F64Vec, F64Scalar, false>(a, head, nvec, tail, numCus, stream);
      break;
    case FRG_I32:
      e = dispatchType<I32Vec, I32Scalar, false>(a, head, nvec, tail, numCus, stream);
      break;
    case FRG_I64:
      e = dispatchType<I64Vec, I64Scalar, false>(a, head, nvec, tail, numCus, stream);
      break;
    case FRG_U8:
      e = dispatchType<U8Vec, U8Scalar, false>(a, head, nvec, tail, numCus, stream);
      break;
    case FRG_I8:
      e = dispatchType<I8Vec, I8Scalar, false>(a, head, nvec, tail, numCus, stream);
      break;
    default:
      break;
  }
  if (e != hipSuccess) {
    return fail(FRG_ERR_HIP, std::string("kernel launch failed: ") + hipGetErrorString(e));
  }
  return FRG_OK;
}

}  // namespace frg
