// The reduction with torch's gradient-compression hooks folded in (gfx950).
//
// With a bf16 or fp16 compression hook registered, every rank of a DDP job
// does, per bucket
// (torch:distributed/algorithms/ddp_comm_hooks/default_hooks.py:57-93):
//     compressed = buffer.to(wire).div_(world)   two passes over the bucket
//     allreduce(compressed)                      fairring/process_group.cc:131-155
//     buffer.copy_(result)                       one more pass
// Here the three are one pass: the rank's own fp32 bucket is cast, divided and
// rounded in registers, the peers' contributions are read in the wire type, the
// fold runs in fp32 in contribution order with one rounding to the wire type
// (as the plain bf16 / fp16 reduction does), and the result is stored widened
// into the fp32 bucket, which may be the very buffer the raw term was read
// from. Per element that is 4 + 2 (K - 1) + 4 bytes of HBM traffic instead of
// (4 + 2) + (2 K + 2) + (2 + 4).
//
// One lane owns 8 consecutive elements: one 16-byte vector of every wire
// contribution, two of the fp32 buffer on either side.

#include <hip/hip_ext.h>
#include <hip/hip_runtime.h>

#include <limits>
#include <type_traits>

#include "../../include/fairring_hip.h"
#include "device_traits.h"
#include "ksum_kernels.h"

namespace frg {
namespace {

// The fp32 side of a group of 8 elements, moved coalesced and exchanged through LDS.
//
// A lane's 8 fp32 values are 32 consecutive bytes, two 16-byte accesses with a
// stride of 32 bytes between lanes: every instruction of a wave then touches
// sixteen 128-byte lines for eight lines' worth of data, which measured 4 %
// on a kernel with one input and the output accessed that way. In whole tiles
// (all 64 lanes of a wave take part) the fp32 side moves in the coalesced
// pattern instead, lane l taking the 16-byte chunks l and l + 64 of the wave's
// 2 KiB, and the two patterns are exchanged through a wave-private 2 KiB of
// LDS (`stage`). A wave executes its LDS instructions in order, so the exchange
// needs no barrier, only that the compiler keeps the order it is given.
// The two halves of the load: the global loads are issued first, so that the
// wire loads that follow them in program order are in flight before the
// exchange waits for these two.
struct StagedChunks {
  f32x4 lo, hi;
};

// Where the raw fp32 term of element e is read from: `origin(e) + e`. One
// buffer; or the tensors a bucket is assembled from, each given by its address
// minus its offset in the bucket (so that adding the element's index lands in
// it) and the element it starts at. Every 16-byte access lies within one
// tensor (the launch code sees to it), so a lane looks its tensor up once per
// access, by straight-line compares over the few entries.
struct RawPlain {
  const float* base;
  __device__ __forceinline__ const float* origin(int64_t) const { return base; }
};
constexpr int kMaxRawPieces = kMaxRawPiecesPerLaunch;  // what the callers are told
struct RawPieces {
  const float* adj[kMaxRawPieces];
  // off[0] = 0; unused entries hold the largest value. 32 bits (a launch of
  // this kind has fewer than 2^31 elements): compares that the scalar unit has.
  int off[kMaxRawPieces];
  __device__ __forceinline__ const float* origin(int64_t e) const {
    const int e32 = static_cast<int>(e);
    const float* p = adj[0];
#pragma unroll
    for (int i = 1; i < kMaxRawPieces; ++i) p = e32 >= off[i] ? adj[i] : p;
    return p;
  }
};

// origin(e) for a lane of a wave whose accesses cover the `span` elements from
// `waveFirst` on: nearly always one tensor holds them all, which two look-ups
// on the scalar unit tell; only a wave that straddles tensors looks up per lane.
template <typename RAW>
__device__ __forceinline__ const float* rawOrigin(const RAW& raw, int64_t waveFirst, int span,
                                                  int64_t e) {
  if constexpr (sizeof(RAW) == sizeof(RawPlain)) {
    return raw.origin(e);
  } else if (span < 512) {
    // the element-wise variant: its lanes need not sit side by side (the
    // scalars at a launch's two ends are reduced by one block)
    return raw.origin(e);
  } else {
    const int first = __builtin_amdgcn_readfirstlane(static_cast<int>(waveFirst));
    const float* a = raw.origin(first);
    const float* b = raw.origin(first + span - 1);
    if (a == b) return a;
    return raw.origin(e);
  }
}

template <typename RAW>
__device__ __forceinline__ StagedChunks issueStaged(const RAW& raw, int64_t elemBase,
                                                    unsigned int lane) {
  const unsigned int waveLane = lane & 63u;
  const int64_t waveBase = elemBase + static_cast<int64_t>(lane - waveLane) * 8;
  const int64_t lo = waveBase + 4 * static_cast<int64_t>(waveLane);
  StagedChunks c;
  c.lo = ldStream(reinterpret_cast<const f32x4*>(rawOrigin(raw, waveBase, 512, lo) + lo));
  c.hi = ldStream(reinterpret_cast<const f32x4*>(rawOrigin(raw, waveBase, 512, lo + 256) + lo + 256));
  return c;
}

__device__ __forceinline__ Fp32Side<8>::regs_t exchangeStaged(const StagedChunks& c,
                                                             unsigned int lane, f32x4* stage) {
  const unsigned int waveLane = lane & 63u;
  stage[waveLane] = c.lo;
  stage[waveLane + 64] = c.hi;
  __builtin_amdgcn_wave_barrier();
  Fp32Side<8>::regs_t r;
  r.a = stage[2 * waveLane];
  r.b = stage[2 * waveLane + 1];
  __builtin_amdgcn_wave_barrier();
  return r;
}

__device__ __forceinline__ void storeStaged(float* base, int64_t elemBase, unsigned int lane,
                                            const float (&f)[8], f32x4* stage) {
  const unsigned int waveLane = lane & 63u;
  const int64_t waveBase = elemBase + static_cast<int64_t>(lane - waveLane) * 8;
  f32x4 lo, hi;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    lo[j] = f[j];
    hi[j] = f[4 + j];
  }
  stage[2 * waveLane] = lo;
  stage[2 * waveLane + 1] = hi;
  __builtin_amdgcn_wave_barrier();
  const f32x4 outLo = stage[waveLane];
  const f32x4 outHi = stage[waveLane + 64];
  __builtin_amdgcn_wave_barrier();
  f32x4* p = reinterpret_cast<f32x4*>(base + waveBase) + waveLane;
  stStream(outLo, p);
  stStream(outHi, p + 64);
}

// State of one lane's fold: the accumulator, whether it holds a term yet, and
// this rank's own term (compressed once the loads that follow it are issued).
template <typename W>
struct Fold {
  float acc[W::kLanes];
  float own[W::kLanes];
  bool first = true;
  bool ownReady = false;
  // where the own term comes from when the fp32 side is staged through LDS
  // (issued by compressedOne, exchanged once the wire loads are in flight)
  StagedChunks chunks;
  f32x4* stage = nullptr;
  unsigned int lane = 0;

  __device__ __forceinline__ void add(const float (&t)[W::kLanes]) {
    if (first) {
#pragma unroll
      for (int j = 0; j < W::kLanes; ++j) acc[j] = t[j];
      first = false;
    } else {
#pragma unroll
      for (int j = 0; j < W::kLanes; ++j) acc[j] = acc[j] + t[j];
    }
  }

  // buffer.to(wire) then div_(world) in the wire type: two roundings
  __device__ __forceinline__ void compress(const typename Fp32Side<W::kLanes>::regs_t& raw,
                                           int scaleMode, float scale) {
    if (ownReady) return;
    bool unpacked = false;
    if constexpr (W::kLanes == 8) {
      if (stage != nullptr) {
        Fp32Side<8>::unpack(exchangeStaged(chunks, lane, stage), own);
        unpacked = true;
      }
    }
    if (!unpacked) Fp32Side<W::kLanes>::unpack(raw, own);
#pragma unroll
    for (int j = 0; j < W::kLanes; ++j) {
      float c = W::roundStorage(own[j]);
      if (scaleMode == FRG_SCALE_MUL) {
        c = W::roundStorage(c * scale);
      } else if (scaleMode == FRG_SCALE_DIV) {
        c = W::roundStorage(c / scale);
      }
      own[j] = c;
    }
    ownReady = true;
  }
};

// Loads wire contributions [k0, k0+N), then folds them in order; the own term
// goes in ahead of wire contribution `rawPos`.
template <typename W, int N>
__device__ __forceinline__ void foldWire(Fold<W>& st, const Ptrs<0>& in, int k0, int64_t elemBase,
                                         unsigned int laneBytes, int rawPos,
                                         const typename Fp32Side<W::kLanes>::regs_t& raw,
                                         int scaleMode, float scale) {
  using vec_t = typename W::vec_t;
  using elem_t = typename W::elem_t;
  vec_t v[N];
#pragma unroll
  for (int k = 0; k < N; ++k) {
    const char* b = reinterpret_cast<const char*>(static_cast<const elem_t*>(in.p[k0 + k]) + elemBase);
    v[k] = ldStream(reinterpret_cast<const vec_t*>(b + laneBytes));
  }
  if (rawPos >= 0) st.compress(raw, scaleMode, scale);
#pragma unroll
  for (int k = 0; k < N; ++k) {
    if (k0 + k == rawPos) st.add(st.own);
    float f[W::kLanes];
    W::unpack(v[k], f);
    st.add(f);
  }
}

// One lane's group of elements. `wire` holds the Kw peers' pointers in order,
// `raw` this rank's fp32 buffer (rawPos = its place in the chain, -1: absent).
// STAGED (whole tiles of the 8-element variant only): the fp32 side goes
// through loadStaged / storeStaged.
template <typename W, bool OUT32, bool STAGED = false, typename RAW = RawPlain>
__device__ __forceinline__ void compressedOne(void* out, const RAW& raw, const Ptrs<0>& wire,
                                              int Kw, int rawPos, int scaleMode, float scale,
                                              int64_t elemBase, unsigned int lane,
                                              f32x4* stage = nullptr) {
  using vec_t = typename W::vec_t;
  using Side = Fp32Side<W::kLanes>;
  const unsigned int laneBytes = lane * static_cast<unsigned int>(sizeof(vec_t));
  typename Side::regs_t rawRegs = {};
  Fold<W> st;
  if (rawPos >= 0) {
    if constexpr (STAGED) {
      st.chunks = issueStaged(raw, elemBase, lane);
      st.stage = stage;
      st.lane = lane;
    } else {
      rawRegs = Side::load(
          rawOrigin(raw, elemBase + static_cast<int64_t>(lane - (lane & 63u)) * W::kLanes,
                    64 * W::kLanes, elemBase + static_cast<int64_t>(lane) * W::kLanes) +
              elemBase,
          lane);
    }
  }
  int k = 0;
  for (; k + kChunk <= Kw; k += kChunk) {
    foldWire<W, kChunk>(st, wire, k, elemBase, laneBytes, rawPos, rawRegs, scaleMode, scale);
  }
  switch (Kw - k) {
    case 7: foldWire<W, 7>(st, wire, k, elemBase, laneBytes, rawPos, rawRegs, scaleMode, scale); break;
    case 6: foldWire<W, 6>(st, wire, k, elemBase, laneBytes, rawPos, rawRegs, scaleMode, scale); break;
    case 5: foldWire<W, 5>(st, wire, k, elemBase, laneBytes, rawPos, rawRegs, scaleMode, scale); break;
    case 4: foldWire<W, 4>(st, wire, k, elemBase, laneBytes, rawPos, rawRegs, scaleMode, scale); break;
    case 3: foldWire<W, 3>(st, wire, k, elemBase, laneBytes, rawPos, rawRegs, scaleMode, scale); break;
    case 2: foldWire<W, 2>(st, wire, k, elemBase, laneBytes, rawPos, rawRegs, scaleMode, scale); break;
    case 1: foldWire<W, 1>(st, wire, k, elemBase, laneBytes, rawPos, rawRegs, scaleMode, scale); break;
    default: break;
  }
  if (rawPos == Kw) {  // own term last (or alone)
    st.compress(rawRegs, scaleMode, scale);
    st.add(st.own);
  }
  // one rounding to the wire type; the fp32 output holds that value widened
  if (OUT32) {
    float r[W::kLanes];
#pragma unroll
    for (int j = 0; j < W::kLanes; ++j) r[j] = W::roundStorage(st.acc[j]);
    if constexpr (STAGED) {
      storeStaged(static_cast<float*>(out), elemBase, lane, r, stage);
    } else {
      Side::store(static_cast<float*>(out) + elemBase, lane, r);
    }
  } else {
    vec_t* o = reinterpret_cast<vec_t*>(
        reinterpret_cast<char*>(static_cast<typename W::elem_t*>(out) + elemBase) + laneBytes);
    stStream(W::pack(st.acc), o);
  }
}

// The hook's own shapes (a raw fp32 bucket, KW = 1, 3 or 7 peers, fp32 output,
// no scale or the multiply by 1/K) with everything but the own term's place
// fixed at compile time: all loads are issued first, the fold is straight-line
// code with one uniform branch per position the own term can take, and the
// body is a tenth of the general one's code (which matters when a launch
// lasts 20 us and every CU starts it with a cold instruction cache). Same
// arithmetic, in the same order, as compressedOne.
// STAGED (whole tiles): the fp32 side goes through loadStaged / storeStaged.
template <typename W, int KW, int SC, bool STAGED = false, typename RAW = RawPlain>
__device__ __forceinline__ void compressedFixed(float* out, const RAW& raw, const Ptrs<KW>& wire,
                                                int rawPos, float scale, int64_t elemBase,
                                                unsigned int lane, f32x4* stage = nullptr) {
  using vec_t = typename W::vec_t;
  using elem_t = typename W::elem_t;
  using Side = Fp32Side<W::kLanes>;
  const unsigned int laneBytes = lane * static_cast<unsigned int>(sizeof(vec_t));
  typename Side::regs_t rawRegs;
  StagedChunks chunks;
  if constexpr (STAGED) {
    chunks = issueStaged(raw, elemBase, lane);
  } else {
    rawRegs = Side::load(
        rawOrigin(raw, elemBase + static_cast<int64_t>(lane - (lane & 63u)) * W::kLanes,
                  64 * W::kLanes, elemBase + static_cast<int64_t>(lane) * W::kLanes) +
            elemBase,
        lane);
  }
  vec_t v[KW];
#pragma unroll
  for (int k = 0; k < KW; ++k) {
    const char* b = reinterpret_cast<const char*>(static_cast<const elem_t*>(wire.p[k]) + elemBase);
    v[k] = ldStream(reinterpret_cast<const vec_t*>(b + laneBytes));
  }
  if constexpr (STAGED) rawRegs = exchangeStaged(chunks, lane, stage);
  // buffer.to(wire) then div_(world) in the wire type: two roundings
  float own[W::kLanes];
  Side::unpack(rawRegs, own);
#pragma unroll
  for (int j = 0; j < W::kLanes; ++j) {
    float c = W::roundStorage(own[j]);
    if (SC == FRG_SCALE_MUL) c = W::roundStorage(c * scale);
    own[j] = c;
  }
  float acc[W::kLanes];
  float f[W::kLanes];
  W::unpack(v[0], f);
  if (rawPos == 0) {
#pragma unroll
    for (int j = 0; j < W::kLanes; ++j) acc[j] = own[j] + f[j];
  } else {
#pragma unroll
    for (int j = 0; j < W::kLanes; ++j) acc[j] = f[j];
  }
#pragma unroll
  for (int k = 1; k < KW; ++k) {
    if (k == rawPos) {
#pragma unroll
      for (int j = 0; j < W::kLanes; ++j) acc[j] = acc[j] + own[j];
    }
    W::unpack(v[k], f);
#pragma unroll
    for (int j = 0; j < W::kLanes; ++j) acc[j] = acc[j] + f[j];
  }
  if (rawPos == KW) {
#pragma unroll
    for (int j = 0; j < W::kLanes; ++j) acc[j] = acc[j] + own[j];
  }
  // one rounding to the wire type, stored widened
#pragma unroll
  for (int j = 0; j < W::kLanes; ++j) acc[j] = W::roundStorage(acc[j]);
  if constexpr (STAGED) {
    storeStaged(out, elemBase, lane, acc, stage);
  } else {
    Side::store(out + elemBase, lane, acc);
  }
}

// KW > 0: the fixed shape above (OUT32, raw term present, scale mode SC);
// KW == 0: the general body.
template <typename W, bool OUT32, int KW, int SC, typename RAW>
__device__ __forceinline__ void compressedLane(void* out, const RAW& raw, const Ptrs<KW>& wire,
                                               int Kw, int rawPos, int scaleMode, float scale,
                                               int64_t elemBase, unsigned int lane) {
  if constexpr (KW > 0) {
    compressedFixed<W, KW, SC, false, RAW>(static_cast<float*>(out), raw, wire, rawPos, scale,
                                           elemBase, lane);
  } else {
    compressedOne<W, OUT32, false, RAW>(out, raw, wire, Kw, rawPos, scaleMode, scale, elemBase,
                                        lane);
  }
}

// Same dealing of tiles, remainder pieces and ragged edges as the plain
// reduction kernel; a "vector" is a lane's group of 8 elements.
template <typename WV, typename WS, bool OUT32, int KW, int SC, typename RAW>
__global__ void __launch_bounds__(kBlock)
    compressedKernel(void* out, const RAW raw, Ptrs<KW> wire, int Kw, int rawPos, int scaleMode,
                     float scale, int64_t head, int lead, int64_t nvec, int64_t tail,
                     int64_t roundTiles, int64_t pieces, int chunkShift) {
  constexpr int64_t kTile = static_cast<int64_t>(kBlock) * kUnroll;
  const int64_t grid = gridDim.x;
  // the first `lead` groups are a piece of their own, so that the tiles start
  // on a 4 KiB boundary of the first wire contribution
  const int64_t bodyBase = head + static_cast<int64_t>(lead) * WV::kLanes;
  const int64_t bodyVecs = nvec - lead;
  // whole tiles: every lane of every wave takes part, so the fp32 side can go
  // through the wave's staging area in LDS
  constexpr bool kStaged = WV::kLanes == 8 && kBlock % 64 == 0;
  __shared__ f32x4 stageAll[kStaged ? (kBlock / 64) * 128 : 1];
  f32x4* stage = stageAll + (kStaged ? (threadIdx.x >> 6) * 128 : 0);
  for (int64_t t0 = blockIdx.x; t0 < roundTiles; t0 += grid) {
    // runs of 2^chunkShift consecutive tiles for the blocks of one XCD (the
    // hardware deals blocks to the 8 XCDs in turn), as in the plain kernel
    int64_t t = t0;
    if (chunkShift > 0) {
      const int64_t low = (int64_t{1} << chunkShift) - 1;
      t = ((t0 >> (3 + chunkShift)) << (3 + chunkShift)) | ((t0 & 7) << chunkShift) |
          ((t0 >> 3) & low);
    }
    const int64_t elemBase = bodyBase + t * kTile * WV::kLanes;
    // one tile with the raw term read as `src` says
    auto tile = [&](const auto& src) {
      using SRC = std::remove_cv_t<std::remove_reference_t<decltype(src)>>;
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        const unsigned int lane = threadIdx.x + u * kBlock;
        if constexpr (kStaged && KW > 0) {
          compressedFixed<WV, KW, SC, true, SRC>(static_cast<float*>(out), src, wire, rawPos,
                                                 scale, elemBase, lane, stage);
        } else if constexpr (kStaged) {
          compressedOne<WV, OUT32, true, SRC>(out, src, wire, Kw, rawPos, scaleMode, scale,
                                              elemBase, lane, stage);
        } else {
          compressedLane<WV, OUT32, KW, SC, SRC>(out, src, wire, Kw, rawPos, scaleMode, scale,
                                                 elemBase, lane);
        }
      }
    };
    if constexpr (sizeof(RAW) == sizeof(RawPlain)) {
      tile(raw);
    } else {
      // Nearly every tile lies within one tensor of the raw term: it then runs
      // the very code of the one-buffer kernel, on that tensor's origin; only
      // a tile that straddles tensors looks them up access by access. (With
      // the look-ups in every tile's code, uniform as they were, the kernel ran
      // 14 % slower: a launch lasts 20 us and starts with cold instruction
      // caches.)
      const float* a = raw.origin(elemBase);
      const float* b = raw.origin(elemBase + kTile * WV::kLanes - 1);
      if (a == b) {
        tile(RawPlain{a});
      } else {
        tile(raw);
      }
    }
  }
  const int64_t restBase = roundTiles * kTile;
  constexpr int kPiece = FRG_REMAINDER_PIECE_UNROLL;
  constexpr int64_t pieceVecs = static_cast<int64_t>(kBlock) * kPiece;
  for (int64_t p = blockIdx.x; p < pieces; p += grid) {
    const int64_t v0 = restBase + p * pieceVecs;
#pragma unroll
    for (int u = 0; u < kPiece; ++u) {
      const unsigned int lane = threadIdx.x + u * kBlock;
      if (v0 + lane < bodyVecs) {
        compressedLane<WV, OUT32, KW, SC, RAW>(out, raw, wire, Kw, rawPos, scaleMode, scale,
                                          bodyBase + v0 * WV::kLanes, lane);
      }
    }
  }
  if (lead > 0 && blockIdx.x == gridDim.x - 1) {
    for (unsigned int lane = threadIdx.x; lane < static_cast<unsigned int>(lead); lane += kBlock) {
      compressedLane<WV, OUT32, KW, SC, RAW>(out, raw, wire, Kw, rawPos, scaleMode, scale, head, lane);
    }
  }
  if (blockIdx.x == 0 && threadIdx.x < head + tail) {
    const int64_t e = threadIdx.x < head
                          ? static_cast<int64_t>(threadIdx.x)
                          : head + nvec * WV::kLanes + (threadIdx.x - head);
    compressedLane<WS, OUT32, KW, SC, RAW>(out, raw, wire, Kw, rawPos, scaleMode, scale, e, 0u);
  }
}

// `leadRef`: the address whose 4 KiB grid the tiles follow when there is no wire
// contribution (the raw buffer's; the output's when the raw term comes in pieces).
template <typename WV, typename WS, bool OUT32, int KW, int SC, typename RAW>
hipError_t launchCompressed(const CompressedArgs& a, const RAW& raw, uintptr_t leadRef,
                            const Ptrs<0>& all, int Kw, int rawPos, int64_t head, int64_t nvec,
                            int64_t tail, int numCus, hipStream_t stream) {
  Ptrs<KW> wire;
  for (int k = 0; k < (KW > 0 ? KW : kMaxContribsPerLaunch); ++k) wire.p[k] = all.p[k];
  // groups between the first one and the next 4 KiB boundary of the first wire
  // contribution (of the fp32 bucket at twice the stride when it stands alone)
  int lead = 0;
  if (sizeof(typename WV::vec_t) == 16) {
    const uintptr_t first =
        Kw > 0 ? reinterpret_cast<uintptr_t>(all.p[0]) + static_cast<uintptr_t>(head) * 2
               : (leadRef + static_cast<uintptr_t>(head) * 4) / 2;
    const int64_t l = static_cast<int64_t>(
        ((kLaunchAlignBytes - (first & (kLaunchAlignBytes - 1))) & (kLaunchAlignBytes - 1)) / 16);
    lead = l < nvec ? static_cast<int>(l) : 0;
  }
  const GridPlan plan = planGrid(nvec - lead, a.K, numCus);
  // Runs per XCD as in the plain kernel, with at least two groups of 8 runs in
  // flight on the grid (512 blocks here: runs of 32 tiles; runs of 128, one
  // group wider than the grid, measured 10 % slower than none).
  int shift = xcdChunkShift();
  while (shift > 0 && (int64_t{16} << shift) > plan.grid) --shift;
  const int chunkShift = (shift > 0 && plan.grid % 8 == 0 && plan.roundTiles > 0 &&
                          plan.roundTiles % (int64_t{8} << shift) == 0)
                             ? shift
                             : 0;
  if (a.startEvent != nullptr || a.stopEvent != nullptr) {
    hipExtLaunchKernelGGL((compressedKernel<WV, WS, OUT32, KW, SC, RAW>),
                          dim3(static_cast<unsigned>(plan.grid)), dim3(kBlock), 0, stream,
                          a.startEvent, a.stopEvent, 0, a.out, raw, wire, Kw, rawPos, a.scale_mode,
                          a.scale, head, lead, nvec, tail, plan.roundTiles, plan.pieces,
                          chunkShift);
  } else {
    hipLaunchKernelGGL((compressedKernel<WV, WS, OUT32, KW, SC, RAW>),
                       dim3(static_cast<unsigned>(plan.grid)), dim3(kBlock), 0, stream, a.out, raw,
                       wire, Kw, rawPos, a.scale_mode, a.scale, head, lead, nvec, tail,
                       plan.roundTiles, plan.pieces, chunkShift);
  }
  return hipGetLastError();
}

template <typename WV, typename WS, typename RAW>
hipError_t dispatchOut(const CompressedArgs& a, const RAW& raw, bool hasRaw, uintptr_t leadRef,
                       const Ptrs<0>& wire, int Kw, int rawPos, int64_t head, int64_t nvec,
                       int64_t tail, int numCus, hipStream_t stream) {
  if (nvec > 0) {
    // the hook's own shapes: a raw fp32 bucket and 1, 3 or 7 peers, fp32 output,
    // no scale or the multiply by 1/K
    if (a.out_dtype == FRG_F32 && hasRaw &&
        (a.scale_mode == FRG_SCALE_NONE || a.scale_mode == FRG_SCALE_MUL)) {
      const bool mul = a.scale_mode == FRG_SCALE_MUL;
#define FRG_FIXED_CASE(KK)                                                                   \
  case KK:                                                                                   \
    return mul ? launchCompressed<WV, WS, true, KK, FRG_SCALE_MUL, RAW>(                     \
                     a, raw, leadRef, wire, Kw, rawPos, head, nvec, tail, numCus, stream)    \
               : launchCompressed<WV, WS, true, KK, FRG_SCALE_NONE, RAW>(                    \
                     a, raw, leadRef, wire, Kw, rawPos, head, nvec, tail, numCus, stream);
      switch (Kw) {
        FRG_FIXED_CASE(1)
        FRG_FIXED_CASE(3)
        FRG_FIXED_CASE(7)
        default:
          break;
      }
#undef FRG_FIXED_CASE
    }
    return a.out_dtype == FRG_F32
               ? launchCompressed<WV, WS, true, 0, 0, RAW>(a, raw, leadRef, wire, Kw, rawPos, head,
                                                           nvec, tail, numCus, stream)
               : launchCompressed<WV, WS, false, 0, 0, RAW>(a, raw, leadRef, wire, Kw, rawPos,
                                                            head, nvec, tail, numCus, stream);
  }
  // element-wise: pointers that cannot be brought to 16-byte boundaries by one
  // common head, or fewer elements than a group
  return a.out_dtype == FRG_F32
             ? launchCompressed<WS, WS, true, 0, 0, RAW>(a, raw, leadRef, wire, Kw, rawPos, 0, a.n,
                                                         0, numCus, stream)
             : launchCompressed<WS, WS, false, 0, 0, RAW>(a, raw, leadRef, wire, Kw, rawPos, 0,
                                                          a.n, 0, numCus, stream);
}

// The raw term's address for element 0 of the launch if tensor `pc` went on
// for ever in both directions (what RawPieces::adj holds).
uintptr_t virtualOrigin(const RawPiece& pc) {
  return reinterpret_cast<uintptr_t>(pc.ptr) - static_cast<uintptr_t>(pc.off) * 4;
}

}  // namespace

int launchCompressedReduce(const CompressedArgs& a, hipStream_t stream, std::string* err) {
  auto fail = [&](int code, const std::string& msg) {
    if (err) *err = msg;
    return code;
  };
  if (a.wire_dtype != FRG_BF16 && a.wire_dtype != FRG_F16) {
    return fail(FRG_ERR_UNSUPPORTED, "the wire type must be bf16 or fp16");
  }
  if (a.out_dtype != FRG_F32 && a.out_dtype != a.wire_dtype) {
    return fail(FRG_ERR_UNSUPPORTED, "the output must be fp32 or of the wire type");
  }
  if (a.K < 1 || a.K > kMaxContribsPerLaunch) {
    return fail(FRG_ERR_INVALID, "K must be in [1, 64], got " + std::to_string(a.K));
  }
  if (a.raw_index < -1 || a.raw_index >= a.K) {
    return fail(FRG_ERR_INVALID, "raw_index out of range");
  }
  if (a.n < 0) return fail(FRG_ERR_INVALID, "negative element count");
  if (a.scale_mode < FRG_SCALE_NONE || a.scale_mode > FRG_SCALE_DIV) {
    return fail(FRG_ERR_INVALID, "bad scale mode (NONE, MUL or DIV on the raw contribution)");
  }
  if (a.contribs == nullptr) return fail(FRG_ERR_INVALID, "null contribution table");
  if (a.n == 0) return FRG_OK;
  if (a.out == nullptr) return fail(FRG_ERR_INVALID, "null output");

  // Every pointer asks for a head h (elements before its first 16-byte
  // boundary): h mod 8 for a 2-byte type, h mod 4 for fp32. One h must do.
  const uintptr_t o = reinterpret_cast<uintptr_t>(a.out);
  const uintptr_t outElsize = a.out_dtype == FRG_F32 ? 4 : 2;
  if (o % outElsize != 0) return fail(FRG_ERR_INVALID, "output not element-aligned");
  const uintptr_t outBytes = static_cast<uintptr_t>(a.n) * outElsize;
  bool vectorOk = true;
  int64_t headWire = -1, headF32 = -1;
  auto want = [&](uintptr_t p, uintptr_t elsize) {
    const int64_t h = static_cast<int64_t>(((16 - (p & 15)) & 15) / elsize);
    int64_t& slot = elsize == 2 ? headWire : headF32;
    if (slot < 0) {
      slot = h;
    } else if (slot != h) {
      vectorOk = false;
    }
  };
  want(o, outElsize);

  const bool pieces = a.num_raw_pieces > 0;
  if (pieces) {
    if (a.raw_index < 0) return fail(FRG_ERR_INVALID, "raw pieces without a raw contribution");
    if (a.n > std::numeric_limits<int>::max()) {
      return fail(FRG_ERR_INVALID, "a launch with raw pieces takes fewer than 2^31 elements");
    }
    if (a.num_raw_pieces > kMaxRawPieces || a.raw_pieces == nullptr) {
      return fail(FRG_ERR_INVALID, "at most " + std::to_string(kMaxRawPieces) + " raw pieces per launch");
    }
    for (int i = 0; i < a.num_raw_pieces; ++i) {
      const RawPiece& pc = a.raw_pieces[i];
      const int64_t end = i + 1 < a.num_raw_pieces ? a.raw_pieces[i + 1].off : a.n;
      if (pc.ptr == nullptr || reinterpret_cast<uintptr_t>(pc.ptr) % 4 != 0 || pc.off < 0 ||
          pc.off >= end) {
        return fail(FRG_ERR_INVALID, "bad raw piece " + std::to_string(i));
      }
      const uintptr_t lo = reinterpret_cast<uintptr_t>(pc.ptr);
      const uintptr_t hi = lo + static_cast<uintptr_t>(end - pc.off) * 4;
      if (lo < o + outBytes && o < hi) {
        return fail(FRG_ERR_INVALID, "output overlaps raw piece " + std::to_string(i));
      }
      want(virtualOrigin(pc), 4);
    }
    if (a.raw_pieces[0].off != 0) return fail(FRG_ERR_INVALID, "the first raw piece starts at 0");
  }
  Ptrs<0> wire;
  int Kw = 0;
  const float* raw = nullptr;
  for (int k = 0; k < a.K; ++k) {
    if (pieces && k == a.raw_index) continue;  // given piecewise
    const uintptr_t p = reinterpret_cast<uintptr_t>(a.contribs[k]);
    if (p == 0) return fail(FRG_ERR_INVALID, "null contribution " + std::to_string(k));
    const uintptr_t elsize = k == a.raw_index ? 4 : 2;
    if (p % elsize != 0) {
      return fail(FRG_ERR_INVALID, "contribution " + std::to_string(k) + " not element-aligned");
    }
    const uintptr_t bytes = static_cast<uintptr_t>(a.n) * elsize;
    // the output may be a contribution of its own element size, exactly in place
    const bool inPlace = p == o && elsize == outElsize;
    if (!inPlace && p < o + outBytes && o < p + bytes) {
      return fail(FRG_ERR_INVALID, "output overlaps contribution " + std::to_string(k));
    }
    want(p, elsize);
    if (k == a.raw_index) {
      raw = static_cast<const float*>(a.contribs[k]);
    } else {
      wire.p[Kw++] = a.contribs[k];
    }
  }
  for (int k = Kw; k < kMaxContribsPerLaunch; ++k) wire.p[k] = Kw > 0 ? wire.p[0] : a.out;
  // the own term goes in ahead of wire contribution rawPos
  const int rawPos = a.raw_index;

  int64_t head = 0, nvec = 0, tail = 0;
  if (headWire >= 0 && headF32 >= 0 && headWire % 4 != headF32) vectorOk = false;
  if (vectorOk) {
    head = headWire >= 0 ? headWire : headF32;
    if (head > a.n) head = a.n;
    nvec = (a.n - head) / 8;
    tail = a.n - head - nvec * 8;
    // a lane's group of 8 must lie within one tensor of the raw term
    for (int i = 1; i < a.num_raw_pieces && pieces; ++i) {
      const int64_t at = a.raw_pieces[i].off;
      if (at > head && at < head + nvec * 8 && (at - head) % 8 != 0) vectorOk = false;
    }
    if (!vectorOk) head = nvec = tail = 0;
  }

  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return fail(FRG_ERR_HIP, "hipGetDevice failed");
  const int numCus = computeUnits(device);
  hipError_t e;
  if (pieces) {
    RawPieces table;
    for (int i = 0; i < kMaxRawPieces; ++i) {
      const bool used = i < a.num_raw_pieces;
      table.adj[i] = reinterpret_cast<const float*>(virtualOrigin(a.raw_pieces[used ? i : 0]));
      table.off[i] = used ? static_cast<int>(a.raw_pieces[i].off) : std::numeric_limits<int>::max();
    }
    e = a.wire_dtype == FRG_BF16
            ? dispatchOut<Bf16Vec, Bf16Scalar, RawPieces>(a, table, true, o, wire, Kw, rawPos, head,
                                                          nvec, tail, numCus, stream)
            : dispatchOut<F16Vec, F16Scalar, RawPieces>(a, table, true, o, wire, Kw, rawPos, head,
                                                        nvec, tail, numCus, stream);
  } else {
    const RawPlain plain{raw};
    const uintptr_t ref = reinterpret_cast<uintptr_t>(raw);
    e = a.wire_dtype == FRG_BF16
            ? dispatchOut<Bf16Vec, Bf16Scalar, RawPlain>(a, plain, raw != nullptr, ref, wire, Kw,
                                                         rawPos, head, nvec, tail, numCus, stream)
            : dispatchOut<F16Vec, F16Scalar, RawPlain>(a, plain, raw != nullptr, ref, wire, Kw,
                                                       rawPos, head, nvec, tail, numCus, stream);
  }
  if (e != hipSuccess) {
    return fail(FRG_ERR_HIP, std::string("kernel launch failed: ") + hipGetErrorString(e));
  }
  return FRG_OK;
}

// Whether a launch over `n` elements at `out` / `contribs` can take the raw
// term from these tensors at full speed (launchCompressedReduce takes them
// either way; tensors that start within a lane's group of 8 elements, or off
// the others' 16-byte phase, send it down the element-wise variant).
bool rawPiecesVectorize(const void* out, int outDtype, const void* const* contribs, int K,
                        int rawIndex, const RawPiece* pieces, int count, int64_t n) {
  if (count < 1 || count > kMaxRawPieces || n > std::numeric_limits<int>::max()) return false;
  const uintptr_t outElsize = outDtype == FRG_F32 ? 4 : 2;
  int64_t headWire = -1, headF32 = -1;
  bool ok = true;
  auto want = [&](uintptr_t p, uintptr_t elsize) {
    const int64_t h = static_cast<int64_t>(((16 - (p & 15)) & 15) / elsize);
    int64_t& slot = elsize == 2 ? headWire : headF32;
    if (slot < 0) {
      slot = h;
    } else if (slot != h) {
      ok = false;
    }
  };
  want(reinterpret_cast<uintptr_t>(out), outElsize);
  for (int k = 0; k < K; ++k) {
    if (k != rawIndex) want(reinterpret_cast<uintptr_t>(contribs[k]), 2);
  }
  for (int i = 0; i < count; ++i) want(virtualOrigin(pieces[i]), 4);
  if (headWire >= 0 && headF32 >= 0 && headWire % 4 != headF32) ok = false;
  if (!ok) return false;
  const int64_t head = headWire >= 0 ? headWire : headF32;
  const int64_t nvec = n > head ? (n - head) / 8 : 0;
  for (int i = 1; i < count; ++i) {
    const int64_t at = pieces[i].off;
    if (at > head && at < head + nvec * 8 && (at - head) % 8 != 0) return false;
  }
  return true;
}

}  // namespace frg
