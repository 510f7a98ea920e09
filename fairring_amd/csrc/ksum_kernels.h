// Internal launcher of the K-way slice reduction kernels (gfx950).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <string>

namespace frg {

constexpr int kMaxContribsPerLaunch = 64;

// Bytes per element of an FRG_* dtype code, 0 for an unknown code.
int64_t elementSize(int dtype);
bool isFloating(int dtype);

struct ReduceArgs {
  void* out = nullptr;
  const void* const* contribs = nullptr;  // host array of K device pointers
  int K = 0;
  int64_t n = 0;  // elements
  int dtype = 0;  // an FRG_* dtype code
  int op = 0;     // FRG_SUM / FRG_MAX
  int scale_mode = 0;
  float scale = 1.0f;
  bool carry = false;  // a carried-in term is read first and takes part as term "-1"
  const void* carry_src = nullptr;  // where it is read from; null = `out` itself
  // bf16 / fp16 SUM only: the carried-in term is read from, or the result is
  // left in, a buffer of fp32 accumulators (unrounded, unscaled), so that a
  // chain of launches rounds once, at its end.
  bool carry_acc = false;
  bool out_acc = false;
  // Blocks of the persistent grid per CU; 0 = the kernel's own rule. The
  // pipeline sets it together with the launch size (whole rounds of the grid).
  int blocks_per_cu = 0;
  // Bytes of the slice ahead of the first tile of the rounds; -1 = the kernel's
  // own rule (up to the first 4 KiB boundary of the first contribution). The
  // pipeline starts the rounds where the output reaches a 4 MiB boundary of its
  // allocation.
  int64_t lead_bytes = -1;
  // The whole tiles in the form that mixes the loads of a lane's two vectors
  // (sums of 2, 4 or 8 contributions without a carry; no scale, the multiply
  // by 1/K or every term times 1/K; ignored elsewhere): for contributions that lie close to one
  // another (closelySpaced() below), which run through memory in step. Same
  // result either way.
  bool mixed_loads = false;
  // Optional timing events (created with timing enabled) that receive the
  // begin and end timestamps of this launch.
  hipEvent_t startEvent = nullptr;
  hipEvent_t stopEvent = nullptr;
};

// Whether the contributions of an operation lie close to one another in the
// address space: the median distance between neighbours (of the distinct
// addresses, in ascending order) is below 768 MiB. Tensors that close run
// through memory in step and want ReduceArgs::mixed_loads; tensors further
// apart are better off without. Measured on MI355X, 8-way fp32, operations of
// 64 MiB, mixed against plain loads: tensors 64 MiB apart +4.5 %, 512 MiB
// +2.0 %, 1 GiB -3.5 %, 2 GiB -1.8 %; whole tensors of 1 GiB +0.1 %, of 1.5 GiB
// -2.2 %, of 5.5 GB -1.4 %.
constexpr uint64_t kMixedLoadsSpacingBytes = 768ull << 20;
inline bool closelySpaced(const void* const* ptrs, int K) {
  uint64_t a[64];
  int n = 0;
  for (int k = 0; k < K && n < 64; ++k) a[n++] = reinterpret_cast<uint64_t>(ptrs[k]);
  // insertion sort, then the distinct ones (an output that is also a contribution)
  for (int i = 1; i < n; ++i) {
    const uint64_t v = a[i];
    int j = i - 1;
    for (; j >= 0 && a[j] > v; --j) a[j + 1] = a[j];
    a[j + 1] = v;
  }
  uint64_t gaps[64];
  int g = 0;
  for (int i = 1; i < n; ++i) {
    if (a[i] != a[i - 1]) gaps[g++] = a[i] - a[i - 1];
  }
  if (g == 0) return false;
  for (int i = 1; i < g; ++i) {
    const uint64_t v = gaps[i];
    int j = i - 1;
    for (; j >= 0 && gaps[j] > v; --j) gaps[j + 1] = gaps[j];
    gaps[j + 1] = v;
  }
  return gaps[g / 2] < kMixedLoadsSpacingBytes;
}

// Where inside a scratch region a chain of launches parks its partial result so
// that the vector variant of the kernel still runs: at the same position within
// 16 bytes as `like` for a buffer of the storage type, or, for fp32 accumulators
// of a 2-byte type (`acc`), such that it reaches a 16-byte boundary after as
// many elements as `like` does. `base` is 16-byte aligned and the region has 16
// bytes to spare.
inline char* placeInScratch(char* base, const void* like, bool acc, int64_t elsize) {
  const uintptr_t pos = reinterpret_cast<uintptr_t>(like) & 15;
  if (!acc) return base + pos;
  const uintptr_t headElems = ((16 - pos) & 15) / static_cast<uintptr_t>(elsize);
  return base + ((16 - (4 * headElems) % 16) % 16);
}

// Validates the arguments, picks the kernel variant that fits K and the
// pointers' alignment, and enqueues one launch on `stream`. Returns an FRG_*
// status; on failure `err` says why. Never synchronises.
int launchReduce(const ReduceArgs& args, hipStream_t stream, std::string* err);

// ---- one launch over several pieces ------------------------------------------
//
// A piece is an elementwise reduction of its own: an output, K contributions
// and a length, anywhere in memory. A segmented launch runs up to
// maxSegmentsPerLaunch(K) pieces with the same K, element type and scale as one
// kernel launch: the tiles of all pieces are dealt to one persistent grid, so a
// bucket whose own contribution lies scattered over many gradient tensors (one
// piece per tensor), or the odds and ends of several operations, cost one
// launch instead of one per piece. SUM of fp32, bf16 or fp16, up to
// kMaxSegmentContribs contributions, nothing carried in; every pointer of a
// piece must sit at the same position within 16 bytes (segmentable() says
// whether a piece qualifies; what does not goes through launchReduce).
struct SegPiece {
  void* out = nullptr;
  const void* const* contribs = nullptr;  // host array of K device pointers
  int64_t n = 0;                          // elements
};

constexpr int kMaxSegmentContribs = 16;
inline constexpr int maxSegmentsPerLaunch(int K) { return K <= 8 ? 24 : 12; }

struct SegmentedArgs {
  const SegPiece* pieces = nullptr;
  int numPieces = 0;
  int K = 0;
  int dtype = 0;
  int scale_mode = 0;
  float scale = 1.0f;
  int blocks_per_cu = 0;  // 0 = 4 per CU
  hipEvent_t startEvent = nullptr;
  hipEvent_t stopEvent = nullptr;
};

// The kernel's tile: 256 vectors of 16 bytes of every contribution.
constexpr int64_t kSegmentTileVectors = 256;
constexpr int64_t kSegmentTileBytes = kSegmentTileVectors * 16;

// Whether a reduction of this kind can be part of a segmented launch at all.
inline bool segmentedKind(int K, int dtype, int op, bool carry) {
  // FRG_F32 = 0, FRG_BF16 = 1, FRG_F16 = 2; FRG_SUM = 0
  return K >= 1 && K <= kMaxSegmentContribs && op == 0 && !carry && dtype >= 0 && dtype <= 2;
}

// Whether a piece can: its pointers sit at one position within 16 bytes.
inline bool segmentable(const void* out, const void* const* contribs, int K, int64_t elsize) {
  const uintptr_t o = reinterpret_cast<uintptr_t>(out);
  if (o % static_cast<uintptr_t>(elsize) != 0) return false;
  for (int k = 0; k < K; ++k) {
    if ((reinterpret_cast<uintptr_t>(contribs[k]) & 15) != (o & 15)) return false;
  }
  return true;
}

// How the kernel walks such a piece: [head scalars][nvec vectors][tail
// scalars], the first `lead` vectors (those ahead of the first 4 KiB boundary of
// the output) as a tile of their own, whole tiles behind it, the last one
// possibly partial.
struct PieceSplit {
  int64_t head = 0, nvec = 0, tail = 0, lead = 0, tiles = 0;
};

inline PieceSplit splitPiece(const void* out, int64_t n, int64_t elsize) {
  const int64_t lanes = 16 / elsize;
  const uintptr_t o = reinterpret_cast<uintptr_t>(out);
  PieceSplit p;
  p.head = static_cast<int64_t>(((16 - (o & 15)) & 15) / static_cast<uintptr_t>(elsize));
  if (p.head > n) p.head = n;
  p.nvec = (n - p.head) / lanes;
  p.tail = n - p.head - p.nvec * lanes;
  const uintptr_t first = o + static_cast<uintptr_t>(p.head * elsize);
  const uintptr_t mask = static_cast<uintptr_t>(kSegmentTileBytes) - 1;
  p.lead = static_cast<int64_t>(((static_cast<uintptr_t>(kSegmentTileBytes) - (first & mask)) & mask) / 16);
  if (p.lead > p.nvec) p.lead = p.nvec;
  p.tiles = (p.lead > 0 ? 1 : 0) + (p.nvec - p.lead + kSegmentTileVectors - 1) / kSegmentTileVectors;
  if (p.tiles == 0 && n > 0) p.tiles = 1;  // scalars only: still a piece of the launch
  return p;
}

// Tiles the kernel deals for a piece, and the elements of the piece ahead of
// its tile `tile` (0 for the first): where a piece may be cut in two.
inline int64_t segmentTiles(const void* out, int64_t n, int64_t elsize) {
  return n > 0 ? splitPiece(out, n, elsize).tiles : 0;
}

inline int64_t segmentTileStart(const void* out, int64_t n, int64_t elsize, int64_t tile) {
  if (tile <= 0) return 0;
  const PieceSplit sp = splitPiece(out, n, elsize);
  const int64_t vec = sp.lead > 0 ? sp.lead + (tile - 1) * kSegmentTileVectors
                                  : tile * kSegmentTileVectors;
  const int64_t start = sp.head + vec * (16 / elsize);
  return start < n ? start : n;
}

int launchSegmented(const SegmentedArgs& args, hipStream_t stream, std::string* err);

// Launch-shape knobs (process-wide); 0 keeps the default.
void setTuning(int blocksPerCu);
// log2 of the consecutive 4 KiB tiles the blocks of one XCD take in a row (6 by
// default: 256 KiB; 0: tile = block index). For measurements.
void setXcdChunkShift(int shift);
int xcdChunkShift();
// Which launches take the mixed form of the main loop: -1 (default) those whose
// ReduceArgs ask for it, 0 none, 1 every launch that has the form. For
// measurements and tests.
void setMixedLoads(int mode);

// Compute units of a device (cached).
int computeUnits(int device);

// The persistent grid for `nvec` 16-byte vectors per contribution: `grid`
// blocks, `roundTiles` full tiles dealt in whole rounds of the grid, and what
// is left dealt in `pieces` smaller pieces. A positive hint fixes the blocks per
// CU unless the process-wide tuning knob is set.
struct GridPlan {
  int64_t grid = 1;
  int64_t roundTiles = 0;
  int64_t pieces = 0;
};
GridPlan planGrid(int64_t nvec, int numContribs, int numCus, int blocksPerCuHint = 0);

// The reduction around torch's gradient-compression hooks: peers' tensors in
// the wire type (bf16 or fp16), this rank's own fp32 buffer compressed in
// registers, the result stored in the wire type or widened into fp32.
// A tensor of the raw fp32 contribution and the element of the launch it starts at.
struct RawPiece {
  const void* ptr = nullptr;
  int64_t off = 0;
};
constexpr int kMaxRawPiecesPerLaunch = 8;
bool rawPiecesVectorize(const void* out, int outDtype, const void* const* contribs, int K,
                        int rawIndex, const RawPiece* pieces, int count, int64_t n);

struct CompressedArgs {
  void* out = nullptr;
  int out_dtype = 0;                      // FRG_F32 or the wire dtype
  const void* const* contribs = nullptr;  // host array of K device pointers
  int K = 0;
  int raw_index = -1;  // which contribution is raw fp32 (-1: none)
  int64_t n = 0;
  int wire_dtype = 0;  // FRG_BF16 / FRG_F16
  int scale_mode = 0;  // applied to the raw contribution after the cast: NONE / MUL / DIV
  float scale = 1.0f;
  // The raw contribution in up to kMaxRawPiecesPerLaunch tensors instead of one
  // buffer (contribs[raw_index] is then ignored): in order, the first at
  // element 0, every one up to where the next starts (the last up to n).
  const RawPiece* raw_pieces = nullptr;
  int num_raw_pieces = 0;
  hipEvent_t startEvent = nullptr;
  hipEvent_t stopEvent = nullptr;
};
int launchCompressedReduce(const CompressedArgs& args, hipStream_t stream, std::string* err);

}  // namespace frg
