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
  // Optional timing events (created with timing enabled) that receive the
  // begin and end timestamps of this launch.
  hipEvent_t startEvent = nullptr;
  hipEvent_t stopEvent = nullptr;
};

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

// Launch-shape knobs (process-wide); 0 keeps the default.
void setTuning(int blocksPerCu);

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
  hipEvent_t startEvent = nullptr;
  hipEvent_t stopEvent = nullptr;
};
int launchCompressedReduce(const CompressedArgs& args, hipStream_t stream, std::string* err);

}  // namespace frg
