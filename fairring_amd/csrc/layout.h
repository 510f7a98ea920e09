// Integer layout and slicing rules of the staging pool (host only, no GPU).
//
// computeLayout follows fairring/utils.h:288-327, the helpers follow
// fairring/utils.h:258-279, the slicing follows fairring/device.cc:315-326.
#pragma once

#include <stdint.h>

#include <limits>

namespace frg {

// Every slot and slice holds a whole number of elements of any supported type;
// 8 bytes (a double) is the widest (fairring/utils.h:276-279).
constexpr int64_t kAlignment = 8;

constexpr int64_t kDefaultTotalMemory = 50ll * 1024 * 1024;   // fairring/__init__.py:26
constexpr int64_t kDefaultPaddingMemory = 1024ll * 1024;      // fairring/__init__.py:30
constexpr int64_t kDefaultParallelism = 16;                   // fairring/__init__.py:34
// Default bytes of one contribution per launch, by number of contributions.
// Measured on MI355X (fp32, two reduce streams, GB/s at 6.25 / 12.5 / 25 / 50 MiB):
// K = 2: 4,530 / 5,990 / 6,290 / 6,340; K = 4: 5,370 / 6,565 / 6,460 / 6,280;
// K = 8: 6,070 / 6,360 / 6,060 / - ; K = 16 (at 1.6 / 3.1 / 6.25 / 12.5 MiB): 4,930 /
// 5,340 / 6,220 / 6,110; K = 64 (0.4 / 1.6 / 3.1 / 12.5 MiB): 3,180 / 6,100 / 6,125 / 6,055.
// The 8-way fp32 sum (the variant that runs 3 blocks per CU) does better still
// with launches of three whole rounds of its 768-block grid, 9 MiB: 6,552 GB/s
// against 6,464 at 12.5 MiB (8 / 8.5 / 9.5 / 10 MiB: 6,505 / 6,461 / 6,527 / 6,468)
// on an operation large enough to be cut into many; operations of a bucket's
// size are best cut into launches that divide them (25 MiB: 2 x 12.5 MiB
// 6,259, 9 + 9 + 7 MiB 6,210), so the 9 MiB apply from 100 MiB per contribution
// (100 / 200 / 400 MiB operations: 6,462 / 6,458 / 6,445 against 6,359 / 6,380 /
// 6,370). bf16 and K = 4 do not share this (12.5 MiB is their best).
constexpr int64_t kDefaultMaxLaunchBytes = 25ll * 1024 * 1024 / 2;
constexpr int64_t kEightWayFp32LaunchBytes = 9ll * 1024 * 1024;
constexpr int64_t kEightWayFp32LaunchFrom = 100ll * 1024 * 1024;
inline constexpr int64_t defaultLaunchBytes(int numContribs, bool fp32Sum = false,
                                            int64_t bytesPerContrib = 0) {
  if (numContribs <= 2) return 50ll * 1024 * 1024;
  if (numContribs == 8 && fp32Sum && bytesPerContrib >= kEightWayFp32LaunchFrom) {
    return kEightWayFp32LaunchBytes;
  }
  if (numContribs <= 8) return kDefaultMaxLaunchBytes;
  const int64_t perContrib = 100ll * 1024 * 1024 / numContribs;
  const int64_t floor = 25ll * 1024 * 1024 / 8;  // 3.125 MiB
  return (perContrib > floor ? perContrib : floor) / 4096 * 4096;
}
// The 8-way reduction with compression folded in (2 blocks per CU, rounds of
// 2 MiB of wire per contribution) wants whole rounds, and more of them: 12.5 /
// 12 / 16 / 20 / 24 / 32 MiB of wire per contribution and launch ran at 6,222 /
// 6,304 / 6,345 / 6,340 / 6,209 / 6,109 GB/s (8 / 9 / 10 / 11 / 14 MiB: 6,307 /
// 6,262 / 6,293 / 6,272 / 6,285). A bucket of up to 24 MiB of wire is one launch.
constexpr int64_t kEightWayCompressedLaunchBytes = 16ll * 1024 * 1024;
constexpr int64_t kLaunchQuantumBytes = 4096;  // launch boundaries within a slice: the kernel's tile

inline constexpr int64_t ceilOfRatio(int64_t num, int64_t den) {
  return num == 0 ? 0 : (num - 1) / den + 1;
}

inline constexpr int64_t roundDownToNearestMultiple(int64_t val, int64_t factor) {
  return (val / factor) * factor;
}

inline constexpr int64_t roundUpToNearestMultiple(int64_t val, int64_t factor) {
  return ceilOfRatio(val, factor) * factor;
}

struct Layout {
  int64_t slotSizeInBytes = 0;
  int64_t sliceSizeInBytes = 0;
  int64_t numPaddingSlots = 0;
  int64_t numStagingSlots = 0;
};

// Returns 0 on success; 1 / 2 name the precondition the reference would
// terminate on (too little padding memory for the parallelism asked for /
// padding alone exceeding the pool).
inline int computeLayout(int64_t maxMemoryAllocatedInBytes,
                         int64_t maxPaddingAllocatedInBytes,
                         int64_t minParallelism, int64_t numMachines,
                         int64_t numDevicesPerMachine, Layout* out) {
  const int64_t unit = numDevicesPerMachine * numMachines * kAlignment;
  Layout l;
  l.numPaddingSlots = maxPaddingAllocatedInBytes / unit;
  if (minParallelism > l.numPaddingSlots) return 1;
  l.sliceSizeInBytes = std::numeric_limits<int64_t>::max();
  if (numDevicesPerMachine == 1) {
    const int64_t reserved = 2 * minParallelism * unit;
    if (reserved > maxMemoryAllocatedInBytes) return 2;
    l.slotSizeInBytes = roundDownToNearestMultiple(
        (maxMemoryAllocatedInBytes - reserved) / minParallelism, unit);
    l.sliceSizeInBytes = l.slotSizeInBytes * numDevicesPerMachine;
    l.numStagingSlots = minParallelism;
    l.numPaddingSlots = minParallelism;
  }
  *out = l;
  return 0;
}

inline int64_t numSlices(int64_t numel, int64_t sliceSizeInBytes, int64_t elsize) {
  return ceilOfRatio(numel, sliceSizeInBytes / elsize);
}

inline void sliceBounds(int64_t numel, int64_t sliceSizeInBytes, int64_t elsize,
                        int64_t idx, int64_t* offset, int64_t* size) {
  const int64_t maxElems = sliceSizeInBytes / elsize;
  *offset = idx * maxElems;
  const int64_t left = numel - *offset;
  *size = left < maxElems ? left : maxElems;
}

}  // namespace frg
