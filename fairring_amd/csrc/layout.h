// Integer layout and slicing rules of the staging pool (host only, no GPU).
//
// computeLayout follows fairring/utils.h:288-327, the helpers follow
// fairring/utils.h:258-279, the slicing follows fairring/device.cc:315-326.
#pragma once

#include <stdint.h>

#include <stddef.h>

#include <limits>
#include <utility>
#include <vector>

namespace frg {

// Every slot and slice holds a whole number of elements of any supported type;
// 8 bytes (a double) is the widest (fairring/utils.h:276-279).
constexpr int64_t kAlignment = 8;

constexpr int64_t kDefaultTotalMemory = 50ll * 1024 * 1024;   // fairring/__init__.py:26
constexpr int64_t kDefaultPaddingMemory = 1024ll * 1024;      // fairring/__init__.py:30
constexpr int64_t kDefaultParallelism = 16;                   // fairring/__init__.py:34
// Default shape of a launch of the plain reduction: bytes of one contribution
// per launch and blocks of the persistent grid per CU (0 = the kernel's own
// rule), by number of contributions and size of the operation. All figures
// measured on MI355X (256 CUs, 4 KiB of every contribution per block and step,
// two reduce streams), GB/s of algorithmic bytes in one process unless noted.
//
// A launch should be a whole number of rounds of its grid, and the grid 4
// blocks per CU (1024 blocks, rounds of 4 MiB), with about 80 MB moved per
// launch:
//   K = 4:  12.5 MiB 6,528 | 4 blocks, 12 / 16 MiB 6,570 / 6,565
//   K = 5:  12.5 MiB (3 blocks) 6,558 | 4 blocks, 8 / 12 MiB 6,562 / 6,627
//   K = 6:  12.5 MiB (2 blocks) 6,378 | 4 blocks, 8 / 12 MiB 6,596 / 6,569
//   K = 7:  12.5 MiB (2 blocks) 6,023 | 4 blocks, 8 / 12 MiB 6,560 / 6,628
//   K = 8 fp32: 3 blocks, 9 / 12.5 MiB 6,549 / 6,464 | 4 blocks, 4 / 8 / 12 / 16 MiB
//           6,256 / 6,600 / 6,546 / 6,486; first process on a fresh box, whole job:
//           6,457 (3 blocks, 12.5 MiB), 6,530 (3 blocks, 9 MiB), 6,580 (4 blocks, 8 MiB)
//   K = 8 bf16, fresh box, whole job: 6,394 (2 blocks, 12.5 MiB), 6,593 (4 blocks, 8 MiB)
//   K = 9:  2 blocks, 11 MiB 6,090 | 4 blocks, 4 / 8 / 12 MiB 5,643 / 6,640 / 6,557
//   K = 10: 2 blocks, 10 MiB 6,308 | 4 blocks, 4 / 8 MiB 5,896 / 6,662
//   K = 12: 2 blocks, 8.3 MiB 6,194 | 4 blocks, 4 / 8 / 12 MiB 6,418 / 6,574 / 6,445
//   K = 14: 4 blocks, 4 / 8 / 12 MiB 6,405 / 6,375 / 6,281
//   K = 16: 2 blocks, 6.25 MiB 6,302 | 4 blocks, 4 / 8 MiB 6,604 / 6,528
//   K = 32: 2 blocks, 3.1 MiB 5,550 | 4 blocks, 4 / 8 / 12 MiB 6,428 / 6,348 / 6,265
//   K = 64: 2 blocks, 3.1 MiB 5,968 | 4 blocks, 4 / 8 MiB 6,552 / 6,481
// (more than 8 contributions are loaded 8 at a time, several dependent load
// phases per tile, which the additional waves hide).
// (Operations of a DDP bucket's size: see LaunchShape below.)
// K = 3 (5 blocks per CU, rounds of 5 MiB): 12.5 MiB 6,395, 15 / 20 / 25 MiB 6,526-6,596 /
// 6,571 / 6,552; 6 blocks, 12 / 18 / 24 MiB 6,113 / 6,365 / 6,343; 4 blocks, 16 MiB 6,235.
// K <= 2 (8 blocks per CU, rounds of 8 MiB): 48 / 50 / 56 MiB 6,450 / 6,407 / 6,433; another
// process: 8 blocks, 32 / 48 / 64 MiB 6,284 / 6,314 / 6,285; 6 blocks, 24 / 48 MiB 6,395 /
// 6,436; 4 blocks, 16 / 32 / 48 MiB 5,753 / 6,394 / 6,208.
//
// From 4 contributions on, operations of every size are cut by planAlignedLaunches
// (below): whole rounds of the 4-blocks-per-CU grid placed where the output's
// allocation has its 4 MiB multiples.
struct LaunchShape {
  int64_t bytes = 0;
  int blocksPerCu = 0;
  // cut the operation with planAlignedLaunches, `bytes` being the size aimed at
  bool wholeRounds = false;
};
constexpr int64_t kTileBytes = 4096;  // of every contribution, per block and step of the kernel
constexpr int64_t kDefaultMaxLaunchBytes = 25ll * 1024 * 1024 / 2;
constexpr int64_t kWholeRoundBytes = 4ll * 1024 * 1024;     // 256 CUs x 4 blocks x 4 KiB
constexpr int64_t kWholeRoundsFrom = 100ll * 1024 * 1024;   // per contribution, up to 8 of them
constexpr int64_t kBytesPerLaunchTarget = 80ll * 1024 * 1024;
inline constexpr LaunchShape defaultLaunchShape(int numContribs, int64_t bytesPerContrib) {
  const bool large = bytesPerContrib >= kWholeRoundsFrom;
  if (numContribs <= 2) return LaunchShape{48ll * 1024 * 1024, large ? 6 : 0};
  if (numContribs == 3) return LaunchShape{large ? 20ll * 1024 * 1024 : kDefaultMaxLaunchBytes, 0};
  // whole rounds nearest to the target, at least one
  const int64_t perContrib = kBytesPerLaunchTarget / (numContribs + 1);
  int64_t rounds = (perContrib + kWholeRoundBytes / 2) / kWholeRoundBytes;
  if (rounds < 1) rounds = 1;
  return LaunchShape{rounds * kWholeRoundBytes, 4, true};
}

// One launch of a partition: its share of every contribution, the grid it runs
// on and the bytes it takes ahead of its first round.
struct LaunchPart {
  int64_t bytes = 0;
  int blocksPerCu = 0;     // 0: the kernel's own rule
  int64_t leadBytes = -1;  // -1: the kernel's own rule (up to the first 4 KiB boundary)
};

// A round of the 4-blocks-per-CU grid: 4 MiB of every contribution on MI355X.
inline constexpr int64_t alignedRoundBytes(int numCus) {
  return static_cast<int64_t>(numCus) * 4 * kTileBytes;
}

// Cuts `bytes` of every contribution into launches of whole rounds of the
// 4-blocks-per-CU grid whose rounds all start `leadBytes` into the operation and
// at multiples of a round from there. What matters is where the rounds lie in
// memory: a round sweeps one window of 4 MiB per buffer, and on MI355X the rate
// depends on where the OUTPUT's windows start relative to the start of its
// allocation, with a period of 4 MiB (8-way fp32, one process, nine buffers
// carved from one allocation at these offsets: all on a 4 MiB multiple 6,576
// GB/s; all 1 MiB past one 6,280; all 2 MiB past one 6,205; the inputs on one
// and the output 2 MiB past 6,322; the inputs 2 MiB past and the output on one
// 6,508; half the inputs 2 MiB past 6,596). The caller therefore passes as
// `leadBytes` the distance from the operation's start to where the output next
// reaches such a multiple: those bytes go to the first launch as extra pieces
// ahead of its rounds, the launches take `targetBytes` worth of rounds each
// (what is left over one more on the last ones), and the bytes behind the last
// whole round go to the last launch as remainder pieces. An operation of fewer
// than two rounds is one launch on the kernel's own grid.
inline std::vector<LaunchPart> planAlignedLaunches(int64_t bytes, int64_t leadBytes,
                                                   int64_t targetBytes, int numCus) {
  const int64_t round = alignedRoundBytes(numCus);
  std::vector<LaunchPart> parts;
  const int64_t body = bytes - leadBytes;
  const int64_t rounds = body > 0 ? body / round : 0;
  if (rounds < 2) {
    parts.push_back(LaunchPart{bytes, 0, -1});
    return parts;
  }
  int64_t perLaunch = (targetBytes + round / 2) / round;
  if (perLaunch < 1) perLaunch = 1;
  int64_t launches = rounds / perLaunch;
  if (launches < 1) launches = 1;
  int64_t extra = rounds - launches * perLaunch;  // rounds no launch has yet
  for (int64_t i = 0; i < launches; ++i) {
    // the extra rounds go one each to the last launches (all to the last one
    // when there are more of them than launches)
    int64_t mine = perLaunch;
    if (launches - i <= extra) mine += 1;
    parts.push_back(LaunchPart{mine * round, 4, -1});
  }
  int64_t given = 0;
  for (const LaunchPart& p : parts) given += p.bytes;
  parts.back().bytes += rounds * round - given;
  parts.front().bytes += leadBytes;
  parts.front().leadBytes = leadBytes;
  parts.back().bytes += body - rounds * round;
  return parts;
}

// Where the rounds of an operation start: `outOffset` is the output's distance
// from the start of its allocation, `firstContrib` the address of the first
// contribution (the kernel keeps its tiles on 4 KiB boundaries of that one).
// The result is the number of bytes ahead of the first round: up to the next
// multiple of a round in the output, moved back to the 4 KiB grid of the first
// contribution where the two disagree.
inline int64_t alignedLeadBytes(uint64_t outOffset, uint64_t firstContrib, int numCus) {
  const uint64_t round = static_cast<uint64_t>(alignedRoundBytes(numCus));
  const uint64_t toRound = (round - outOffset % round) % round;
  const uint64_t toTile = (kTileBytes - firstContrib % kTileBytes) % kTileBytes;
  return static_cast<int64_t>(toTile + (toRound + round - toTile) % round / kTileBytes * kTileBytes);
}

// Launches of `size` bytes cut on multiples of the kernel's 4 KiB tile from the
// operation's start; the last one takes up to one and a half times that.
inline std::vector<LaunchPart> planEqualLaunches(int64_t bytes, int64_t size, int blocksPerCu) {
  std::vector<LaunchPart> parts;
  int64_t part = size / kTileBytes * kTileBytes;
  if (part < kTileBytes) part = (size + 15) / 16 * 16;  // below a tile: 16-byte boundaries
  int64_t off = 0;
  while (2 * (bytes - off) > 3 * part) {
    parts.push_back(LaunchPart{part, blocksPerCu, -1});
    off += part;
  }
  if (bytes > off || parts.empty()) parts.push_back(LaunchPart{bytes - off, blocksPerCu, -1});
  return parts;
}

// Whether the rounds of an operation can be put on the output's multiples of
// a round at little cost: at most a quarter of a round lies ahead of the first
// such multiple.
inline bool alignmentIsCheap(uint64_t outOffset, uint64_t firstContrib, int numCus) {
  const int64_t toTile = static_cast<int64_t>((kTileBytes - firstContrib % kTileBytes) % kTileBytes);
  return alignedLeadBytes(outOffset, firstContrib, numCus) - toTile <= alignedRoundBytes(numCus) / 4;
}
// An operation of this many rounds or more is aligned whatever lies ahead of its
// first multiple: the two partial ends are spread over enough whole rounds.
constexpr int64_t kAlwaysAlignFromRounds = 16;

// The launches of an operation over `bytes` of each of `numContribs`
// device-resident contributions when the caller asked for no launch size.
// Up to 3 contributions: equal launches of the shape's size. From 4 on: whole
// rounds (planAlignedLaunches) that start on the output's multiples of a round
// for an operation of 16 rounds or more, and for a shorter one when
// `alignShortOperations` says so and it is cheap (alignmentIsCheap). A shorter
// operation that starts further from a multiple (a bucket cut from the middle
// of a gradient) gains nothing from the alignment that the partial rounds at
// its ends do not take back (25 MiB buckets at offsets of 0 to 3 MiB from a
// multiple, one process: aligned 6,050 GB/s, equal halves on the kernel's own
// grid 6,290), and a stream of buckets that changes shape from one to the next
// loses more than the alignment gains (the same buckets, every fourth one
// aligned: 5,900; 28 MiB buckets that all sit on a multiple: 6,386 aligned,
// 6,236 in equal launches): the pipeline passes `alignShortOperations` only
// while the short operations it sees keep being cheap to align. Otherwise, up
// to 8 contributions, the operation is cut into equal launches of 12.5 MiB on
// the kernel's own grid, beyond that into whole rounds from its start.
inline std::vector<LaunchPart> planDefaultLaunches(int numContribs, int64_t bytes,
                                                   uint64_t outOffset, uint64_t firstContrib,
                                                   int numCus, bool alignShortOperations) {
  const LaunchShape shape = defaultLaunchShape(numContribs, bytes);
  if (!shape.wholeRounds) return planEqualLaunches(bytes, shape.bytes, shape.blocksPerCu);
  const int64_t round = alignedRoundBytes(numCus);
  const int64_t toTile = static_cast<int64_t>((kTileBytes - firstContrib % kTileBytes) % kTileBytes);
  const int64_t lead = alignedLeadBytes(outOffset, firstContrib, numCus);
  const bool large = (bytes - lead) / round >= kAlwaysAlignFromRounds;
  if (large || (alignShortOperations && alignmentIsCheap(outOffset, firstContrib, numCus))) {
    return planAlignedLaunches(bytes, lead, shape.bytes, numCus);
  }
  if (numContribs <= 8) return planEqualLaunches(bytes, kDefaultMaxLaunchBytes, 0);
  return planAlignedLaunches(bytes, toTile, shape.bytes, numCus);
}

// The reduction with compression folded in (2 blocks per CU, rounds of 2 MiB
// of wire per contribution; 3 and 4 blocks per CU are worse at every size)
// wants whole rounds too, and again about 80 MB per launch. 8-way hook (22
// bytes per element) on a whole gradient: 4 / 6 / 8 / 10 / 12 / 16 / 20 MiB of
// wire per contribution and launch ran at 6,456 / 6,562 / 6,613 / 6,568 / 6,534
// / 6,450 / 6,367 GB/s; 16-way (38 bytes): 2 / 4 / 8 / 12.5 MiB 5,217 / 6,100 /
// 6,104 / 5,902; 64-way (134 bytes): 2 / 4 / 8 / 12.5 MiB 6,292 / 6,087 / 5,966 /
// 5,798. A bucket of up to 8 contributions (25 MiB of fp32 = 12.5 MiB of wire)
// is best left as one launch: 6,167-6,185 against 5,441 cut 8 + 4.5 and 5,660 cut
// 6.25 + 6.25; so below 100 MiB of wire per contribution those take 16 MiB (one
// launch up to 24 MiB).
constexpr int64_t kCompressedRoundBytes = 2ll * 1024 * 1024;  // 256 CUs x 2 blocks x 4 KiB
constexpr int64_t kCompressedBucketLaunchBytes = 16ll * 1024 * 1024;
inline constexpr int64_t defaultCompressedLaunchBytes(int numContribs, bool rawTerm,
                                                      bool fp32Output, int64_t wireBytesPerContrib) {
  if (numContribs <= 8 && wireBytesPerContrib < kWholeRoundsFrom) {
    return kCompressedBucketLaunchBytes;
  }
  const int64_t bytesPerElem = 2 * static_cast<int64_t>(numContribs) + (rawTerm ? 2 : 0) +
                               (fp32Output ? 4 : 2);
  const int64_t perContrib = 2 * kBytesPerLaunchTarget / bytesPerElem;
  // rounded up: 32-way (70 bytes per element, 2.3 MiB) 2 / 4 / 6 MiB 5,852 / 6,176 / 6,066
  const int64_t rounds = (perContrib + kCompressedRoundBytes - 1) / kCompressedRoundBytes;
  return (rounds < 1 ? 1 : rounds) * kCompressedRoundBytes;
}
// An operation of at most this many launches runs on one reduce stream, and
// the next operation on the next stream; a longer one deals its launches over
// all of them. With the default shapes that is every operation below 100 MiB
// per contribution (8 launches of 12.5 MiB), where the whole-round shape begins.
constexpr int kOneStreamLaunches = 8;
constexpr int64_t kLaunchQuantumBytes = kTileBytes;  // launch boundaries within a slice: the kernel's tile

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
