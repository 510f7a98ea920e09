// The schedule of an operation whose contributions all lie in device memory:
// launches dealt to the reduce streams, and the chain through scratch memory
// for more contributions than one launch takes.
#include "pipeline.h"

#include "ksum_kernels.h"
#include "pipeline_internal.h"

namespace frg {

// The scratch region of a reduce stream (reused in stream order), placed so that the vector variant of the kernel still runs:
// at the same position within 16 bytes as `like` for a buffer of the storage
// type, or, for fp32 accumulators of a 2-byte type, such that it reaches a
// 16-byte boundary after as many elements as `like` does.
char* Context::scratchFor(size_t streamIdx, const void* like, bool acc, int64_t elsize) {
  char* base = carryScratch_ + streamIdx * static_cast<size_t>(carryScratchBytes_ + 16);
  return placeInScratch(base, like, acc, elsize);
}

// One part of a slice with more contributions than a launch takes, chained
// through a scratch buffer in pieces of that buffer's size; only the last
// launch of each piece writes `out`. Needed where `out` is itself one of the
// contributions beyond the first launch's (the partial result must not land in
// it early), and for bf16 / fp16 sums (`acc`: the partial sums stay in fp32).
void Context::chainThroughScratch(const Request& req, const std::vector<const void*>& ptrs,
                                  int64_t off, int64_t len, size_t streamIdx, bool acc) {
  const int64_t elsize = elementSize(req.dtype);
  const int total = static_cast<int>(ptrs.size());
  hipStream_t s = reduceStreams_[streamIdx];
  char* outBase = static_cast<char*>(req.out) + off * elsize;
  char* scratch = scratchFor(streamIdx, acc ? ptrs[0] : outBase, acc, elsize);
  const int64_t pieceLen = carryScratchBytes_ / (acc ? 4 : elsize);
  std::vector<const void*> shifted(ptrs.size());
  for (int64_t q = 0; q < len; q += pieceLen) {
    const int64_t qlen = len - q < pieceLen ? len - q : pieceLen;
    for (size_t k = 0; k < ptrs.size(); ++k) {
      shifted[k] = static_cast<const char*>(ptrs[k]) + q * elsize;
    }
    for (int k0 = 0; k0 < total; k0 += kMaxContribsPerLaunch) {
      const int kn = total - k0 < kMaxContribsPerLaunch ? total - k0 : kMaxContribsPerLaunch;
      const bool lastLaunch = k0 + kn == total;
      ReduceArgs a;
      a.out = lastLaunch ? outBase + q * elsize : scratch;
      a.out_acc = acc && !lastLaunch;
      a.contribs = shifted.data() + k0;
      a.K = kn;
      a.n = qlen;
      a.dtype = req.dtype;
      a.op = req.op;
      a.scale_mode = (lastLaunch || req.scaleMode >= FRG_SCALE_PRE_MUL) ? req.scaleMode
                                                                        : FRG_SCALE_NONE;
      a.scale = req.scale;
      a.carry = k0 > 0;
      a.carry_src = scratch;
      a.carry_acc = acc;
      launch(a, s);
    }
  }
}

// Device-resident contributions: the tensor is cut into launches of the launch
// size (or one per slice of fairring/device.cc:315-326 when asked for), dealt
// round-robin to the reduce streams so that neighbouring launches overlap.
// Returns the streams the operation's work ended on.
std::vector<hipStream_t> Context::runResident(const Request& req,
                                              const std::vector<hipEvent_t>& initialEvents,
                                              int64_t slices) {
  const int64_t elsize = elementSize(req.dtype);
  const int64_t nSlices =
      slices >= 0 ? slices : numSlices(req.numel, layout_.sliceSizeInBytes, elsize);
  std::vector<char> initialsFired(initialEvents.size(), 0);
  // the first launch on a stream follows every producer's event
  auto waitInitials = [&](hipStream_t stream) {
    for (size_t i = 0; i < initialEvents.size(); ++i) {
      bool fired = initialsFired[i] != 0;
      waitInitial(stream, initialEvents[i], &fired);
      initialsFired[i] = fired ? 1 : 0;
    }
  };
  const size_t nStreams = reduceStreams_.size();
  std::vector<char> waited(nStreams, 0);
  std::vector<const void*> ptrs(req.contribs.size());
  const int total = static_cast<int>(ptrs.size());
  // Launch size and grid go together (whole rounds of the grid); a size asked
  // for by the caller leaves the grid to the kernel's own rule.
  LaunchShape shape{maxLaunchBytes_, 0};
  if (launchBytesByContribs_) {
    shape = req.compressed
                ? LaunchShape{defaultCompressedLaunchBytes(total, req.rawIndex >= 0,
                                                           req.outDtype == FRG_F32,
                                                           req.numel * elsize),
                              0}
                : defaultLaunchShape(total, req.numel * elsize);
  }
  const int64_t launchBytes = shape.bytes;
  const int64_t maxLaunchElems = launchBytes > 0 ? launchBytes / elsize : 0;
  size_t lastIdx = static_cast<size_t>(nextLaunch_) % nStreams;
  // Reduced in place into a contribution that only a later launch of the chain
  // reads: the partial result must not land in `out` before that.
  bool lateAlias = false;
  for (int k = kMaxContribsPerLaunch; k < total && !req.compressed; ++k) {
    if (req.contribs[k] == req.out) lateAlias = true;
  }
  // A chain over bf16 / fp16 contributions keeps its partial sums in fp32
  // between launches, so that it rounds once like a single launch.
  const bool accChain = !req.compressed && total > kMaxContribsPerLaunch && req.op == FRG_SUM &&
                        (req.dtype == FRG_BF16 || req.dtype == FRG_F16);

  // Every slice takes its turn in the slot rotation (fairring/device.cc:482),
  // but device-resident contributions need no slot, and the sum is elementwise:
  // the launches need not follow the slice boundaries. The tensor is cut into
  // launches of the launch size, on multiples of the kernel's 4 KiB tile from
  // its start (a launch that starts off a tile boundary measured 8 % slower),
  // whatever the slice size; the last launch takes up to one and a half times
  // that. With the default layout (16 slices of 3.1 MiB in flight) launches cut
  // at slice boundaries ran at 5.0 TB/s, these run at 6.3. A launch size of
  // "whole slice" (max_launch_bytes < 0) keeps one launch per slice.
  nextStagingSlot_ += nSlices;
  struct Range {
    int64_t first;   // offset in elements
    int64_t second;  // length in elements
    int blocksPerCu;
    int64_t leadBytes;
  };
  std::vector<Range> ranges;
  auto addRange = [&](int64_t off, int64_t len) {
    ranges.push_back(Range{off, len, shape.blocksPerCu, -1});
  };
  const bool identity = !req.compressed && total == 1 && req.contribs[0] == req.out &&
                        req.scaleMode == FRG_SCALE_NONE;
  if (identity) {
    // A lone contribution reduced in place: nothing to do (what the reference
    // does for one machine and one device: device.cc:523,569).
  } else if (maxLaunchElems <= 0) {
    for (int64_t i = 0; i < nSlices; ++i) {
      int64_t off, len;
      sliceBounds(req.numel, layout_.sliceSizeInBytes, elsize, i, &off, &len);
      addRange(off, len);
    }
  } else if (launchBytesByContribs_ && !req.compressed) {
    // no launch size asked for: the library's own partition (layout.h)
    const int numCus = computeUnits(device_);
    const uint64_t outOffset = (reinterpret_cast<uint64_t>(req.out) - allocationBase(req.out)) %
                               static_cast<uint64_t>(alignedRoundBytes(numCus));
    const uint64_t first = reinterpret_cast<uint64_t>(req.contribs[0]);
    const int64_t bytes = req.numel * elsize;
    // A stream of short operations keeps one launch shape: they are aligned
    // only once several in a row were cheap to align, and not again after one
    // that is not until as many have been.
    const bool shortOp = bytes / alignedRoundBytes(numCus) < kAlwaysAlignFromRounds;
    if (shortOp) {
      cheapStreak_ = alignmentIsCheap(outOffset, first, numCus) ? cheapStreak_ + 1 : 0;
    }
    const bool alignShort = cheapStreak_ > kAlignAfterStreak;
    if (bytes != planBytes_ || outOffset != planOutOffset_ || first % kTileBytes != planFirst_ ||
        total != planContribs_ || alignShort != planAlignShort_) {
      plan_ = planDefaultLaunches(total, bytes, outOffset, first, numCus, alignShort);
      planAlignShort_ = alignShort;
      planBytes_ = bytes;
      planOutOffset_ = outOffset;
      planFirst_ = first % kTileBytes;
      planContribs_ = total;
    }
    int64_t off = 0;
    for (const LaunchPart& p : plan_) {
      if (p.bytes > 0) ranges.push_back(Range{off, p.bytes / elsize, p.blocksPerCu, p.leadBytes});
      off += p.bytes / elsize;
    }
  } else {
    const int64_t quantum = kLaunchQuantumBytes / elsize;
    int64_t partLen = roundDownToNearestMultiple(maxLaunchElems, quantum);
    if (partLen < quantum) {  // launch sizes below a tile: 16-byte boundaries instead
      partLen = roundUpToNearestMultiple(maxLaunchElems, 16 / elsize);
    }
    int64_t off = 0;
    while (2 * (req.numel - off) > 3 * partLen) {
      addRange(off, partLen);
      off += partLen;
    }
    if (req.numel > off) addRange(off, req.numel - off);
  }

  // An operation of a few launches (a DDP bucket) stays on one stream and the
  // next operation takes the next stream: neighbouring operations overlap, each
  // ends on a single stream (nothing to join for its completion), and nothing is
  // recorded between two launches. A large operation deals its own launches
  // round-robin over the streams.
  const bool oneStream = ranges.size() <= static_cast<size_t>(oneStreamLaunches_);
  const size_t opStream = static_cast<size_t>(nextLaunch_) % nStreams;
  if (oneStream && !ranges.empty()) ++nextLaunch_;
  const OpSpans spans = spansOf(req);
  std::vector<size_t> targets;
  if (!ranges.empty()) {
    if (oneStream) {
      targets.push_back(opStream);
    } else {
      for (size_t si = 0; si < nStreams; ++si) targets.push_back(si);
    }
    orderAfterConflicts(spans, targets);
  }

  // Tensors that lie close to one another (a bucket's, allocated one by one)
  // run through memory in step: their launches mix the loads of a lane's two
  // vectors (8-way fp32, 48 buckets of 25 MiB: 6,45x GB/s against 6,37x). The
  // tensors of a whole gradient, gigabytes apart, do better without (-1.4 %).
  const bool mixedLoads =
      total <= kMaxContribsPerLaunch && closelySpaced(req.contribs.data(), total);

  for (const auto& range : ranges) {
    const int64_t off = range.first;
    const int64_t len = range.second;
    const size_t si = oneStream ? opStream : static_cast<size_t>(nextLaunch_++) % nStreams;
    hipStream_t s = reduceStreams_[si];
    if (!waited[si]) {
      // Only the first launch on a stream needs the producer's event; later
      // ones follow it in stream order (fairring/device.cc:334-336,507-509).
      waitInitials(s);
      waited[si] = 1;
    }
    for (size_t k = 0; k < ptrs.size(); ++k) {
      const int64_t es = (req.compressed && static_cast<int>(k) == req.rawIndex) ? 4 : elsize;
      ptrs[k] = static_cast<const char*>(req.contribs[k]) + off * es;
    }
    if (req.compressed) {
      CompressedArgs a;
      a.out = static_cast<char*>(req.out) + off * elementSize(req.outDtype);
      a.out_dtype = req.outDtype;
      a.contribs = ptrs.data();
      a.K = total;
      a.raw_index = req.rawIndex;
      a.n = len;
      a.wire_dtype = req.dtype;
      a.scale_mode = req.scaleMode;
      a.scale = req.scale;
      launchCompressed(a, s);
      lastIdx = si;
      continue;
    }
    if (lateAlias || accChain) {
      chainThroughScratch(req, ptrs, off, len, si, accChain);
      lastIdx = si;
      continue;
    }
    // More contributions than one launch takes: chain launches, carrying the
    // partial result in `out`; the post-scale goes on the last one only.
    for (int k0 = 0; k0 < total; k0 += kMaxContribsPerLaunch) {
      const int kn = total - k0 < kMaxContribsPerLaunch ? total - k0 : kMaxContribsPerLaunch;
      const bool lastLaunch = k0 + kn == total;
      ReduceArgs a;
      a.out = static_cast<char*>(req.out) + off * elsize;
      a.contribs = ptrs.data() + k0;
      a.K = kn;
      a.n = len;
      a.dtype = req.dtype;
      a.op = req.op;
      // a post-scale goes on the last launch only, a pre-scale on every one
      a.scale_mode = (lastLaunch || req.scaleMode >= FRG_SCALE_PRE_MUL) ? req.scaleMode
                                                                        : FRG_SCALE_NONE;
      a.scale = req.scale;
      a.carry = k0 > 0;
      a.blocks_per_cu = range.blocksPerCu;
      a.lead_bytes = range.leadBytes;
      a.mixed_loads = mixedLoads;
      launch(a, s);
    }
    lastIdx = si;
  }
  if (!ranges.empty()) {
    std::vector<size_t> ran;
    for (size_t si = 0; si < nStreams; ++si) {
      if (waited[si]) ran.push_back(si);
    }
    remember(spans, ran);
  }
  // The streams that took part, the one of the last launch at the back.
  if (!waited[lastIdx]) {
    waitInitials(reduceStreams_[lastIdx]);
    waited[lastIdx] = 1;
  }
  std::vector<hipStream_t> used;
  for (size_t si = 0; si < nStreams; ++si) {
    if (si != lastIdx && waited[si]) used.push_back(reduceStreams_[si]);
  }
  used.push_back(reduceStreams_[lastIdx]);
  return used;
}

}  // namespace frg
