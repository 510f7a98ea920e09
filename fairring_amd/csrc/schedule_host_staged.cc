// The schedule of an operation whose contributions lie in pinned host memory:
// copies into staging slots, folded into the output in index order.
#include "pipeline.h"

#include "ksum_kernels.h"
#include "pipeline_internal.h"

namespace frg {

// Contributions in pinned host memory (server-side accumulation,
// fairring/device.cc:543-589: collect into a staging slot, then reduce).
// Contribution 0 lands directly in `out`; the later ones are copied into
// staging slots and folded into `out` in index order.
//
// The pool's slots are split evenly among the staging streams (one by default,
// which then owns the whole pool), and a stream works through its share batch
// by batch: it copies a batch of contributions into its slots and then runs the
// fold that reads them, so a slot is never overwritten before its last reader
// has finished (the slot rule of device.cc:543-545,587-589) by stream order
// alone. What crosses streams, when there are several, is the order of the
// folds: each one waits for an event recorded behind the fold before it, when
// that ran on another stream. (Two streams, each copying under the other's
// fold, measured no faster than one: 53.9 against 54.3 GB/s. Two concurrent
// host copies share the link and end together.)
//
// (The folds used to run on a reduce stream, with a "filled" event from the copy
// stream to it and a "free" event back per slot. On MI355X / ROCm 7.2
// hipMemcpyAsync then held the calling thread up for 0.2 to 0.45 ms per copy, up
// to 11 ms, whenever the copy stream's last packet was such a wait, so the
// command thread paced the copies one at a time: 64 contributions of 25 MiB
// crossed the link at 46 to 50 GB/s. In this form the same call returns in 1.5
// us and the link runs at 54 of the 56 GB/s that bare copies get on the same
// box.)
std::vector<hipStream_t> Context::runHostStaged(const Request& req, hipEvent_t initialEvent) {
  const int64_t elsize = elementSize(req.dtype);
  // A staged slice must fit a slot as well as the slice size.
  int64_t sliceBytes =
      layout_.sliceSizeInBytes < slotBytes_ ? layout_.sliceSizeInBytes : slotBytes_;
  const int K = static_cast<int>(req.contribs.size());
  hipStream_t s = reduceStreams_[0];
  const std::vector<hipStream_t> all = copyStreams();  // created on first use
  // the pool is split evenly among the staging streams: each fills its share, then folds it
  int64_t batch = numSlots_ / static_cast<int64_t>(all.size());
  if (batch < 1) batch = 1;
  if (batch > kMaxContribsPerLaunch) batch = kMaxContribsPerLaunch;
  const int64_t groups = numSlots_ / batch;
  const size_t nStaging = static_cast<int64_t>(all.size()) < groups ? all.size()
                                                                    : static_cast<size_t>(groups);
  const std::vector<hipStream_t> staging(all.begin(), all.begin() + static_cast<long>(nStaging));
  // The staging streams write `out` and the slots and know nothing of earlier
  // operations: the whole operation is ordered after everything enqueued so far
  // (it is bound by the host link; a few event packets do not show).
  for (size_t src = 1; src < reduceStreams_.size(); ++src) {
    if (!history_[src].empty()) joinTail(src, 0);
  }
  {
    hipEvent_t tail = takeEvent();
    hipError_t r = hipEventRecord(tail, s);
    for (hipStream_t st : staging) {
      if (r == hipSuccess) r = hipStreamWaitEvent(st, tail, 0);
    }
    giveEvent(tail);
    FRG_HIP_CHECK(r);
  }
  bool initialFired = false;
  for (hipStream_t st : staging) waitInitial(st, initialEvent, &initialFired);
  // bf16 / fp16 sums folded in more than one batch keep their partial sums in
  // fp32 between the launches (one rounding, like a single launch); the slices
  // are then as short as the scratch buffer that holds those partial sums.
  const bool accChain = req.op == FRG_SUM && (req.dtype == FRG_BF16 || req.dtype == FRG_F16) &&
                        K - (req.carry ? 0 : 1) > batch;
  if (accChain && sliceBytes > carryScratchBytes_ / 4 * elsize) {
    sliceBytes = carryScratchBytes_ / 4 * elsize;
  }
  const int64_t nSlices = numSlices(req.numel, sliceBytes, elsize);

  // The fold enqueued last, anywhere: the stream it ran on and an event behind it.
  size_t lastFoldStream = nStaging;  // none yet
  hipEvent_t lastFold = nullptr;
  auto orderAfterLastFold = [&](size_t si) {
    if (lastFold != nullptr && lastFoldStream != si) {
      FRG_HIP_CHECK(hipStreamWaitEvent(staging[si], lastFold, 0));
    }
  };
  auto foldEnqueued = [&](size_t si) {
    giveEvent(lastFold);
    lastFold = nullptr;
    lastFold = takeEvent();
    lastFoldStream = si;
    FRG_HIP_CHECK(hipEventRecord(lastFold, staging[si]));
  };
  std::vector<char> took(nStaging, 0);
  try {
    for (int64_t i = 0; i < nSlices; ++i) {
      int64_t off, len;
      sliceBounds(req.numel, sliceBytes, elsize, i, &off, &len);
      const size_t bytes = static_cast<size_t>(len * elsize);
      char* outp = static_cast<char*>(req.out) + off * elsize;

      int firstStaged = 0;
      if (!req.carry) {
        // Contribution 0 needs no staging: it lands in `out` directly, on the
        // stream of the group that comes next, behind whatever fold wrote this
        // part of `out` last (none within this operation: the slices are
        // disjoint ranges; an earlier operation's is covered by the joins above).
        const size_t si = static_cast<size_t>((nextStagingSlot_ / batch) % groups) % nStaging;
        orderAfterLastFold(si);  // keeps the folds of all slices in one chain (they share the scratch)
        FRG_HIP_CHECK(hipMemcpyAsync(outp,
                                     static_cast<const char*>(req.contribs[0]) + off * elsize,
                                     bytes, hipMemcpyHostToDevice, staging[si]));
        took[si] = 1;
        firstStaged = 1;
        if (K == 1) {
          if (req.scaleMode != FRG_SCALE_NONE) {
            // nothing left to fold, but the post-scale is still owed
            const void* self = outp;
            ReduceArgs a;
            a.out = outp;
            a.contribs = &self;
            a.K = 1;
            a.n = len;
            a.dtype = req.dtype;
            a.op = req.op;
            a.scale_mode = req.scaleMode;
            a.scale = req.scale;
            launch(a, staging[si]);
          }
          continue;
        }
        // the first fold of the slice reads what this copy wrote
        giveEvent(lastFold);
        lastFold = nullptr;
        lastFold = takeEvent();
        lastFoldStream = si;
        FRG_HIP_CHECK(hipEventRecord(lastFold, staging[si]));
      }

      std::vector<const void*> staged;
      char* accBuf = accChain ? scratchFor(0, outp, /*acc=*/true, elsize) : nullptr;
      bool inAcc = false;  // the partial sum sits in accBuf (fp32), not in `out`
      for (int k = firstStaged; k < K;) {
        const int64_t group = (nextStagingSlot_ / batch) % groups;
        nextStagingSlot_ += batch;  // the rotation of fairring/device.cc:482, a group at a time
        const size_t si = static_cast<size_t>(group) % nStaging;
        hipStream_t st = staging[si];
        const int k0 = k;
        const int kn = K - k < batch ? K - k : static_cast<int>(batch);
        k += kn;
        // Two streams that start their copies together share the link, finish
        // together and then fold one after the other with the link idle (8 % of
        // the time with 25 MiB slots). The first batch of every stream but the
        // first therefore goes in two halves, copy and fold each: from then on
        // that stream's copies end half a copy apart from its neighbour's, and
        // one of them is always in flight.
        int64_t cuts[3] = {0, len, len};
        int parts = 1;
        if (si > 0 && !took[si] && bytes >= (4u << 20)) {
          cuts[1] = len / 2 / (kTileBytes / elsize) * (kTileBytes / elsize);
          parts = 2;
        }
        took[si] = 1;
        for (int part = 0; part < parts; ++part) {
          const int64_t lo = cuts[part], hi = cuts[part + 1];
          staged.clear();
          for (int j = 0; j < kn; ++j) {
            char* dst = stagingPool_ + (group * batch + j) * slotBytes_;
            FRG_HIP_CHECK(hipMemcpyAsync(
                dst + lo * elsize,
                static_cast<const char*>(req.contribs[k0 + j]) + (off + lo) * elsize,
                static_cast<size_t>((hi - lo) * elsize), hipMemcpyHostToDevice, st));
            staged.push_back(dst + lo * elsize);
          }
          orderAfterLastFold(si);
          ReduceArgs a;
          a.out = outp + lo * elsize;
          a.contribs = staged.data();
          a.K = kn;
          a.n = hi - lo;
          a.dtype = req.dtype;
          a.op = req.op;
          a.scale_mode = k == K ? req.scaleMode : FRG_SCALE_NONE;
          a.scale = req.scale;
          a.carry = true;
          if (accChain) {
            a.carry_src = inAcc ? accBuf + lo * 4 : outp + lo * elsize;
            a.carry_acc = inAcc;
            if (k < K) {  // more batches follow
              a.out = accBuf + lo * 4;
              a.out_acc = true;
            }
          }
          launch(a, st);
          foldEnqueued(si);
        }
        if (accChain && k < K) inAcc = true;
      }
    }
    // The operation ends on the first reduce stream, like any other: whatever
    // comes later is ordered against that.
    for (size_t si = 0; si < nStaging; ++si) {
      if (!took[si]) continue;
      hipEvent_t e = takeEvent();
      hipError_t r = hipEventRecord(e, staging[si]);
      if (r == hipSuccess) r = hipStreamWaitEvent(s, e, 0);
      giveEvent(e);
      FRG_HIP_CHECK(r);
    }
  } catch (...) {
    giveEvent(lastFold);
    throw;
  }
  giveEvent(lastFold);
  if (req.numel > 0) remember(spansOf(req), {0});
  return {s};
}

}  // namespace frg
