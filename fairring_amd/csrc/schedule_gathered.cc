// The schedules of an operation with one contribution given piecewise (a
// bucket's own gradients, each still in its own tensor), plain and with a
// compression hook folded in.
#include "pipeline.h"

#include "ksum_kernels.h"
#include "pipeline_internal.h"

namespace frg {

// One contribution given piecewise (a bucket's own gradients, each still in its
// own tensor): the output is cut where the pieces end, every piece is an
// elementwise reduction of its own (the output and the other contributions at
// the piece's offset, the piece itself in the gathered contribution's place),
// and the pieces are packed into segmented launches, cut on 4 KiB tiles of the
// output, of about the size a plain operation's launches have. The copy of
// every gradient into the bucket that DDP makes ahead of the allreduce
// (torch:csrc/distributed/c10d/reducer.cpp, copy_grad_to_bucket) is thereby
// part of the reduction: 8 bytes per element of HBM traffic less. A piece whose
// pointers disagree modulo 16 (an odd-sized tensor ahead of it in the bucket),
// and any reduction the segmented kernel does not cover (MAX, more than 16
// contributions, other element types), runs as a plain launch of its own.
std::vector<hipStream_t> Context::runGathered(const Request& req,
                                              const std::vector<hipEvent_t>& initialEvents) {
  if (req.compressed) return runGatheredCompressed(req, initialEvents);
  const int64_t elsize = elementSize(req.dtype);
  const int total = static_cast<int>(req.contribs.size());
  const int g = req.gatheredIndex;
  nextStagingSlot_ += numSlices(req.numel, layout_.sliceSizeInBytes, elsize);
  const bool kindOk = segmentedKind(total, req.dtype, req.op, false);
  const int maxSegs = maxSegmentsPerLaunch(total);
  int64_t targetTiles = defaultLaunchShape(total, req.numel * elsize).bytes / kTileBytes;
  if (targetTiles < 1) targetTiles = 1;
  const bool accChain = total > kMaxContribsPerLaunch && req.op == FRG_SUM &&
                        (req.dtype == FRG_BF16 || req.dtype == FRG_F16);

  // A unit is one launch: several pieces through the segmented kernel, or one
  // piece through the plain one.
  struct Unit {
    bool segmented = true;
    std::vector<SegPiece> pieces;
    int64_t off = 0;  // plain: offset of the piece in the output
  };
  std::vector<Unit> units;
  std::deque<std::vector<const void*>> tables;  // the pieces' pointer tables stay put
  auto tableOf = [&](const Request::Segment& seg, int64_t off) {
    std::vector<const void*> tab(static_cast<size_t>(total));
    for (int k = 0; k < total; ++k) {
      tab[static_cast<size_t>(k)] =
          k == g ? seg.ptr
                 : static_cast<const char*>(req.contribs[static_cast<size_t>(k)]) + off * elsize;
    }
    return tab;
  };
  // Launches of `targetTiles` each, the last one with what is left over when
  // that is less than half a launch's worth: a bucket of 25 MiB is 8 + 8 + 9
  // MiB like a plain operation's, not three launches and a sliver.
  int64_t segmentedTiles = 0;
  {
    int64_t off = 0;
    for (const Request::Segment& seg : req.gathered) {
      if (seg.numel <= 0) continue;
      char* outp = static_cast<char*>(req.out) + off * elsize;
      const std::vector<const void*> tab = tableOf(seg, off);
      if (kindOk && segmentable(outp, tab.data(), total, elsize)) {
        segmentedTiles += segmentTiles(outp, seg.numel, elsize);
      }
      off += seg.numel;
    }
  }
  int64_t tilesLeft = segmentedTiles;  // not yet given to a launch
  Unit cur;
  int64_t curTiles = 0;
  auto flush = [&] {
    if (!cur.pieces.empty()) units.push_back(std::move(cur));
    cur = Unit();
    curTiles = 0;
  };
  int64_t off = 0;
  for (const Request::Segment& seg : req.gathered) {
    const int64_t len = seg.numel;
    if (len <= 0) continue;
    char* outp = static_cast<char*>(req.out) + off * elsize;
    std::vector<const void*> tab = tableOf(seg, off);
    if (!kindOk || !segmentable(outp, tab.data(), total, elsize)) {
      flush();
      tables.push_back(std::move(tab));
      Unit plain;
      plain.segmented = false;
      plain.off = off;
      plain.pieces.push_back(SegPiece{outp, tables.back().data(), len});
      units.push_back(std::move(plain));
      off += len;
      continue;
    }
    const int64_t tiles = segmentTiles(outp, len, elsize);
    for (int64_t t = 0; t < tiles;) {
      int64_t take = tiles - t;
      // a launch holds targetTiles, unless what would be left behind it is less
      // than half a launch's worth: then it takes that too
      const int64_t room = targetTiles - curTiles;
      const bool openEnded = tilesLeft - room < targetTiles / 2;
      if (!openEnded && take > room) take = room;
      const int64_t e0 = segmentTileStart(outp, len, elsize, t);
      const int64_t e1 = t + take == tiles ? len : segmentTileStart(outp, len, elsize, t + take);
      std::vector<const void*> part(static_cast<size_t>(total));
      for (int k = 0; k < total; ++k) {
        part[static_cast<size_t>(k)] = static_cast<const char*>(tab[static_cast<size_t>(k)]) + e0 * elsize;
      }
      tables.push_back(std::move(part));
      cur.pieces.push_back(SegPiece{outp + e0 * elsize, tables.back().data(), e1 - e0});
      curTiles += take;
      tilesLeft -= take;
      t += take;
      if ((!openEnded && curTiles >= targetTiles) ||
          static_cast<int>(cur.pieces.size()) == maxSegs) {
        flush();
      }
    }
    off += len;
  }
  flush();

  const size_t nStreams = reduceStreams_.size();
  std::vector<char> initialsFired(initialEvents.size(), 0);
  auto waitInitials = [&](hipStream_t stream) {
    for (size_t i = 0; i < initialEvents.size(); ++i) {
      bool fired = initialsFired[i] != 0;
      waitInitial(stream, initialEvents[i], &fired);
      initialsFired[i] = fired ? 1 : 0;
    }
  };
  std::vector<char> waited(nStreams, 0);
  const bool oneStream = units.size() <= static_cast<size_t>(oneStreamLaunches_);
  const size_t opStream = static_cast<size_t>(nextLaunch_) % nStreams;
  size_t lastIdx = opStream;
  if (oneStream && !units.empty()) ++nextLaunch_;
  const OpSpans spans = spansOf(req);
  if (!units.empty()) {
    std::vector<size_t> targets;
    if (oneStream) {
      targets.push_back(opStream);
    } else {
      for (size_t si = 0; si < nStreams; ++si) targets.push_back(si);
    }
    orderAfterConflicts(spans, targets);
  }
  for (const Unit& u : units) {
    const size_t si = oneStream ? opStream : static_cast<size_t>(nextLaunch_++) % nStreams;
    hipStream_t s = reduceStreams_[si];
    if (!waited[si]) {
      waitInitials(s);
      waited[si] = 1;
    }
    lastIdx = si;
    if (u.segmented && u.pieces.size() == 1) {
      // A launch that holds one piece (a weight matrix fills whole launches on
      // its own) is the plain kernel's: its pointers sit in registers from the
      // start, where the segmented kernel first reads the table's prefix sums
      // and then the piece's row (two dependent loads ahead of every block's
      // first tile; 8 MiB launches of one piece: 3 % slower through the table).
      const SegPiece& one = u.pieces[0];
      ReduceArgs a;
      a.out = one.out;
      a.contribs = one.contribs;
      a.K = total;
      a.n = one.n;
      a.dtype = req.dtype;
      a.op = req.op;
      a.scale_mode = req.scaleMode;
      a.scale = req.scale;
      a.blocks_per_cu = 4;
      a.mixed_loads = closelySpaced(one.contribs, total);  // see runResident
      launch(a, s);
      continue;
    }
    if (u.segmented) {
      SegmentedArgs a;
      a.pieces = u.pieces.data();
      a.numPieces = static_cast<int>(u.pieces.size());
      a.K = total;
      a.dtype = req.dtype;
      a.scale_mode = req.scaleMode;
      a.scale = req.scale;
      launchSegments(a, s);
      continue;
    }
    const SegPiece& pc = u.pieces[0];
    if (accChain) {
      std::vector<const void*> ptrs(pc.contribs, pc.contribs + total);
      chainThroughScratch(req, ptrs, u.off, pc.n, si, true);
      continue;
    }
    for (int k0 = 0; k0 < total; k0 += kMaxContribsPerLaunch) {
      const int kn = total - k0 < kMaxContribsPerLaunch ? total - k0 : kMaxContribsPerLaunch;
      const bool lastLaunch = k0 + kn == total;
      ReduceArgs a;
      a.out = pc.out;
      a.contribs = pc.contribs + k0;
      a.K = kn;
      a.n = pc.n;
      a.dtype = req.dtype;
      a.op = req.op;
      a.scale_mode = (lastLaunch || req.scaleMode >= FRG_SCALE_PRE_MUL) ? req.scaleMode
                                                                        : FRG_SCALE_NONE;
      a.scale = req.scale;
      a.carry = k0 > 0;
      launch(a, s);
    }
  }
  if (!units.empty()) {
    std::vector<size_t> ran;
    for (size_t si = 0; si < nStreams; ++si) {
      if (waited[si]) ran.push_back(si);
    }
    remember(spans, ran);
  }
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

// The reduction with a compression hook folded in, with the raw fp32
// contribution still in the gradient tensors it is assembled from (what
// torch's bf16 / fp16 compression hooks see with gradient_as_bucket_view=False
// is a bucket that the reducer has just copied those tensors into). The bucket
// is cut into launches as an assembled one would be (a bucket of 25 MiB: one),
// and a launch reads its raw term from the tensors that lie in its range: up
// to eight, by a table in the kernel arguments, provided every tensor starts
// where a lane's group of 8 elements does and on the others' 16-byte phase
// (layer sizes that are multiples of 8 and the allocator's alignment give
// that); a launch whose tensors do not fit goes tensor by tensor, each a
// launch with that tensor as its raw buffer, as the copy kernel it replaces
// was.
std::vector<hipStream_t> Context::runGatheredCompressed(
    const Request& req, const std::vector<hipEvent_t>& initialEvents) {
  const int64_t wireSize = elementSize(req.dtype);
  const int64_t outSize = elementSize(req.outDtype);
  const int total = static_cast<int>(req.contribs.size());
  const int g = req.gatheredIndex;
  nextStagingSlot_ += numSlices(req.numel, layout_.sliceSizeInBytes, wireSize);
  struct Part {
    int64_t off;  // in the bucket, elements
    int64_t len;
    std::vector<RawPiece> pieces;  // offsets counted from `off`
  };
  // the tensors that hold anything, and where they start in the bucket
  struct Tensor {
    const float* ptr;
    int64_t off, len;
  };
  std::vector<Tensor> tensors;
  {
    int64_t off = 0;
    for (const Request::Segment& seg : req.gathered) {
      if (seg.numel > 0) tensors.push_back(Tensor{static_cast<const float*>(seg.ptr), off, seg.numel});
      off += seg.numel;
    }
  }
  std::vector<Part> parts;
  const int64_t quantum = kLaunchQuantumBytes / wireSize;
  int64_t partLen = roundDownToNearestMultiple(
      defaultCompressedLaunchBytes(total, /*hasRaw=*/true, req.outDtype == FRG_F32,
                                   req.numel * wireSize) / wireSize, quantum);
  if (partLen < quantum) partLen = quantum;
  std::vector<const void*> probe(static_cast<size_t>(total));
  size_t ti = 0;  // first tensor that reaches into what is left
  for (int64_t lo = 0; lo < req.numel;) {
    int64_t hi = 2 * (req.numel - lo) > 3 * partLen ? lo + partLen : req.numel;
    while (ti < tensors.size() && tensors[ti].off + tensors[ti].len <= lo) ++ti;
    Part part;
    part.off = lo;
    for (size_t t = ti; t < tensors.size() && tensors[t].off < hi; ++t) {
      if (static_cast<int>(part.pieces.size()) == kMaxRawPiecesPerLaunch) {
        hi = tensors[t].off;  // the launch ends where the ninth tensor starts
        break;
      }
      const int64_t from = tensors[t].off > lo ? tensors[t].off : lo;
      part.pieces.push_back(RawPiece{tensors[t].ptr + (from - tensors[t].off), from - lo});
    }
    part.len = hi - lo;
    for (int k = 0; k < total; ++k) {
      probe[static_cast<size_t>(k)] =
          static_cast<const char*>(req.contribs[static_cast<size_t>(k)]) + lo * wireSize;
    }
    const bool fits =
        part.pieces.size() == 1 ||
        rawPiecesVectorize(static_cast<char*>(req.out) + lo * outSize, req.outDtype, probe.data(),
                           total, g, part.pieces.data(), static_cast<int>(part.pieces.size()),
                           part.len);
    if (fits) {
      parts.push_back(std::move(part));
    } else {
      // tensor by tensor
      for (size_t i = 0; i < part.pieces.size(); ++i) {
        const int64_t from = part.pieces[i].off;
        const int64_t to = i + 1 < part.pieces.size() ? part.pieces[i + 1].off : part.len;
        Part one;
        one.off = lo + from;
        one.len = to - from;
        one.pieces.push_back(RawPiece{part.pieces[i].ptr, 0});
        parts.push_back(std::move(one));
      }
    }
    lo = hi;
  }
  const size_t nStreams = reduceStreams_.size();
  std::vector<char> initialsFired(initialEvents.size(), 0);
  auto waitInitials = [&](hipStream_t stream) {
    for (size_t i = 0; i < initialEvents.size(); ++i) {
      bool fired = initialsFired[i] != 0;
      waitInitial(stream, initialEvents[i], &fired);
      initialsFired[i] = fired ? 1 : 0;
    }
  };
  std::vector<char> waited(nStreams, 0);
  const bool oneStream = parts.size() <= static_cast<size_t>(oneStreamLaunches_);
  const size_t opStream = static_cast<size_t>(nextLaunch_) % nStreams;
  size_t lastIdx = opStream;
  if (oneStream && !parts.empty()) ++nextLaunch_;
  const OpSpans spans = spansOf(req);
  if (!parts.empty()) {
    std::vector<size_t> targets;
    if (oneStream) {
      targets.push_back(opStream);
    } else {
      for (size_t si = 0; si < nStreams; ++si) targets.push_back(si);
    }
    orderAfterConflicts(spans, targets);
  }
  std::vector<const void*> ptrs(static_cast<size_t>(total));
  for (const Part& part : parts) {
    const size_t si = oneStream ? opStream : static_cast<size_t>(nextLaunch_++) % nStreams;
    hipStream_t s = reduceStreams_[si];
    if (!waited[si]) {
      waitInitials(s);
      waited[si] = 1;
    }
    lastIdx = si;
    for (int k = 0; k < total; ++k) {
      ptrs[static_cast<size_t>(k)] =
          k == g ? part.pieces[0].ptr
                 : static_cast<const char*>(req.contribs[static_cast<size_t>(k)]) + part.off * wireSize;
    }
    CompressedArgs a;
    if (part.pieces.size() > 1) {
      a.raw_pieces = part.pieces.data();
      a.num_raw_pieces = static_cast<int>(part.pieces.size());
    }
    a.out = static_cast<char*>(req.out) + part.off * outSize;
    a.out_dtype = req.outDtype;
    a.contribs = ptrs.data();
    a.K = total;
    a.raw_index = g;
    a.n = part.len;
    a.wire_dtype = req.dtype;
    a.scale_mode = req.scaleMode;
    a.scale = req.scale;
    launchCompressed(a, s);
  }
  if (!parts.empty()) {
    std::vector<size_t> ran;
    for (size_t si = 0; si < nStreams; ++si) {
      if (waited[si]) ran.push_back(si);
    }
    remember(spans, ran);
  }
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
