// The C ABI declared in include/fairring_hip.h: argument checks, error strings
// and nothing else; the work is in pipeline.cc, the schedule_*.cc files and the kernels.
#include <string>
#include <vector>

#include "../../include/fairring_hip.h"
#include <cstring>

#include "ksum_kernels.h"
#include "layout.h"
#include "pipeline.h"

using frg::Context;
using frg::Work;

namespace {

int fail(int code, const std::string& msg) {
  frg::setLastError(msg);
  return code;
}

// No C++ exception may cross the ABI: whatever escapes the C++ side (an
// allocation failure, in practice) becomes a status and a message.
template <typename F>
int guarded(F&& body) {
  try {
    return body();
  } catch (const std::exception& e) {
    return fail(FRG_ERR_HIP, std::string("internal failure: ") + e.what());
  } catch (...) {
    return fail(FRG_ERR_HIP, "internal failure");
  }
}

Context* asCtx(frg_ctx* c) { return reinterpret_cast<Context*>(c); }
Work* asWork(frg_work* w) { return reinterpret_cast<Work*>(w); }

int submitCommon(frg_ctx* ctx, void* out, const void* const* contribs, int K, int64_t numel,
                 int dtype, int op, int scale_mode, float scale, void* producer_stream,
                 frg_done_fn done, void* user, frg_work** work, bool fromHost, bool carry) {
  if (work) *work = nullptr;
  if (ctx == nullptr) return fail(FRG_ERR_INVALID, "null context");
  if (K < 0 || (K > 0 && contribs == nullptr) || (K == 0 && !carry)) {
    return fail(FRG_ERR_INVALID, "at least one contribution is required");
  }
  return guarded([&] {
    Context::Request r;
    r.out = out;
    if (K > 0) r.contribs.assign(contribs, contribs + K);
    r.carry = carry;
    r.numel = numel;
    r.dtype = dtype;
    r.op = op;
    r.scaleMode = scale_mode;
    r.scale = scale;
    r.fromHost = fromHost;
    r.producerStream = static_cast<hipStream_t>(producer_stream);
    r.done = done;
    r.user = user;
    std::string err;
    Work* w = nullptr;
    const int rc = asCtx(ctx)->submit(std::move(r), work ? &w : nullptr, &err);
    if (rc != FRG_OK) return fail(rc, err);
    if (work) *work = reinterpret_cast<frg_work*>(w);
    return static_cast<int>(FRG_OK);
  });
}

}  // namespace

extern "C" {

int frg_compute_layout(int64_t max_memory_allocated_in_bytes,
                       int64_t max_padding_allocated_in_bytes, int64_t min_parallelism,
                       int64_t num_machines, int64_t num_devices_per_machine, frg_layout* out) {
  if (out == nullptr) return fail(FRG_ERR_INVALID, "null layout output");
  if (num_machines < 1 || num_devices_per_machine < 1 || min_parallelism < 1) {
    return fail(FRG_ERR_INVALID, "machines, devices per machine and parallelism must be >= 1");
  }
  frg::Layout l;
  const int rc = frg::computeLayout(max_memory_allocated_in_bytes,
                                    max_padding_allocated_in_bytes, min_parallelism,
                                    num_machines, num_devices_per_machine, &l);
  if (rc == 1) {
    return fail(FRG_ERR_LAYOUT, "min_parallelism exceeds the number of padding slots");
  }
  if (rc == 2) return fail(FRG_ERR_LAYOUT, "padding memory exceeds the total staging memory");
  out->slot_size_in_bytes = l.slotSizeInBytes;
  out->slice_size_in_bytes = l.sliceSizeInBytes;
  out->num_padding_slots = l.numPaddingSlots;
  out->num_staging_slots = l.numStagingSlots;
  return FRG_OK;
}

int64_t frg_num_slices(int64_t numel, int64_t slice_size_in_bytes, int64_t element_size) {
  if (numel < 0 || element_size < 1 || slice_size_in_bytes < element_size) return -1;
  return frg::numSlices(numel, slice_size_in_bytes, element_size);
}

int frg_slice_bounds(int64_t numel, int64_t slice_size_in_bytes, int64_t element_size,
                     int64_t idx, int64_t* offset_in_elems, int64_t* size_in_elems) {
  if (numel < 0 || element_size < 1 || slice_size_in_bytes < element_size ||
      offset_in_elems == nullptr || size_in_elems == nullptr) {
    return fail(FRG_ERR_INVALID, "bad slicing arguments");
  }
  if (idx < 0 || idx >= frg::numSlices(numel, slice_size_in_bytes, element_size)) {
    return fail(FRG_ERR_INVALID, "slice index out of range");
  }
  frg::sliceBounds(numel, slice_size_in_bytes, element_size, idx, offset_in_elems,
                   size_in_elems);
  return FRG_OK;
}

int frg_plan_launches(int K, int64_t numel, int64_t element_size,
                      uint64_t first_contribution_address, uint64_t out_offset_in_allocation,
                      int align_short_operations, int num_cus, int64_t* launch_elems,
                      int32_t* blocks_per_cu, int capacity, int* count) {
  if (K < 1 || numel < 0 || element_size < 1 || frg::kTileBytes % element_size != 0 ||
      num_cus < 1 || count == nullptr) {
    return fail(FRG_ERR_INVALID, "bad arguments to frg_plan_launches");
  }
  return guarded([&] {
    const int64_t bytes = numel * element_size;
    const std::vector<frg::LaunchPart> parts = frg::planDefaultLaunches(
        K, bytes, out_offset_in_allocation, first_contribution_address, num_cus,
        align_short_operations != 0);
    int n = 0;
    for (const frg::LaunchPart& p : parts) {
      if (p.bytes <= 0) continue;
      if (n < capacity && launch_elems != nullptr) launch_elems[n] = p.bytes / element_size;
      if (n < capacity && blocks_per_cu != nullptr) blocks_per_cu[n] = p.blocksPerCu;
      ++n;
    }
    *count = n;
    return static_cast<int>(FRG_OK);
  });
}

int frg_reduce_slice(void* out, const void* const* contribs, int K, int64_t n, int dtype,
                     int op, int scale_mode, float scale, int carry, void* stream) {
  frg::ReduceArgs a;
  a.out = out;
  a.contribs = contribs;
  a.K = K;
  a.n = n;
  a.dtype = dtype;
  a.op = op;
  a.scale_mode = scale_mode;
  a.scale = scale;
  a.carry = carry != 0;
  // the pipeline's rule: tensors that lie close together take the mixed loads
  a.mixed_loads = contribs != nullptr && K >= 1 && K <= frg::kMaxContribsPerLaunch &&
                  frg::closelySpaced(contribs, K);
  std::string err;
  const int rc = frg::launchReduce(a, static_cast<hipStream_t>(stream), &err);
  if (rc != FRG_OK) return fail(rc, err);
  return FRG_OK;
}

int frg_reduce_pieces(const frg_piece* pieces, int num_pieces, int K, int dtype, int op,
                      int scale_mode, float scale, void* stream) {
  if (num_pieces < 0 || (num_pieces > 0 && pieces == nullptr)) {
    return fail(FRG_ERR_INVALID, "bad piece list");
  }
  if (K < 1 || K > frg::kMaxContribsPerLaunch) {
    return fail(FRG_ERR_INVALID, "K must be in [1, 64], got " + std::to_string(K));
  }
  const int64_t elsize = frg::elementSize(dtype);
  if (elsize == 0) return fail(FRG_ERR_UNSUPPORTED, "unsupported dtype " + std::to_string(dtype));
  return guarded([&] {
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool kindOk = frg::segmentedKind(K, dtype, op, false);
    const int cap = frg::maxSegmentsPerLaunch(K);
    std::vector<frg::SegPiece> batch;
    std::string err;
    auto flush = [&]() -> int {
      if (batch.empty()) return FRG_OK;
      frg::SegmentedArgs a;
      a.pieces = batch.data();
      a.numPieces = static_cast<int>(batch.size());
      a.K = K;
      a.dtype = dtype;
      a.scale_mode = scale_mode;
      a.scale = scale;
      const int rc = frg::launchSegmented(a, s, &err);
      batch.clear();
      return rc;
    };
    for (int i = 0; i < num_pieces; ++i) {
      const frg_piece& pc = pieces[i];
      if (pc.numel < 0) return fail(FRG_ERR_INVALID, "negative element count");
      if (pc.numel == 0) continue;
      if (pc.out == nullptr || pc.contribs == nullptr) return fail(FRG_ERR_INVALID, "null piece");
      for (int k = 0; k < K; ++k) {
        if (pc.contribs[k] == nullptr) return fail(FRG_ERR_INVALID, "null contribution");
      }
      if (kindOk && frg::segmentable(pc.out, pc.contribs, K, elsize)) {
        batch.push_back(frg::SegPiece{pc.out, pc.contribs, pc.numel});
        if (static_cast<int>(batch.size()) == cap) {
          const int rc = flush();
          if (rc != FRG_OK) return fail(rc, err);
        }
        continue;
      }
      // not one for the segmented kernel: a launch of its own
      frg::ReduceArgs a;
      a.out = pc.out;
      a.contribs = pc.contribs;
      a.K = K;
      a.n = pc.numel;
      a.dtype = dtype;
      a.op = op;
      a.scale_mode = scale_mode;
      a.scale = scale;
      const int rc = frg::launchReduce(a, s, &err);
      if (rc != FRG_OK) return fail(rc, err);
    }
    const int rc = flush();
    if (rc != FRG_OK) return fail(rc, err);
    return static_cast<int>(FRG_OK);
  });
}

int frg_reduce_slice_compressed(void* out, int out_dtype, const void* const* contribs, int K,
                                int raw_index, int64_t n, int wire_dtype, int scale_mode,
                                float scale, void* stream) {
  frg::CompressedArgs a;
  a.out = out;
  a.out_dtype = out_dtype;
  a.contribs = contribs;
  a.K = K;
  a.raw_index = raw_index;
  a.n = n;
  a.wire_dtype = wire_dtype;
  a.scale_mode = scale_mode;
  a.scale = scale;
  std::string err;
  const int rc = frg::launchCompressedReduce(a, static_cast<hipStream_t>(stream), &err);
  if (rc != FRG_OK) return fail(rc, err);
  return FRG_OK;
}

int frg_create(int device, const frg_options* opts, frg_ctx** out) {
  if (out == nullptr) return fail(FRG_ERR_INVALID, "null context output");
  *out = nullptr;
  frg_options o = {};
  if (opts) o = *opts;
  int count = 0;
  if (hipGetDeviceCount(&count) != hipSuccess || count < 1) {
    (void)hipGetLastError();
    return fail(FRG_ERR_HIP, "no HIP device available");
  }
  if (device < 0 || device >= count) return fail(FRG_ERR_INVALID, "device index out of range");
  return guarded([&] {
    Context* c = nullptr;
    std::string err;
    const int rc = Context::create(device, o, &c, &err);
    if (rc != FRG_OK) return fail(rc, err);
    *out = reinterpret_cast<frg_ctx*>(c);
    return static_cast<int>(FRG_OK);
  });
}

int frg_destroy(frg_ctx* ctx) {
  if (ctx == nullptr) return FRG_OK;
  delete asCtx(ctx);
  return FRG_OK;
}

int frg_get_layout(frg_ctx* ctx, frg_layout* out) {
  if (ctx == nullptr || out == nullptr) return fail(FRG_ERR_INVALID, "null argument");
  const frg::Layout& l = asCtx(ctx)->layout();
  out->slot_size_in_bytes = l.slotSizeInBytes;
  out->slice_size_in_bytes = l.sliceSizeInBytes;
  out->num_padding_slots = l.numPaddingSlots;
  out->num_staging_slots = l.numStagingSlots;
  return FRG_OK;
}

int frg_get_streams(frg_ctx* ctx, void** streams, int capacity, int* count) {
  if (ctx == nullptr || count == nullptr) return fail(FRG_ERR_INVALID, "null argument");
  return guarded([&] {
    const std::vector<hipStream_t> v = asCtx(ctx)->streams();
    *count = static_cast<int>(v.size());
    for (int i = 0; i < *count && i < capacity && streams != nullptr; ++i) streams[i] = v[i];
    return static_cast<int>(FRG_OK);
  });
}

int frg_get_copy_streams(frg_ctx* ctx, void** streams, int capacity, int* count) {
  if (ctx == nullptr || count == nullptr) return fail(FRG_ERR_INVALID, "null argument");
  return guarded([&] {
    const std::vector<hipStream_t> v = asCtx(ctx)->copyStreams();
    *count = static_cast<int>(v.size());
    for (int i = 0; i < *count && i < capacity && streams != nullptr; ++i) streams[i] = v[i];
    return static_cast<int>(FRG_OK);
  });
}

int frg_allreduce(frg_ctx* ctx, void* out, const void* const* contribs, int K, int64_t numel,
                  int dtype, int op, int scale_mode, float scale, void* producer_stream,
                  frg_done_fn done, void* user, frg_work** work) {
  return submitCommon(ctx, out, contribs, K, numel, dtype, op, scale_mode, scale,
                      producer_stream, done, user, work, /*fromHost=*/false, /*carry=*/false);
}

int frg_allreduce_gathered(frg_ctx* ctx, void* out, const void* const* contribs, int K,
                           int gathered_index, const frg_segment* segments, int num_segments,
                           int64_t numel, int dtype, int op, int scale_mode, float scale,
                           void* producer_stream, frg_done_fn done, void* user, frg_work** work) {
  if (work) *work = nullptr;
  if (ctx == nullptr) return fail(FRG_ERR_INVALID, "null context");
  if (K < 1 || contribs == nullptr) {
    return fail(FRG_ERR_INVALID, "at least one contribution is required");
  }
  if (num_segments < 0 || (num_segments > 0 && segments == nullptr)) {
    return fail(FRG_ERR_INVALID, "bad segment list");
  }
  if (gathered_index < 0 || gathered_index >= K) {
    return fail(FRG_ERR_INVALID, "gathered_index out of range");
  }
  return guarded([&] {
    Context::Request r;
    r.out = out;
    r.contribs.assign(contribs, contribs + K);
    r.numel = numel;
    r.dtype = dtype;
    r.op = op;
    r.scaleMode = scale_mode;
    r.scale = scale;
    r.gatheredIndex = gathered_index;
    r.gathered.reserve(static_cast<size_t>(num_segments));
    for (int i = 0; i < num_segments; ++i) {
      r.gathered.push_back(Context::Request::Segment{segments[i].ptr, segments[i].numel});
    }
    r.producerStream = static_cast<hipStream_t>(producer_stream);
    r.done = done;
    r.user = user;
    std::string err;
    Work* w = nullptr;
    const int rc = asCtx(ctx)->submit(std::move(r), work ? &w : nullptr, &err);
    if (rc != FRG_OK) return fail(rc, err);
    if (work) *work = reinterpret_cast<frg_work*>(w);
    return static_cast<int>(FRG_OK);
  });
}

int frg_allreduce_compressed(frg_ctx* ctx, void* out, int out_dtype, const void* const* contribs,
                             int K, int raw_index, int64_t numel, int wire_dtype, int scale_mode,
                             float scale, void* producer_stream, frg_done_fn done, void* user,
                             frg_work** work) {
  if (work) *work = nullptr;
  if (ctx == nullptr) return fail(FRG_ERR_INVALID, "null context");
  if (K < 1 || contribs == nullptr) {
    return fail(FRG_ERR_INVALID, "at least one contribution is required");
  }
  return guarded([&] {
    Context::Request r;
    r.out = out;
    r.contribs.assign(contribs, contribs + K);
    r.numel = numel;
    r.dtype = wire_dtype;
    r.op = FRG_SUM;
    r.scaleMode = scale_mode;
    r.scale = scale;
    r.compressed = true;
    r.outDtype = out_dtype;
    r.rawIndex = raw_index;
    r.producerStream = static_cast<hipStream_t>(producer_stream);
    r.done = done;
    r.user = user;
    std::string err;
    Work* w = nullptr;
    const int rc = asCtx(ctx)->submit(std::move(r), work ? &w : nullptr, &err);
    if (rc != FRG_OK) return fail(rc, err);
    if (work) *work = reinterpret_cast<frg_work*>(w);
    return static_cast<int>(FRG_OK);
  });
}

int frg_allreduce_compressed_gathered(frg_ctx* ctx, void* out, int out_dtype,
                                      const void* const* contribs, int K, int raw_index,
                                      const frg_segment* segments, int num_segments, int64_t numel,
                                      int wire_dtype, int scale_mode, float scale,
                                      void* producer_stream, frg_done_fn done, void* user,
                                      frg_work** work) {
  if (work) *work = nullptr;
  if (ctx == nullptr) return fail(FRG_ERR_INVALID, "null context");
  if (K < 1 || contribs == nullptr) {
    return fail(FRG_ERR_INVALID, "at least one contribution is required");
  }
  if (num_segments < 0 || (num_segments > 0 && segments == nullptr)) {
    return fail(FRG_ERR_INVALID, "bad segment list");
  }
  if (raw_index < 0 || raw_index >= K) {
    return fail(FRG_ERR_INVALID, "raw_index out of range (the piecewise contribution is the raw one)");
  }
  return guarded([&] {
    Context::Request r;
    r.out = out;
    r.contribs.assign(contribs, contribs + K);
    r.numel = numel;
    r.dtype = wire_dtype;
    r.op = FRG_SUM;
    r.scaleMode = scale_mode;
    r.scale = scale;
    r.compressed = true;
    r.outDtype = out_dtype;
    r.rawIndex = raw_index;
    r.gatheredIndex = raw_index;
    r.gathered.reserve(static_cast<size_t>(num_segments));
    for (int i = 0; i < num_segments; ++i) {
      r.gathered.push_back(Context::Request::Segment{segments[i].ptr, segments[i].numel});
    }
    r.producerStream = static_cast<hipStream_t>(producer_stream);
    r.done = done;
    r.user = user;
    std::string err;
    Work* w = nullptr;
    const int rc = asCtx(ctx)->submit(std::move(r), work ? &w : nullptr, &err);
    if (rc != FRG_OK) return fail(rc, err);
    if (work) *work = reinterpret_cast<frg_work*>(w);
    return static_cast<int>(FRG_OK);
  });
}

int frg_allreduce_host(frg_ctx* ctx, void* out, const void* const* host_contribs, int K,
                       int64_t numel, int dtype, int op, int scale_mode, float scale, int carry,
                       void* producer_stream, frg_done_fn done, void* user, frg_work** work) {
  return submitCommon(ctx, out, host_contribs, K, numel, dtype, op, scale_mode, scale,
                      producer_stream, done, user, work, /*fromHost=*/true, carry != 0);
}

int frg_work_wait(frg_work* work) {
  if (work == nullptr) return fail(FRG_ERR_INVALID, "null work");
  return guarded([&] {
    std::string err;
    const int rc = Context::waitWork(asWork(work), &err);
    if (rc != FRG_OK) return fail(rc, err);
    return static_cast<int>(FRG_OK);
  });
}

int frg_set_wait_timeout(double seconds) {
  frg::setWaitTimeout(seconds);
  return FRG_OK;
}

int frg_get_progress(frg_ctx* ctx, frg_progress* out) {
  if (ctx == nullptr || out == nullptr) return fail(FRG_ERR_INVALID, "null argument");
  const frg::Progress& p = asCtx(ctx)->progress();
  out->submitted = p.submitted.load();
  out->started = p.started.load();
  out->enqueued = p.enqueued.load();
  out->launches = p.launches.load();
  return FRG_OK;
}

int frg_get_progress2(frg_ctx* ctx, frg_progress2* out, uint64_t size) {
  if (ctx == nullptr || out == nullptr) return fail(FRG_ERR_INVALID, "null argument");
  if (size < sizeof(frg_progress) || size % sizeof(int64_t) != 0) {
    return fail(FRG_ERR_INVALID, "struct size must be a multiple of 8, at least 32");
  }
  const frg::Progress& p = asCtx(ctx)->progress();
  frg_progress2 all = {};
  all.submitted = p.submitted.load();
  all.started = p.started.load();
  all.enqueued = p.enqueued.load();
  all.launches = p.launches.load();
  all.on_callers_stream = p.onCallersStream.load();
  all.merged = p.merged.load();
  all.segmented_launches = p.segmentedLaunches.load();
  std::memcpy(out, &all, size < sizeof(all) ? static_cast<size_t>(size) : sizeof(all));
  return FRG_OK;
}

int frg_work_is_completed(frg_work* work) {
  if (work == nullptr) return fail(FRG_ERR_INVALID, "null work");
  return Context::workEnqueued(asWork(work)) ? FRG_OK : FRG_ERR_NOT_READY;
}

int frg_work_block_stream(frg_work* work, void* stream) {
  if (work == nullptr) return fail(FRG_ERR_INVALID, "null work");
  return guarded([&] {
    std::string err;
    const int rc = Context::blockStream(asWork(work), static_cast<hipStream_t>(stream), &err);
    if (rc != FRG_OK) return fail(rc, err);
    return static_cast<int>(FRG_OK);
  });
}

int frg_work_release(frg_work* work) {
  if (work == nullptr) return FRG_OK;
  Context::releaseWork(asWork(work));
  return FRG_OK;
}

int frg_synchronize(frg_ctx* ctx) {
  if (ctx == nullptr) return fail(FRG_ERR_INVALID, "null context");
  return guarded([&] {
    std::string err;
    const int rc = asCtx(ctx)->synchronize(&err);
    if (rc != FRG_OK) return fail(rc, err);
    return static_cast<int>(FRG_OK);
  });
}

int frg_profile_mark(frg_ctx* ctx) {
  if (ctx == nullptr) return fail(FRG_ERR_INVALID, "null context");
  return guarded([&] {
    std::string err;
    const int rc = asCtx(ctx)->profileMark(&err);
    if (rc != FRG_OK) return fail(rc, err);
    return static_cast<int>(FRG_OK);
  });
}

int frg_set_profiling(frg_ctx* ctx, int per_launch) {
  if (ctx == nullptr) return fail(FRG_ERR_INVALID, "null context");
  asCtx(ctx)->setProfiling(per_launch != 0);
  return FRG_OK;
}

int frg_kernel_times(frg_ctx* ctx, float* ms, int capacity, int* count) {
  if (ctx == nullptr) return fail(FRG_ERR_INVALID, "null context");
  return guarded([&] {
    std::string err;
    const int rc = asCtx(ctx)->kernelTimes(ms, capacity, count, &err);
    if (rc != FRG_OK) return fail(rc, err);
    return static_cast<int>(FRG_OK);
  });
}

int frg_launch_records(frg_ctx* ctx, frg_launch_record* records, int capacity, int* count) {
  if (ctx == nullptr) return fail(FRG_ERR_INVALID, "null context");
  return guarded([&] {
    std::string err;
    const int rc = asCtx(ctx)->launchRecords(records, capacity, count, &err);
    if (rc != FRG_OK) return fail(rc, err);
    return static_cast<int>(FRG_OK);
  });
}

int frg_set_tuning(int blocks_per_cu) {
  frg::setTuning(blocks_per_cu);
  return FRG_OK;
}

int frg_set_tile_runs(int log2_tiles) {
  if (log2_tiles < 0 || log2_tiles > 12) return fail(FRG_ERR_INVALID, "log2_tiles must be in [0, 12]");
  frg::setXcdChunkShift(log2_tiles);
  return FRG_OK;
}

int frg_set_mixed_loads(int mode) {
  if (mode < -1 || mode > 1) return fail(FRG_ERR_INVALID, "mode must be -1, 0 or 1");
  frg::setMixedLoads(mode);
  return FRG_OK;
}

const char* frg_last_error(void) { return frg::lastError(); }

const char* frg_version(void) { return "0.3"; }

}  // extern "C"
