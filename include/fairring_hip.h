/*
 * fairring_hip.h - C ABI of the MI355X (gfx950) K-way gradient-slice reduction.
 *
 * This is the boundary a host program binds to (the c10d backend in
 * fairring_amd/csrc/torch_ext, Python ctypes, a C benchmark). Plain pointers,
 * sizes and opaque handles only; every function returns an int status
 * (FRG_OK == 0) and leaves a message for frg_last_error() on failure; no C++
 * exception or type crosses it. Device pointers are HIP device pointers on the
 * context's device; streams and events are passed as void* (hipStream_t).
 *
 * Each entry point cites the part of the reference (facebookresearch/fairring,
 * paths relative to its root) that it stands in for.
 */
#ifndef FAIRRING_HIP_H_
#define FAIRRING_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FRG_API __attribute__((visibility("default")))

/* ---- status codes ---------------------------------------------------- */
enum {
  FRG_OK = 0,
  FRG_ERR_INVALID = 1,     /* contract violation (the reference's MY_CHECK, utils.h:29-33) */
  FRG_ERR_HIP = 2,         /* a HIP runtime call failed (the reference's CUDA_CHECK, utils.h:35-45) */
  FRG_ERR_LAYOUT = 3,      /* computeLayout precondition failed (utils.h:297,305) */
  FRG_ERR_UNSUPPORTED = 4, /* dtype / op outside the supported set (machine.cc:181) */
  FRG_ERR_NOT_READY = 5    /* non-blocking query: work not finished yet */
};

/* Element types of a slice: the types the reference maps to NCCL types
 * (fairring/utils.h:221-245). Storage type; the fold runs in fp32 for fp32,
 * bf16 and fp16 (one rounding on the store), in fp64 for fp64, and with
 * two's-complement wrap-around in the element's own width for integers. */
enum {
  FRG_F32 = 0,
  FRG_BF16 = 1,
  FRG_F16 = 2,
  FRG_F64 = 3,
  FRG_I32 = 4,
  FRG_I64 = 5,
  FRG_U8 = 6,
  FRG_I8 = 7
};

/* reduction ops accepted by MachineFairring::allReduce (machine.cc:181) */
enum { FRG_SUM = 0, FRG_MAX = 1 };

/* Fused scale, floating-point types only. The post-scales are applied once to
 * the accumulated value before the store. The pre-scales are applied to every
 * contribution before it is folded in, each product rounded to the storage
 * type, which is bit for bit what DDP leaves in every rank's bucket ahead of
 * the allreduce (tensor.div_(world) in torch's allreduce_hook,
 * torch:distributed/algorithms/ddp_comm_hooks/default_hooks.py:18-32; the
 * reducer's own mul_out by 1/world when no hook is registered). ATen divides
 * by a scalar as written on the CPU and multiplies by its reciprocal on the
 * GPU: DIV and MUL exist for both. A carried-in term is never pre-scaled. */
enum {
  FRG_SCALE_NONE = 0,    /* out = acc                                     */
  FRG_SCALE_MUL = 1,     /* out = acc * scale  (scale = 1/K; exact for K = 2^p) */
  FRG_SCALE_DIV = 2,     /* out = acc / scale  (scale = K; IEEE division, at::div) */
  FRG_SCALE_PRE_MUL = 3, /* term k = x[k] * scale, then the fold */
  FRG_SCALE_PRE_DIV = 4  /* term k = x[k] / scale, then the fold */
};

/* ---- layout and slicing (pure integer functions, no GPU) ---------------- */

/* Layout: fairring/utils.h:281-286 */
typedef struct frg_layout {
  int64_t slot_size_in_bytes;
  int64_t slice_size_in_bytes;
  int64_t num_padding_slots;
  int64_t num_staging_slots;
} frg_layout;

/* computeLayout: fairring/utils.h:288-327. FRG_ERR_LAYOUT where the reference
 * terminates. */
FRG_API int frg_compute_layout(int64_t max_memory_allocated_in_bytes,
                               int64_t max_padding_allocated_in_bytes,
                               int64_t min_parallelism, int64_t num_machines,
                               int64_t num_devices_per_machine, frg_layout* out);

/* numSlices = ceilOfRatio(numel, sliceBytes / elsize): fairring/device.cc:315-319 */
FRG_API int64_t frg_num_slices(int64_t numel, int64_t slice_size_in_bytes,
                               int64_t element_size);

/* slice idx -> (offset, length) in elements: fairring/device.cc:321-326 */
FRG_API int frg_slice_bounds(int64_t numel, int64_t slice_size_in_bytes,
                             int64_t element_size, int64_t idx,
                             int64_t* offset_in_elems, int64_t* size_in_elems);

/* Not in the reference, which hands every slice to one library call: the
 * launches into which frg_allreduce cuts an operation over `numel` elements of
 * `element_size` bytes and K device-resident contributions when no launch size
 * was asked for (frg_options.max_launch_bytes == 0), in order: elements per
 * launch and blocks of the persistent grid per CU (0: the kernel's own rule).
 * From 4 contributions on, an operation of 64 MiB or more per contribution is
 * cut into whole rounds of a grid of 4 blocks per CU (a round: num_cus x 4
 * blocks x 4 KiB of every contribution, 4 MiB on MI355X), and the rounds start
 * where the output reaches a multiple of a round counted from the start of its
 * allocation (`out_offset_in_allocation`: the output's address minus what
 * hipMemGetAddressRange reports as the base; where the rounds lie in physical
 * memory sets the rate) on the 4 KiB grid of the first contribution
 * (`first_contribution_address`). The first launch also takes the bytes ahead
 * of that point and the last one those behind the last whole round. A shorter
 * operation is cut the same way when `align_short_operations` is set and at
 * most a quarter of a round lies ahead of that point (the pipeline sets it once
 * four short operations in a row met that condition, so that a stream of
 * buckets keeps one shape); otherwise, up to 8 contributions, into equal
 * launches of 12.5 MiB on the kernel's own grid. `num_cus`: compute units of
 * the device (256 on MI355X). `*count` receives the number of launches, also
 * when it exceeds `capacity`. */
FRG_API int frg_plan_launches(int K, int64_t numel, int64_t element_size,
                              uint64_t first_contribution_address,
                              uint64_t out_offset_in_allocation,
                              int align_short_operations, int num_cus,
                              int64_t* launch_elems, int32_t* blocks_per_cu, int capacity,
                              int* count);

/* ---- one reduction launch (no pipeline) -------------------------------- */

/* doReduction: fairring/device.cc:108-131 (at::sum_out / at::amax_out over
 * dim 0 of operand[K, n]) and the arithmetic of doReduceScatter
 * (device.cc:33-70), as one kernel launch on `stream`.
 *
 *   out[i] = scale( (carry ? out[i] : nothing) (+) in[0][i] (+) ... (+) in[K-1][i] )
 *
 * folded left to right in fp32 in exactly that order. `out` may be the same
 * pointer as one of the contributions (in-place, as the reference reduces into
 * the caller's own shard); partial overlaps are rejected. 1 <= K <= 64 per
 * launch; chain launches with carry = 1 for more. Such a chain carries its
 * partial result in `out`, in the storage type: exact for fp32, fp64, the
 * integer types and MAX, but a bf16 / fp16 SUM then rounds once per launch.
 * frg_allreduce chains those through fp32 accumulators instead and rounds once
 * for any K. n == 0 is a no-op (device.cc:120-122). Asynchronous: returns
 * after enqueueing. The call allocates nothing, records no event and clears
 * no memory, so it may be issued on a stream that is being captured into a
 * HIP graph (the pointer table is copied into the launch, the graph replays
 * on the captured addresses); the same holds for frg_reduce_slice_compressed.
 * The pipeline entry points (frg_allreduce*) hand work to another thread and
 * are not for capture: with a producer stream that is being captured they
 * return FRG_ERR_UNSUPPORTED. */
FRG_API int frg_reduce_slice(void* out, const void* const* contribs, int K,
                             int64_t n, int dtype, int op, int scale_mode,
                             float scale, int carry, void* stream);

/* Not in the reference, which reduces one contiguous shard per library call:
 * several reductions of the same kind (K, element type, operator, scale) as one
 * call on `stream`. Each piece is an elementwise reduction of its own, with an
 * output, K contributions and a length, anywhere in device memory; an output
 * may be one of its piece's contributions, pieces must not overlap each other.
 * Sums of fp32, bf16 or fp16 with up to 16 contributions whose pointers agree
 * modulo 16 bytes within a piece are packed up to 24 at a time (12 beyond 8
 * contributions) into launches of one kernel that deals the 4 KiB tiles of all
 * of them to one grid: many small tensors cost one launch, not one each.
 * Whatever does not fit that (MAX, other types, more contributions, a piece
 * with misaligned pointers) is launched on its own, as frg_reduce_slice would.
 * Results are those of frg_reduce_slice piece by piece, bit for bit. Allocates
 * nothing and records no event: fit for a stream under graph capture. */
typedef struct frg_piece {
  void* out;
  const void* const* contribs; /* K device pointers */
  int64_t numel;
} frg_piece;
FRG_API int frg_reduce_pieces(const frg_piece* pieces, int num_pieces, int K, int dtype, int op,
                              int scale_mode, float scale, void* stream);

/* No counterpart in the reference. frg_reduce_slice for any number of
 * contributions, for callers that cannot allocate: a stream that is being
 * captured into a HIP graph, a tight serving loop, a harness that forbids
 * hipMalloc. More than 64 contributions are folded by a chain of launches on
 * `stream` with the result of one fold over all of them, as frg_allreduce gives
 * (one rounding for bf16 / fp16, whose partial sums travel as fp32; exact also
 * when `out` is one of the later contributions). Where frg_allreduce parks the
 * partial result of such a chain in a scratch buffer that its context
 * allocates, this call parks it in an array that is part of the library's
 * device code (FRG_STATIC_SCRATCH_BYTES per GPU, there for the life of the
 * process), so the call allocates nothing, creates no event and no stream, and
 * clears no memory. A chain that needs the array (a bf16 / fp16 SUM, or `out`
 * among contributions 64 and up) is limited to what it holds:
 * FRG_STATIC_SCRATCH_BYTES / 4 elements for the fp32 accumulators of a 2-byte
 * type, FRG_STATIC_SCRATCH_BYTES / element size otherwise; beyond that, and
 * beyond FRG_STATIC_MAX_CONTRIBUTIONS, the call fails with FRG_ERR_INVALID and
 * says so. Everything else (up to 64 contributions; chains of fp32, fp64,
 * integers or MAX, which carry their exact partial result in `out`) takes any
 * size. All calls on one GPU share that GPU's array: two of them that overlap
 * in time (different streams, or two graphs replayed at once) race on it; calls
 * on one stream do not. The array's address is looked up on the first call on a
 * device (frg_create does it for its device beforehand). */
#define FRG_STATIC_SCRATCH_BYTES (8 * 1024 * 1024)
#define FRG_STATIC_MAX_CONTRIBUTIONS 4096
FRG_API int frg_reduce_slice_static(void* out, const void* const* contribs, int K,
                                    int64_t n, int dtype, int op, int scale_mode,
                                    float scale, void* stream);

/* The same reduction with torch's gradient-compression hooks folded in
 * (bf16_compress_hook / fp16_compress_hook,
 * torch:distributed/algorithms/ddp_comm_hooks/default_hooks.py:57-134, wrapped
 * around the allreduce of fairring/process_group.cc:131-155). `wire_dtype` is
 * FRG_BF16 or FRG_F16. contribs[raw_index] (raw_index -1: none) is this rank's
 * own fp32 bucket: it is cast to the wire type and scaled there
 * (FRG_SCALE_MUL: * scale, FRG_SCALE_DIV: / scale, each rounded to the wire
 * type; FRG_SCALE_NONE: the cast alone), in registers. Every other contribution
 * is a peer's tensor already in the wire type. The fold runs in fp32 in
 * contribution order with one rounding to the wire type. `out_dtype` is the
 * wire type, or FRG_F32 to store the result widened (the hook's decompress
 * step); `out` may be the raw contribution itself (the bucket, in place).
 * K <= 64. Per element 4 + 2 (K - 1) + 4 bytes cross HBM instead of the
 * 14 + 2 K of the three separate passes. */
FRG_API int frg_reduce_slice_compressed(void* out, int out_dtype, const void* const* contribs,
                                        int K, int raw_index, int64_t n, int wire_dtype,
                                        int scale_mode, float scale, void* stream);

/* ---- the per-GPU slice pipeline ----------------------------------------- */

typedef struct frg_ctx frg_ctx;   /* DeviceFairring: fairring/device.h:22-117 */
typedef struct frg_work frg_work; /* the ivalue::Future behind WorkFairring: process_group.cc:35-75 */

/* Options: OptionsFairring (fairring/process_group.h:52-77) plus the README's
 * FAIRRING_SLICE_SIZE (README.md:62). Zero-initialise, then set fields. */
typedef struct frg_options {
  int64_t max_memory_allocated_in_bytes;  /* FAIRRING_TOTAL_MEMORY, default 50 MiB (__init__.py:18-26) */
  int64_t max_padding_allocated_in_bytes; /* FAIRRING_PADDING_MEMORY, default 1 MiB (__init__.py:27-30) */
  int64_t min_parallelism;                /* FAIRRING_PARALLELISM, default 16 (__init__.py:31-34) */
  int64_t slice_size_in_bytes;            /* FAIRRING_SLICE_SIZE; 0 = derive with computeLayout */
  int64_t num_machines;                   /* M used by computeLayout (simulated peers), >= 1 */
  int32_t num_reduce_streams;             /* 0 = default (2) */
  int32_t num_copy_streams;               /* host-staged path; 0 = default (2), at most 4;
                                             created on first use */
  int64_t max_launch_bytes;               /* bytes of one contribution that a single reduction
                                             launch covers: device-resident tensors are cut into
                                             launches of this size on 4 KiB boundaries (the last
                                             one up to 1.5 times as long). 0 = default: the
                                             library's own partition (frg_plan_launches: from 4
                                             contributions on, whole rounds of a 4-blocks-per-CU
                                             grid placed on the 4 MiB multiples of the output's
                                             allocation, about 80 MB per launch), < 0 = one launch
                                             per slice */
} frg_options;

/* DeviceFairring ctor: fairring/device.cc:213-284 (streams, staging pool,
 * per-slot events, command thread). No padding pool: ragged tails are handled
 * inside the kernel. The streams come from a pool that lives as long as the
 * process: a context created after another one was destroyed runs on that
 * one's streams. Every device allocation a context ever makes (staging pool,
 * chain scratch) is made here. */
FRG_API int frg_create(int device, const frg_options* opts, frg_ctx** out);

/* DeviceFairring dtor: fairring/device.cc:286-289 (drain the command queue,
 * join the thread). Streams are never destroyed, as machine.cc:162-175
 * requires for streams that consumers may still hold events on: they go back
 * to the process's pool. */
FRG_API int frg_destroy(frg_ctx* ctx);

/* The layout in force (slice size, number of staging slots). */
FRG_API int frg_get_layout(frg_ctx* ctx, frg_layout* out);

/* The streams the pipeline launches on (reduce streams first, then the copy
 * streams that exist so far), for callers that must tell an allocator which
 * streams touch a buffer (the reference calls record_stream on its five
 * streams, device.cc:297-301). */
FRG_API int frg_get_streams(frg_ctx* ctx, void** streams, int capacity, int* count);

/* The copy streams of the host-staged path (the role of the reference's
 * collectStream_, device.cc:239-243,547-566: where contributions arrive in the
 * staging slots). They are created by the first call of this function or by the
 * first frg_allreduce_host, whichever comes first, so that a context that only
 * reduces device-resident tensors holds its reduce streams and nothing else. A
 * caller that records buffers on the pipeline's streams calls this before it
 * submits a host-staged operation (they write `out`). */
FRG_API int frg_get_copy_streams(frg_ctx* ctx, void** streams, int capacity, int* count);

/* Called once the last slice of an operation has been enqueued (status FRG_OK)
 * or enqueueing failed; `last_stream` is the stream on which completion is
 * ordered (device.cc:337-340 marks the future under a guard of that stream).
 * It runs on the command thread, or, for a small operation that frg_allreduce
 * launches itself (see there), on the calling thread before that call returns:
 * it must not take a lock the caller holds across the call. */
typedef void (*frg_done_fn)(void* user, int status, void* last_stream);

/* DeviceFairring::allReduce: fairring/device.cc:291-353, with the
 * contributions that peers would have delivered passed in explicitly.
 * Device-resident contributions: `contribs[k]` are device pointers to `numel`
 * elements each. The slices of the layout only count here (they advance the
 * slot cursor): resident contributions need no slot, so the tensor is reduced
 * by launches cut as frg_options.max_launch_bytes says (by default the
 * partition of frg_plan_launches), whatever the slice size (max_launch_bytes
 * < 0: one launch per slice). An operation of up to 8 launches (a DDP bucket) runs
 * on one reduce stream and the next operation on the next one; a longer one
 * deals its launches over all reduce streams. Operations are ordered as on one
 * stream wherever that can be observed: one that writes memory an earlier
 * operation of this context reads or writes, or reads what that one writes,
 * runs after it (the streams involved are joined with an event); operations on
 * disjoint buffers, such as the buckets of a gradient, overlap. Waiting for an
 * operation therefore covers every earlier one it shares memory with, not the
 * others. More than 64 contributions are folded by a chain of
 * launches per range; the result is that of one fold over all of them, with
 * one rounding (bf16 / fp16 partial sums travel as fp32), also when `out` is
 * one of the contributions. `producer_stream` is the stream the caller's
 * producer work was enqueued on (the reference records its initial event on
 * the current stream, device.cc:294-295). Returns immediately; `*work`
 * (optional) receives a handle to wait on.
 * A small operation (one launch that moves at most 16 MiB, contributions and
 * output together; FAIRRING_INLINE_BYTES overrides the figure, 0 switches the
 * rule off) that arrives while nothing of this context is queued or running is
 * launched by this call on `producer_stream` itself, behind the producer's
 * work: handing it to a reduce stream and the result back costs two
 * cross-stream waits of 6 to 13 us of host time each, against 3 us for the
 * launch. Its completion is then ordered on `producer_stream`
 * (frg_work_block_stream on that stream is free); whatever this context is
 * handed afterwards from another stream is ordered after it with an event, and
 * frg_synchronize covers it.
 * Operations that wait in the queue while the command thread is busy and
 * continue one another (the same reduction over buffers that lie directly
 * below or above the previous operation's, output and every contribution
 * alike: the buckets of one gradient, handed over faster than they run) are
 * run as one operation over the joint range, 4 to 16 at a time
 * (FAIRRING_MERGE_OPERATIONS sets the upper limit, 1 switches this off): a
 * bucket's launches have ragged ends, a run of buckets has only two. Every
 * operation keeps its own work handle and callback (called in submission
 * order); all of the run complete together. Operations of which one reads what
 * another writes are never joined. */
FRG_API int frg_allreduce(frg_ctx* ctx, void* out, const void* const* contribs,
                          int K, int64_t numel, int dtype, int op,
                          int scale_mode, float scale, void* producer_stream,
                          frg_done_fn done, void* user, frg_work** work);

/* frg_allreduce with one contribution given piecewise: the caller at
 * fairring/process_group.cc:131-155 is DDP's per-bucket allreduce, and with
 * DDP's default (gradient_as_bucket_view=False) every gradient has been copied
 * into the bucket just before (torch:csrc/distributed/c10d/reducer.cpp,
 * mark_variable_ready_dense -> copy_grad_to_bucket; with no hook registered the
 * copy also multiplies by 1/world). Here contribution `gathered_index` is read
 * from where autograd left it: `segments` lists the gradient tensors in the
 * order they lie in the bucket (their lengths add up to `numel`), `out` is the
 * bucket, contribs[gathered_index] is ignored and the other contributions are
 * whole buckets as in frg_allreduce. The result is that of frg_allreduce on the
 * bucket with the segments copied into it, bit for bit (with a pre-scale, as
 * everywhere, every term is scaled and rounded before the fold, which is what
 * the fused copy-and-divide leaves); the copy itself, 8 bytes per element of
 * HBM traffic, is not made. `out` must not be one of the other contributions.
 * Segments whose position in the bucket is a multiple of 16 bytes away from
 * their own address modulo 16 run through the kernel of frg_reduce_pieces,
 * packed into launches of a plain operation's size; the others, and reductions
 * that kernel does not cover, as launches of their own. */
typedef struct frg_segment {
  const void* ptr;
  int64_t numel;
} frg_segment;
FRG_API int frg_allreduce_gathered(frg_ctx* ctx, void* out, const void* const* contribs, int K,
                                   int gathered_index, const frg_segment* segments,
                                   int num_segments, int64_t numel, int dtype, int op,
                                   int scale_mode, float scale, void* producer_stream,
                                   frg_done_fn done, void* user, frg_work** work);

/* frg_reduce_slice_compressed through the pipeline: sliced by the wire type's
 * element size (the tensor the reference would be handed is the compressed
 * one), launches dealt to the reduce streams like frg_allreduce's. */
FRG_API int frg_allreduce_compressed(frg_ctx* ctx, void* out, int out_dtype,
                                     const void* const* contribs, int K, int raw_index,
                                     int64_t numel, int wire_dtype, int scale_mode, float scale,
                                     void* producer_stream, frg_done_fn done, void* user,
                                     frg_work** work);

/* The same with the raw fp32 contribution still in the tensors the bucket is
 * assembled from (what torch's compression hooks meet with DDP's default
 * gradient_as_bucket_view=False, after the reducer has copied every gradient
 * into the bucket: torch:csrc/distributed/c10d/reducer.cpp, copy_grad_to_bucket):
 * contribution `raw_index` is read from `segments` (fp32, in bucket order,
 * lengths adding up to `numel`; contribs[raw_index] is ignored). The bucket is
 * cut into launches as an assembled one would be, and a launch reads its raw
 * term from up to eight tensors through a table in its arguments, provided
 * every tensor starts where a lane's group of 8 elements does and on the
 * others' 16-byte phase (sizes that are multiples of 8, 16-byte aligned
 * tensors); a launch whose tensors do not fit goes tensor by tensor. */
FRG_API int frg_allreduce_compressed_gathered(frg_ctx* ctx, void* out, int out_dtype,
                                              const void* const* contribs, int K,
                                              int raw_index, const frg_segment* segments,
                                              int num_segments, int64_t numel, int wire_dtype,
                                              int scale_mode, float scale,
                                              void* producer_stream, frg_done_fn done,
                                              void* user, frg_work** work);

/* Server-side accumulation with contributions in pinned host memory
 * (device.cc:543-589: collect into a staging slot, then reduce): the staging
 * slots are taken in rotation, (next++) % numSlots, a batch of contributions
 * is copied with hipMemcpyAsync into the slots of its turn and folded into
 * `out`, in contribution order, by the stream that copied them, so that a
 * slot is not filled again before its last reader has run.
 * `host_contribs[k]` are host pointers (hipHostMalloc'd).
 * carry = 0: the K host contributions are all there is (the first one is
 * copied straight into `out`). carry = 1: `out` already holds the device's own
 * contribution, which comes first in the order (the reference reduces the
 * staged shards into its own shard of the caller's tensor, device.cc:570-575);
 * K may then be 0. */
FRG_API int frg_allreduce_host(frg_ctx* ctx, void* out,
                               const void* const* host_contribs, int K,
                               int64_t numel, int dtype, int op, int scale_mode,
                               float scale, int carry, void* producer_stream,
                               frg_done_fn done, void* user, frg_work** work);

/* WorkFairring::wait / synchronize (process_group.cc:60-68): block the host
 * until the operation has been enqueued and its GPU work has finished. */
FRG_API int frg_work_wait(frg_work* work);

/* Not in the reference, whose wait ignores its timeout (process_group.cc:64-68):
 * a process-wide limit, in seconds, after which frg_work_wait gives up with
 * FRG_ERR_NOT_READY and a message that says where the pipeline stands
 * (operations submitted / started / fully enqueued, launches issued, which
 * stream has not drained). The work stays valid and can be waited on again.
 * 0 = no limit (the default, unless FAIRRING_WAIT_TIMEOUT_S is set). */
FRG_API int frg_set_wait_timeout(double seconds);

/* Where the pipeline stands, for such reports: operations accepted, begun by
 * the command thread and fully enqueued, and kernel launches issued so far.
 * This struct keeps the four fields it had in version 0.1 of the ABI. */
typedef struct frg_progress {
  int64_t submitted;
  int64_t started;
  int64_t enqueued;
  int64_t launches;
} frg_progress;
FRG_API int frg_get_progress(frg_ctx* ctx, frg_progress* out);

/* The same with the counters added since, in a struct that may grow: `size` is
 * sizeof(frg_progress2) as the caller was compiled, and no more than that many
 * bytes are written (fields the library does not know of are left alone, so a
 * caller zero-initialises). on_callers_stream: operations small enough, with
 * nothing in flight, to be launched by the call itself on the producer stream;
 * merged: operations run as one with others that were waiting in the queue;
 * segmented_launches: launches that each covered pieces of several such
 * operations (see frg_allreduce for all three). */
typedef struct frg_progress2 {
  int64_t submitted;
  int64_t started;
  int64_t enqueued;
  int64_t launches;
  int64_t on_callers_stream;
  int64_t merged;
  int64_t segmented_launches;
} frg_progress2;
FRG_API int frg_get_progress2(frg_ctx* ctx, frg_progress2* out, uint64_t size);

/* WorkFairring::isCompleted (process_group.cc:43-45): FRG_OK once the command
 * thread has enqueued the whole operation, FRG_ERR_NOT_READY before. */
FRG_API int frg_work_is_completed(frg_work* work);

/* What waiting on the reference's device-aware future does for a consumer
 * stream: make `stream` wait for the operation without blocking the host
 * longer than the enqueue takes. */
FRG_API int frg_work_block_stream(frg_work* work, void* stream);

FRG_API int frg_work_release(frg_work* work);

/* Block until every operation submitted so far has been enqueued and finished. */
FRG_API int frg_synchronize(frg_ctx* ctx);

/* ---- measurement hooks -------------------------------------------------- */

/* Timing with HIP events on the streams the reduction kernel is launched on.
 *
 * frg_profile_mark: goes through the command queue like an operation and
 * records one timing event on every reduce stream, at that point of the
 * stream. Two consecutive marks bracket a region: for each reduce stream that
 * launched anything in between, frg_launch_records yields one record spanning
 * the two events, with the launches and elements that stream ran in the
 * region. Launches on a stream run back to back, so span / launches is the
 * average launch duration on that stream; the cost is one event record per
 * stream and mark, nothing per launch.
 *
 * frg_set_profiling(ctx, 1): instead, every launch gets the begin and end
 * timestamps of its own dispatch (one record per launch). Exact per launch,
 * but the per-dispatch bookkeeping slows a two-stream pipeline by several
 * percent. 0 switches it off. */
FRG_API int frg_profile_mark(frg_ctx* ctx);
FRG_API int frg_set_profiling(frg_ctx* ctx, int per_launch);

/* Durations in milliseconds of the records collected since the last call
 * (after synchronising); consumes them. */
FRG_API int frg_kernel_times(frg_ctx* ctx, float* ms, int capacity, int* count);

/* The same records with their position in time: begin and end in milliseconds
 * after the first record began, the elements and launches they cover, the
 * number of contributions and the index of the reduce stream. Records on
 * different streams overlap; the union of their intervals is the time during
 * which the kernel was running at all. Consumes the records. */
typedef struct frg_launch_record {
  float begin_ms;
  float end_ms;
  int64_t numel;
  int32_t num_contributions;
  int32_t stream_index;
  int32_t launches;
  int32_t reserved;
} frg_launch_record;
FRG_API int frg_launch_records(frg_ctx* ctx, frg_launch_record* records, int capacity,
                               int* count);

/* Launch-shape knob of the reduction kernel: blocks of the persistent grid per
 * CU (0 keeps the built-in default, which depends on the loads per lane). */
FRG_API int frg_set_tuning(int blocks_per_cu);

/* Launch-shape knob of the reduction kernels: log2 of the number of consecutive
 * 4 KiB tiles that the blocks running on one XCD take in a row within a round
 * of the grid (the hardware deals the blocks of a launch to the 8 XCDs in
 * turn). 6, the default, gives every XCD runs of 256 KiB in sums of 8 or more
 * contributions (fewer contributions keep the plain order) and runs of 128 KiB
 * of wire in the compressed reduction (whose grid is half as large: a run is
 * at most a sixteenth of the grid); 0 gives every block the tile of its own
 * index, so that an XCD reads every eighth tile. Results do not depend on it.
 * For measurements. */
FRG_API int frg_set_tile_runs(int log2_tiles);

/* Launch-shape knob of the reduction kernel: which launches run the form of
 * the main loop that mixes the loads of a lane's two 16-byte vectors of a tile
 * (half of the contributions at the first vector together with the other half
 * at the second, 2 KiB further on, then the rest), so that the loads in flight
 * do not all sit at the same position within 4 KiB. -1, the default: the
 * launches of frg_allreduce* and frg_reduce_slice whose contributions lie
 * close to one another in the address space (median distance between
 * neighbours below 768 MiB: a bucket's tensors, allocated one by one), which
 * run through memory in step (8-way fp32: tensors 64 MiB apart +4.5 %, 512 MiB
 * apart +2 %, 1 GiB apart -3.5 %, the 5.5 GB tensors of a whole gradient
 * -1.4 %, hence the rule). 0: no launch. 1: every launch that has the form
 * (sums of 2, 4 or 8 fp32 / bf16 / fp16 contributions; no scale, the multiply
 * by 1/K, or every term times 1/K). Results do not depend on it. For
 * measurements. */
FRG_API int frg_set_mixed_loads(int mode);

/* Message of the last failure on the calling thread (or of the failed work). */
FRG_API const char* frg_last_error(void);

/* "major.minor" of this ABI. 0.2: frg_plan_launches, frg_get_copy_streams,
 * frg_reduce_slice_static added (and frg_progress grew in place, which 0.3
 * takes back). 0.3: frg_progress has its four fields of 0.1 again and
 * frg_get_progress2 carries the later counters with the caller's struct size;
 * frg_allreduce_gathered, frg_allreduce_compressed_gathered, frg_reduce_pieces,
 * frg_set_tile_runs and frg_set_mixed_loads added. */
FRG_API const char* frg_version(void);

#ifdef __cplusplus
}
#endif
#endif /* FAIRRING_HIP_H_ */
