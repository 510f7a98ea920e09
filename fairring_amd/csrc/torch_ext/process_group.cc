#include <Python.h>

#include "process_group.h"

#include <algorithm>
#include <chrono>
#include <cstdlib>
#include <thread>

#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <c10/core/StreamGuard.h>

#include <cstdio>
#include <exception>

namespace fairring {

namespace {

// Contract violations end the process, as the reference's MY_CHECK does
// (fairring/utils.h:29-33); the message goes to stderr first.
#define FRG_CHECK(cond)                                                        \
  if (!(cond)) {                                                               \
    std::fprintf(stderr, "[fairring] Condition %s is false (%s:%d)\n", #cond,  \
                 __FILE__, __LINE__);                                          \
    std::terminate();                                                          \
  }

// Flat 1-D view over the same storage, valid for any dense permutation
// (fairring/utils.h:353-361).
at::Tensor viewAsFlat(const at::Tensor& t) {
  FRG_CHECK(t.layout() == at::kStrided);
  FRG_CHECK(t.is_non_overlapping_and_dense());
  // already flat (what DDP hands over): the same view, without a dispatcher call
  if (t.dim() == 1 && (t.numel() <= 1 || t.stride(0) == 1)) return t;
  return at::as_strided(t, {t.numel()}, {1}, t.storage_offset());
}

int dtypeCode(const at::Tensor& t) {
  switch (t.scalar_type()) {
    case at::kFloat:
      return FRG_F32;
    case at::kBFloat16:
      return FRG_BF16;
    case at::kHalf:
      return FRG_F16;
    case at::kDouble:
      return FRG_F64;
    case at::kInt:
      return FRG_I32;
    case at::kLong:
      return FRG_I64;
    case at::kByte:
      return FRG_U8;
    case at::kChar:
      return FRG_I8;
    default:
      return -1;
  }
}

// What travels through the C ABI's completion callback.
struct Pending {
  c10::intrusive_ptr<c10::ivalue::Future> future;
  at::Tensor tensor;               // the result tensor (the caller's, reduced in place)
  std::vector<at::Tensor> inputs;  // keep-alive: own input, peers' contributions
  c10::DeviceIndex device;
};

// Runs on the pipeline's command thread once the last slice is enqueued:
// completes the future under a guard of the last stream, so that consumers
// are ordered after it on the GPU without a host wait
// (fairring/device.cc:337-348).
void onDone(void* user, int status, void* lastStream) {
  std::unique_ptr<Pending> p(static_cast<Pending*>(user));
  c10::Stream s = c10::hip::getStreamFromExternalMasqueradingAsCUDA(
      static_cast<hipStream_t>(lastStream), p->device);
  c10::StreamGuard g(s);
  if (status == FRG_OK) {
    p->future->markCompleted(std::vector<at::Tensor>{std::move(p->tensor)});
  } else {
    p->future->setError(std::make_exception_ptr(
        std::runtime_error("fairring: allreduce failed with status " + std::to_string(status))));
  }
}

// Lets go of Python's global lock for a scope if this thread holds it. The
// command thread's completion callbacks may need that lock (a future's Python
// callbacks; the last reference to a tensor that Python created), so nothing
// here may wait for the command thread while holding it. Python's bindings of
// Work.wait and Future.wait let go of it themselves; those of Work.result and
// Work.synchronize, and the deallocation of a group, do not.
class GilRelease {
 public:
  GilRelease() {
    if (Py_IsInitialized() && PyGILState_Check()) saved_ = PyEval_SaveThread();
  }
  ~GilRelease() {
    if (saved_ != nullptr) PyEval_RestoreThread(saved_);
  }
  GilRelease(const GilRelease&) = delete;
  GilRelease& operator=(const GilRelease&) = delete;

 private:
  PyThreadState* saved_ = nullptr;
};


}  // namespace

// The state of one operation in flight. The result tensor and the status are
// written before `done` is set and not changed after it; the future is made by
// the first getFuture(), and completed by whoever finds both it and `done`:
// the completion callback if the future was there first, else getFuture().
struct ProcessGroupFairring::OpState {
  std::mutex mu;
  std::atomic<bool> done{false};
  int status = FRG_OK;
  hipStream_t lastStream = nullptr;
  c10::intrusive_ptr<c10::ivalue::Future> future;
  at::Tensor tensor;               // the result tensor (the caller's, reduced in place)
  std::vector<at::Tensor> inputs;  // kept alive until the operation is enqueued
  c10::DeviceIndex device = 0;
};

namespace {

using OpState = ProcessGroupFairring::OpState;

std::string failureText(int status) {
  return "fairring: allreduce failed with status " + std::to_string(status);
}

// Completes the future under a guard of the operation's last stream, so that
// consumers are ordered after it on the GPU without a host wait
// (fairring/device.cc:337-348).
void completeFuture(const OpState& st, const c10::intrusive_ptr<c10::ivalue::Future>& future) {
  c10::Stream s = c10::hip::getStreamFromExternalMasqueradingAsCUDA(st.lastStream, st.device);
  c10::StreamGuard g(s);
  if (st.status == FRG_OK) {
    future->markCompleted(std::vector<at::Tensor>{st.tensor});
  } else {
    future->setError(std::make_exception_ptr(std::runtime_error(failureText(st.status))));
  }
}

// Runs once the last slice is enqueued: on the pipeline's command thread, or on
// the caller's (inside frg_allreduce, before the Work exists) for a small
// operation launched on the caller's stream. What the caller handed in is let
// go of here: from now on its memory is protected by stream order (the
// caller's own stream) or by what was recorded on the reduce streams.
void onEnqueued(void* user, int status, void* lastStream) {
  std::unique_ptr<std::shared_ptr<OpState>> holder(static_cast<std::shared_ptr<OpState>*>(user));
  OpState& st = **holder;
  c10::intrusive_ptr<c10::ivalue::Future> future;
  std::vector<at::Tensor> inputs;
  {
    std::lock_guard<std::mutex> g(st.mu);
    st.status = status;
    st.lastStream = static_cast<hipStream_t>(lastStream);
    st.done.store(true, std::memory_order_release);
    future = st.future;
    inputs.swap(st.inputs);
  }
  if (future) completeFuture(st, future);
}

}  // namespace

// ---- WorkFairring ---------------------------------------------------------

ProcessGroupFairring::WorkFairring::WorkFairring(
    c10d::OpType opType, c10::intrusive_ptr<c10::ivalue::Future> future,
    c10::intrusive_ptr<c10d::Backend> group, frg_ctx* ctx)
    : c10d::Work(-1, opType),
      future_(std::move(future)),
      group_(std::move(group)),
      ctx_(ctx) {}

ProcessGroupFairring::WorkFairring::WorkFairring(
    c10d::OpType opType, std::shared_ptr<OpState> state, frg_work* handle,
    c10::intrusive_ptr<c10d::Backend> group, frg_ctx* ctx)
    : c10d::Work(-1, opType),
      state_(std::move(state)),
      handle_(handle),
      group_(std::move(group)),
      ctx_(ctx) {}

ProcessGroupFairring::WorkFairring::~WorkFairring() {
  if (handle_ != nullptr) (void)frg_work_release(handle_);
}

bool ProcessGroupFairring::WorkFairring::isCompleted() {
  return state_ ? state_->done.load(std::memory_order_acquire) : future_->completed();
}

bool ProcessGroupFairring::WorkFairring::isSuccess() const {
  if (!state_) return future_->hasValue();
  return state_->done.load(std::memory_order_acquire) && state_->status == FRG_OK;
}

std::exception_ptr ProcessGroupFairring::WorkFairring::exception() const {
  if (!state_) return future_->exception_ptr();
  if (state_->done.load(std::memory_order_acquire) && state_->status != FRG_OK) {
    return std::make_exception_ptr(std::runtime_error(failureText(state_->status)));
  }
  return nullptr;
}

std::vector<at::Tensor> ProcessGroupFairring::WorkFairring::result() {
  awaitCompletion();
  if (state_) return {state_->tensor};
  return future_->value().toTensorVector();
}

// The caller's current stream waits for the operation; the host only until the
// command thread has enqueued it (what waiting on the reference's future does:
// fairring/process_group.cc:64-68). A limit set with FAIRRING_WAIT_TIMEOUT_S
// applies inside the handle's own wait.
void ProcessGroupFairring::WorkFairring::awaitCompletion() {
  if (!state_) {
    awaitFuture();
    return;
  }
  hipStream_t current =
      c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(state_->device).stream();
  int rc;
  {
    GilRelease unlocked;
    rc = frg_work_block_stream(handle_, current);
  }
  if (rc == FRG_ERR_NOT_READY) {
    TORCH_CHECK(false, "fairring: ", frg_last_error());
  }
  if (rc != FRG_OK) throw std::runtime_error(failureText(rc));
}

// FAIRRING_WAIT_TIMEOUT_S (seconds, unset or 0: no limit, as in the reference):
// a wait that sees no completion for that long raises with a report of where
// the pipeline stands, instead of blocking for good.
void ProcessGroupFairring::WorkFairring::awaitFuture() {
  static const double limit = [] {
    const char* v = std::getenv("FAIRRING_WAIT_TIMEOUT_S");
    const double s = v ? std::atof(v) : 0.0;
    return s > 0.0 ? s : 0.0;
  }();
  if (future_->completed()) {
    future_->wait();  // orders the current stream after the result, no more
    return;
  }
  GilRelease unlocked;
  // A small operation completes within microseconds of the call: poll for a
  // short while before sleeping on the future (a sleeping thread takes tens of
  // microseconds to wake).
  {
    static const long long spinMicros = [] {
      const char* e = std::getenv("FAIRRING_SPIN_US");
      const long long us = e != nullptr ? std::atoll(e) : 200;
      return us < 0 ? 0ll : (us > 100000 ? 100000ll : us);
    }();
    const auto until = std::chrono::steady_clock::now() + std::chrono::microseconds(spinMicros);
    while (!future_->completed() && std::chrono::steady_clock::now() < until) {
#if defined(__x86_64__)
      __builtin_ia32_pause();
#endif
    }
  }
  if (limit > 0.0) {
    const auto deadline = std::chrono::steady_clock::now() +
                          std::chrono::duration_cast<std::chrono::steady_clock::duration>(
                              std::chrono::duration<double>(limit));
    while (!future_->completed()) {
      if (std::chrono::steady_clock::now() > deadline) {
        std::string where = "no context";
        frg_progress p = {};
        if (ctx_ != nullptr && frg_get_progress(ctx_, &p) == FRG_OK) {
          where = std::to_string(p.submitted) + " operations submitted, " +
                  std::to_string(p.started) + " started by the command thread, " +
                  std::to_string(p.enqueued) + " fully enqueued, " + std::to_string(p.launches) +
                  " kernel launches issued";
        }
        TORCH_CHECK(false, "fairring: gave up after ", limit,
                    " s waiting for an operation to complete (", where, ")");
      }
      std::this_thread::sleep_for(std::chrono::microseconds(100));
    }
  }
  future_->wait();
}

void ProcessGroupFairring::WorkFairring::synchronize() { awaitCompletion(); }

// The timeout is ignored, as in the reference (process_group.cc:64-68).
bool ProcessGroupFairring::WorkFairring::wait(std::chrono::milliseconds /*timeout*/) {
  awaitCompletion();
  return true;
}

void ProcessGroupFairring::WorkFairring::abort() {}

c10::intrusive_ptr<c10::ivalue::Future> ProcessGroupFairring::WorkFairring::getFuture() {
  if (!state_) return future_;
  c10::intrusive_ptr<c10::ivalue::Future> future;
  bool completeHere = false;
  {
    std::lock_guard<std::mutex> g(state_->mu);
    if (!state_->future) {
      state_->future = c10::make_intrusive<c10::ivalue::Future>(
          c10::ListType::ofTensors(),
          std::vector<c10::Device>{c10::Device(c10::kCUDA, state_->device)});
      // enqueued already: the callback has been and gone
      completeHere = state_->done.load(std::memory_order_acquire);
    }
    future = state_->future;
  }
  if (completeHere) completeFuture(*state_, future);
  return future;
}

// ---- OptionsFairring -------------------------------------------------------

ProcessGroupFairring::OptionsFairring::OptionsFairring(
    int64_t maxMemory, int64_t maxPadding, int64_t minPar, bool highPriority,
    std::chrono::milliseconds timeout, int64_t sliceSize)
    : c10d::Backend::Options(kPgName, timeout),
      maxMemoryAllocatedInBytes(maxMemory),
      maxPaddingAllocatedInBytes(maxPadding),
      minParallelism(minPar),
      isHighPriorityStream(highPriority),
      sliceSizeInBytes(sliceSize) {}

ProcessGroupFairring::OptionsFairring::~OptionsFairring() = default;

c10::intrusive_ptr<ProcessGroupFairring::OptionsFairring>
ProcessGroupFairring::OptionsFairring::create(int64_t maxMemory, int64_t maxPadding,
                                              int64_t minPar, bool highPriority,
                                              std::chrono::milliseconds timeout,
                                              int64_t sliceSize) {
  return c10::make_intrusive<OptionsFairring>(maxMemory, maxPadding, minPar, highPriority,
                                              timeout, sliceSize);
}

// ---- ProcessGroupFairring --------------------------------------------------

ProcessGroupFairring::ProcessGroupFairring(const c10::intrusive_ptr<c10d::Store>& store,
                                           int rank, int size,
                                           c10::intrusive_ptr<OptionsFairring> options)
    : c10d::Backend(rank, size), store_(store), options_(std::move(options)) {
  TORCH_CHECK(0 <= rank && rank < size, "fairring: rank ", rank, " outside group of ", size);
}

ProcessGroupFairring::~ProcessGroupFairring() {
  // Destroying a context drains its command thread, whose completion callbacks
  // may run Python code (future.then) or drop the last reference to a tensor
  // that Python created: both take the GIL. When this destructor runs from
  // Python's deallocation of the group, the GIL is held here.
  GilRelease unlocked;
  for (auto& kv : contexts_) frg_destroy(kv.second);
}

const std::string ProcessGroupFairring::getBackendName() const { return kPgName; }

frg_ctx* ProcessGroupFairring::contextFor(c10::DeviceIndex device) {
  auto it = contexts_.find(device);
  if (it != contexts_.end()) return it->second;
  frg_options o = {};
  o.max_memory_allocated_in_bytes = options_->maxMemoryAllocatedInBytes;
  o.max_padding_allocated_in_bytes = options_->maxPaddingAllocatedInBytes;
  o.min_parallelism = options_->minParallelism;
  o.slice_size_in_bytes = options_->sliceSizeInBytes;
  o.num_machines = getSize();  // every simulated peer counts as a machine with one device
  o.num_reduce_streams = kNumReduceStreams;
  o.num_copy_streams = kNumCopyStreams;
  frg_ctx* ctx = nullptr;
  const int rc = frg_create(device, &o, &ctx);
  if (rc == FRG_ERR_LAYOUT) {
    // the reference terminates inside computeLayout (fairring/utils.h:297,305)
    std::fprintf(stderr, "[fairring] %s\n", frg_last_error());
    std::terminate();
  }
  TORCH_CHECK(rc == FRG_OK, "fairring: ", frg_last_error());
  // the layout in force, once per device (the reference logs it from
  // computeLayout, fairring/utils.h:314-319)
  frg_layout l = {};
  if (frg_get_layout(ctx, &l) == FRG_OK) {
    std::fprintf(stderr, "[fairring] device %d: %lld staging slots, slice size %lld bytes\n",
                 static_cast<int>(device), static_cast<long long>(l.num_staging_slots),
                 static_cast<long long>(l.slice_size_in_bytes));
  }
  // the reduce streams; the copy streams do not exist until something is staged
  void* raw[16];
  int nStreams = 0;
  TORCH_CHECK(frg_get_streams(ctx, raw, 16, &nStreams) == FRG_OK, frg_last_error());
  std::vector<c10::Stream>& streams = streams_[device];
  for (int i = 0; i < nStreams && i < 16; ++i) {
    streams.push_back(c10::hip::getStreamFromExternalMasqueradingAsCUDA(
        static_cast<hipStream_t>(raw[i]), device));
  }
  contexts_.emplace(device, ctx);
  return ctx;
}

const std::vector<c10::Stream>& ProcessGroupFairring::copyStreamsFor(c10::DeviceIndex device,
                                                                     frg_ctx* ctx) {
  std::vector<c10::Stream>& streams = copyStreams_[device];
  if (streams.empty()) {
    void* raw[8];
    int n = 0;
    TORCH_CHECK(frg_get_copy_streams(ctx, raw, 8, &n) == FRG_OK, frg_last_error());
    for (int i = 0; i < n && i < 8; ++i) {
      streams.push_back(c10::hip::getStreamFromExternalMasqueradingAsCUDA(
          static_cast<hipStream_t>(raw[i]), device));
    }
  }
  return streams;
}

// Tells the caching allocator which streams will touch these buffers
// (fairring/device.cc:297-301): the reduce streams, and the copy streams as
// well when contributions are staged from the host (they write `out`).
void ProcessGroupFairring::recordOnPipelineStreams(
    c10::DeviceIndex device, bool copyStreamsToo, std::initializer_list<const at::Tensor*> tensors,
    const std::vector<at::Tensor>* more) {
  auto record = [&](const std::vector<c10::Stream>& streams) {
    for (const c10::Stream& s : streams) {
      for (const at::Tensor* t : tensors) t->record_stream(s);
      if (more != nullptr) {
        for (const at::Tensor& t : *more) t.record_stream(s);
      }
    }
  };
  record(streams_[device]);
  if (copyStreamsToo) record(copyStreamsFor(device, contexts_.at(device)));
}

void ProcessGroupFairring::setSimulatedPeerContributions(std::vector<at::Tensor> peers) {
  // Checked and flattened here, once, rather than by every operation that uses them.
  bool fromHost = false;
  for (size_t i = 0; i < peers.size(); ++i) {
    at::Tensor& p = peers[i];
    TORCH_CHECK(p.layout() == at::kStrided && p.is_non_overlapping_and_dense(),
                "fairring: peer contribution must be dense");
    if (i == 0) fromHost = !p.is_cuda();
    TORCH_CHECK(fromHost == !p.is_cuda(), "fairring: peers must be all on the GPU or all pinned");
    if (fromHost) {
      TORCH_CHECK(p.is_pinned(), "fairring: host-side peer contributions must be pinned");
    }
    p = viewAsFlat(p);
  }
  std::vector<at::Tensor> old;
  bool drainFirst = false;
  {
    std::lock_guard<std::mutex> g(mutex_);
    // pinned tensors cannot be recorded on a stream: what may still be copied
    // from them is waited for before they go
    drainFirst = peersUsed_ && peersFromHost_ && !peers_.empty();
  }
  if (drainFirst) synchronizeAll();
  {
    std::lock_guard<std::mutex> g(mutex_);
    old.swap(peers_);
    peers_ = std::move(peers);
    peersFromHost_ = fromHost;
    // The group holds its peers' tensors for as long as they are in use, so an
    // operation does not record them on the pipeline's streams; the ones that
    // go now may still be read by launches in flight, and are recorded here.
    // (Operations that have not been enqueued yet hold their peers themselves
    // until they are: the allocator's events then land behind their launches.)
    if (peersUsed_) {
      for (const at::Tensor& t : old) {
        if (!t.is_cuda()) continue;
        auto it = streams_.find(t.device().index());
        if (it == streams_.end()) continue;
        for (const c10::Stream& st : it->second) t.record_stream(st);
        for (const c10::Stream& st : peersUsedFrom_) {
          if (st.device_index() == t.device().index()) t.record_stream(st);
        }
      }
    }
    peersUsed_ = false;
    peersUsedFrom_.clear();
  }
}

void ProcessGroupFairring::setFusedDivide(bool on) {
  std::lock_guard<std::mutex> g(mutex_);
  fusedDivide_ = on;
}

std::vector<int64_t> ProcessGroupFairring::layout() {
  std::lock_guard<std::mutex> g(mutex_);
  TORCH_CHECK(!contexts_.empty(), "fairring: no device initialised yet");
  frg_layout l;
  TORCH_CHECK(frg_get_layout(contexts_.begin()->second, &l) == FRG_OK, frg_last_error());
  return {l.slot_size_in_bytes, l.slice_size_in_bytes, l.num_padding_slots,
          l.num_staging_slots};
}

void ProcessGroupFairring::profileMark() {
  std::lock_guard<std::mutex> g(mutex_);
  TORCH_CHECK(!contexts_.empty(), "fairring: no device initialised yet");
  TORCH_CHECK(frg_profile_mark(contexts_.begin()->second) == FRG_OK, frg_last_error());
}

std::vector<std::tuple<double, double, int64_t, int, int, int>>
ProcessGroupFairring::launchRecords() {
  frg_ctx* ctx = nullptr;
  {
    std::lock_guard<std::mutex> g(mutex_);
    TORCH_CHECK(!contexts_.empty(), "fairring: no device initialised yet");
    ctx = contexts_.begin()->second;
  }
  std::vector<frg_launch_record> recs(1 << 16);
  int n = 0;
  TORCH_CHECK(frg_launch_records(ctx, recs.data(), static_cast<int>(recs.size()), &n) == FRG_OK,
              frg_last_error());
  std::vector<std::tuple<double, double, int64_t, int, int, int>> out;
  for (int i = 0; i < n && i < static_cast<int>(recs.size()); ++i) {
    out.emplace_back(recs[i].begin_ms, recs[i].end_ms, recs[i].numel, recs[i].num_contributions,
                     recs[i].stream_index, recs[i].launches);
  }
  return out;
}

void ProcessGroupFairring::synchronizeAll() {
  std::vector<frg_ctx*> all;
  {
    std::lock_guard<std::mutex> g(mutex_);
    for (auto& kv : contexts_) all.push_back(kv.second);
  }
  for (frg_ctx* ctx : all) TORCH_CHECK(frg_synchronize(ctx) == FRG_OK, frg_last_error());
}

c10::intrusive_ptr<c10d::Work> ProcessGroupFairring::allreduce(
    std::vector<at::Tensor>& data, const c10d::AllreduceOptions& opts) {
  // One tensor per local device (fairring/machine.cc:183); one device here.
  FRG_CHECK(data.size() == 1);
  at::Tensor& t = data[0];
  FRG_CHECK(t.layout() == at::kStrided);
  FRG_CHECK(t.is_cuda());
  FRG_CHECK(t.is_non_overlapping_and_dense());
  t = viewAsFlat(t);
  return reduceCommon(c10d::OpType::ALLREDUCE, opts.reduceOp, t, t, /*chunkOffset=*/0,
                      /*peerNumel=*/t.numel(), {});
}

// fairring/process_group.cc:330-364: input holds `size` chunks, chunk r goes to
// rank r; this rank's output is the reduction of everyone's chunk `rank`.
c10::intrusive_ptr<c10d::Work> ProcessGroupFairring::_reduce_scatter_base(
    at::Tensor& outputBuffer, at::Tensor& inputBuffer, const c10d::ReduceScatterOptions& opts) {
  FRG_CHECK(inputBuffer.layout() == at::kStrided);
  FRG_CHECK(inputBuffer.is_cuda());
  FRG_CHECK(inputBuffer.is_non_overlapping_and_dense());
  FRG_CHECK(outputBuffer.layout() == at::kStrided);
  FRG_CHECK(outputBuffer.is_cuda());
  FRG_CHECK(outputBuffer.is_non_overlapping_and_dense());
  FRG_CHECK(inputBuffer.device() == outputBuffer.device());
  FRG_CHECK(inputBuffer.scalar_type() == outputBuffer.scalar_type());
  FRG_CHECK(inputBuffer.numel() == outputBuffer.numel() * getSize());
  at::Tensor in = viewAsFlat(inputBuffer);
  at::Tensor out = viewAsFlat(outputBuffer);
  return reduceCommon(c10d::OpType::_REDUCE_SCATTER_BASE, opts.reduceOp, in, out,
                      /*chunkOffset=*/out.numel() * getRank(), /*peerNumel=*/in.numel(), {});
}

// fairring/process_group.cc:283-328: the list form; inputTensors[0][r] is the
// chunk this rank contributes to rank r.
c10::intrusive_ptr<c10d::Work> ProcessGroupFairring::reduce_scatter(
    std::vector<at::Tensor>& outputTensors, std::vector<std::vector<at::Tensor>>& inputTensors,
    const c10d::ReduceScatterOptions& opts) {
  FRG_CHECK(inputTensors.size() == outputTensors.size());
  FRG_CHECK(outputTensors.size() == 1);  // one device per process here
  FRG_CHECK(static_cast<int64_t>(inputTensors[0].size()) == getSize());
  at::Tensor& o = outputTensors[0];
  FRG_CHECK(o.layout() == at::kStrided);
  FRG_CHECK(o.is_cuda());
  FRG_CHECK(o.is_non_overlapping_and_dense());
  std::vector<at::Tensor> keep;
  for (const at::Tensor& t : inputTensors[0]) {
    FRG_CHECK(t.layout() == at::kStrided);
    FRG_CHECK(t.is_cuda());
    FRG_CHECK(t.is_non_overlapping_and_dense());
    FRG_CHECK(t.device() == o.device());
    FRG_CHECK(t.scalar_type() == o.scalar_type());
    FRG_CHECK(t.numel() == o.numel());
    keep.push_back(t);
  }
  at::Tensor own = viewAsFlat(inputTensors[0][getRank()]);
  at::Tensor out = viewAsFlat(o);
  return reduceCommon(c10d::OpType::REDUCE_SCATTER, opts.reduceOp, own, out, /*chunkOffset=*/0,
                      /*peerNumel=*/out.numel() * getSize(), std::move(keep));
}

// The shared body: `out` (n elements) = reduction in rank order of this rank's
// own n elements (own[ownOffset ...]) and, from every simulated peer, the n
// elements at offset rank*n of its flat input when the peer hands in a whole
// input (peerNumel == size*n), or its n elements when it hands in just that.
c10::intrusive_ptr<c10d::Work> ProcessGroupFairring::reduceCommon(
    c10d::OpType opType, const c10d::ReduceOp& reduceOp, at::Tensor own, at::Tensor out,
    int64_t chunkOffset, int64_t peerNumel, std::vector<at::Tensor> keepAlive, bool preDivide) {
  // fairring/machine.cc:181: SUM and MAX only
  const c10d::ReduceOp::RedOpType op = reduceOp.op_;
  FRG_CHECK(op == c10d::ReduceOp::SUM || op == c10d::ReduceOp::MAX);
  // fairring/device.cc:316
  FRG_CHECK(8 % out.element_size() == 0);
  const int dtype = dtypeCode(out);
  TORCH_CHECK(dtype >= 0, "fairring: unsupported dtype ", out.scalar_type());

  std::lock_guard<std::mutex> g(mutex_);
  const c10::DeviceIndex device = out.device().index();
  frg_ctx* ctx = contextFor(device);

  const int size = getSize();
  const int rank = getRank();
  const int64_t n = out.numel();
  const int64_t elsize = out.element_size();
  const std::vector<at::Tensor>& peers = peers_;  // checked and flattened when they were set
  TORCH_CHECK(static_cast<int>(peers.size()) == size - 1,
              "fairring: this build runs on one GPU without a transport; a group of size ",
              size, " needs ", size - 1, " simulated peer contributions, got ", peers.size());
  const bool fromHost = !peers.empty() && peersFromHost_;
  if (fromHost) {
    // Switched off by default: one run of this path through the process group
    // (pinned peers, 2 staging slots, completion through the future) stopped
    // making progress on an MI355X and no cause has been found. The same
    // staging through the C ABI (frg_allreduce_host) is unaffected.
    static const bool allowed = std::getenv("FAIRRING_PINNED_PEERS") != nullptr;
    TORCH_CHECK(allowed, "fairring: peer contributions in pinned host memory are switched off "
                         "in the process group (set FAIRRING_PINNED_PEERS=1 to enable them); "
                         "hand them in as GPU tensors, or use frg_allreduce_host");
  }
  const at::ScalarType outType = out.scalar_type();
  const int64_t rankOffset = n * rank;
  for (const at::Tensor& p : peers) {
    const int64_t pn = p.numel();
    TORCH_CHECK(p.scalar_type() == outType && (pn == n || pn == peerNumel),
                "fairring: peer contribution must match the operation's dtype and hold ", n,
                " or ", peerNumel, " elements, got ", pn);
    TORCH_CHECK(fromHost || p.device() == out.device(),
                "fairring: peer contribution on another device");
  }
  peersUsed_ = true;

  // Contribution table in rank order, this rank's own chunk at its index.
  const char* ownPtr = static_cast<const char*>(own.data_ptr()) + chunkOffset * elsize;
  std::vector<const void*> table;
  table.reserve(size);
  for (int r = 0, pi = 0; r < size; ++r) {
    if (r == rank) {
      table.push_back(ownPtr);
      continue;
    }
    // a whole flat input: the chunk meant for this rank; otherwise just that chunk
    const at::Tensor& p = peers[pi++];
    table.push_back(static_cast<const char*>(p.data_ptr()) +
                    (p.numel() == n ? 0 : rankOffset) * elsize);
  }

  // the caller's tensors; the peers' are held by the group (setSimulatedPeerContributions)
  if (own.data_ptr() == out.data_ptr()) {  // in place: one storage
    recordOnPipelineStreams(device, fromHost, {&out}, nullptr);
  } else {
    recordOnPipelineStreams(device, fromHost, {&out, &own}, nullptr);
  }

  const bool divide = fusedDivide_ && op == c10d::ReduceOp::SUM && size > 1;
  const bool pow2 = (size & (size - 1)) == 0;
  int scaleMode = !divide ? FRG_SCALE_NONE : (pow2 ? FRG_SCALE_MUL : FRG_SCALE_DIV);
  float scale = !divide ? 1.0f : (pow2 ? 1.0f / static_cast<float>(size)
                                        : static_cast<float>(size));
  if (preDivide) {
    // tensor.div_(size) on every rank ahead of the sum; ATen on the GPU
    // multiplies by the reciprocal of a scalar divisor
    TORCH_CHECK(op == c10d::ReduceOp::SUM && at::isFloatingType(out.scalar_type()),
                "fairring: a pre-divided allreduce is a SUM of a floating-point tensor");
    TORCH_CHECK(!fromHost, "fairring: a pre-divided allreduce takes GPU-resident peers");
    scaleMode = FRG_SCALE_PRE_MUL;
    scale = 1.0f / static_cast<float>(size);
  }
  const int frgOp = op == c10d::ReduceOp::SUM ? FRG_SUM : FRG_MAX;

  if (fromHost) {
    // Server-side accumulation: this rank's own shard sits in `out`, the
    // peers' are staged from pinned memory and folded into it in rank order.
    // The fixed order needs the resident contribution to be first.
    TORCH_CHECK(rank == 0, "fairring: pinned peer contributions are folded after the resident "
                           "tensor, which must therefore be rank 0 (got rank ", rank, ")");
    if (out.data_ptr() != static_cast<const void*>(ownPtr)) {
      out.copy_(own.narrow(0, chunkOffset, n), /*non_blocking=*/true);  // on the current stream
    }
  }

  const auto currentStream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(device);
  hipStream_t current = currentStream.stream();
  {
    const c10::Stream asStream = currentStream.unwrap();
    bool seen = false;
    for (const c10::Stream& st : peersUsedFrom_) seen = seen || st == asStream;
    if (!seen) peersUsedFrom_.push_back(asStream);
  }
  keepAlive.push_back(own);
  // The peers' tensors as well, until the command thread has enqueued the
  // operation: the group may be handed new peers (and the caller may free the
  // old ones) while this operation still waits in the queue, and what
  // setSimulatedPeerContributions records on the streams at that moment only
  // covers launches that are already enqueued.
  keepAlive.insert(keepAlive.end(), peers.begin(), peers.end());
  auto state = std::make_shared<OpState>();
  state->tensor = out;
  state->inputs = std::move(keepAlive);
  state->device = device;
  auto* holder = new std::shared_ptr<OpState>(state);
  frg_work* handle = nullptr;
  int rc;
  if (fromHost) {
    rc = frg_allreduce_host(ctx, out.data_ptr(), table.data() + 1, size - 1, n, dtype, frgOp,
                            scaleMode, scale, /*carry=*/1, current, &onEnqueued, holder, &handle);
  } else {
    rc = frg_allreduce(ctx, out.data_ptr(), table.data(), size, n, dtype, frgOp, scaleMode,
                       scale, current, &onEnqueued, holder, &handle);
  }
  if (rc != FRG_OK) {
    delete holder;
    TORCH_CHECK(false, "fairring: ", frg_last_error());
  }
  return c10::make_intrusive<WorkFairring>(
      opType, std::move(state), handle,
      c10::intrusive_ptr<c10d::Backend>::unsafe_reclaim_from_nonowning(this), ctx);
}

// ---- a group of one: collectives that only move data ------------------------

void ProcessGroupFairring::requireGroupOfOne(const char* what) const {
  TORCH_CHECK(getSize() == 1, "fairring: ", what, " needs a transport between ranks; this build "
              "runs on one GPU and supports it for a group of size 1 only (got size ", getSize(),
              ")");
}

// A finished Work whose future is marked under the caller's current stream, so
// that whatever was enqueued there (a copy) is what consumers are ordered after.
c10::intrusive_ptr<c10d::Work> ProcessGroupFairring::completedWork(
    c10d::OpType opType, std::vector<at::Tensor> tensors) {
  std::vector<c10::Device> devices;
  for (const at::Tensor& t : tensors) {
    if (t.is_cuda() && (devices.empty() || devices.back() != t.device())) {
      devices.push_back(t.device());
    }
  }
  auto future =
      c10::make_intrusive<c10::ivalue::Future>(c10::ListType::ofTensors(), std::move(devices));
  future->markCompleted(std::move(tensors));
  return c10::make_intrusive<WorkFairring>(opType, std::move(future));
}

c10::intrusive_ptr<c10d::Work> ProcessGroupFairring::broadcast(
    std::vector<at::Tensor>& data, const c10d::BroadcastOptions& /*opts*/) {
  requireGroupOfOne("broadcast");
  return completedWork(c10d::OpType::BROADCAST, data);  // the root already holds its own data
}

c10::intrusive_ptr<c10d::Work> ProcessGroupFairring::allgather(
    std::vector<std::vector<at::Tensor>>& outputTensors, std::vector<at::Tensor>& inputTensors,
    const c10d::AllgatherOptions& /*opts*/) {
  requireGroupOfOne("allgather");
  TORCH_CHECK(outputTensors.size() == inputTensors.size(),
              "fairring: allgather takes one output list per input tensor");
  std::vector<at::Tensor> outs;
  for (size_t i = 0; i < inputTensors.size(); ++i) {
    TORCH_CHECK(outputTensors[i].size() == 1, "fairring: allgather output list must hold ",
                getSize(), " tensor(s)");
    outputTensors[i][0].copy_(inputTensors[i], /*non_blocking=*/true);
    outs.push_back(outputTensors[i][0]);
  }
  return completedWork(c10d::OpType::ALLGATHER, std::move(outs));
}

c10::intrusive_ptr<c10d::Work> ProcessGroupFairring::_allgather_base(
    at::Tensor& outputBuffer, at::Tensor& inputBuffer, const c10d::AllgatherOptions& /*opts*/) {
  requireGroupOfOne("_allgather_base");
  TORCH_CHECK(outputBuffer.numel() == inputBuffer.numel(),
              "fairring: _allgather_base output must hold size * input elements");
  FRG_CHECK(outputBuffer.is_non_overlapping_and_dense());
  FRG_CHECK(inputBuffer.is_non_overlapping_and_dense());
  viewAsFlat(outputBuffer).copy_(viewAsFlat(inputBuffer), /*non_blocking=*/true);
  return completedWork(c10d::OpType::_ALLGATHER_BASE, {outputBuffer});
}

c10::intrusive_ptr<c10d::Work> ProcessGroupFairring::barrier(const c10d::BarrierOptions& /*opts*/) {
  requireGroupOfOne("barrier");
  return completedWork(c10d::OpType::BARRIER, {});
}

c10::intrusive_ptr<c10d::Work> ProcessGroupFairring::allreducePreDivided(at::Tensor bucket) {
  FRG_CHECK(bucket.layout() == at::kStrided);
  FRG_CHECK(bucket.is_cuda());
  FRG_CHECK(bucket.is_non_overlapping_and_dense());
  at::Tensor t = viewAsFlat(bucket);
  return reduceCommon(c10d::OpType::ALLREDUCE, c10d::ReduceOp(c10d::ReduceOp::SUM), t, t,
                      /*chunkOffset=*/0, /*peerNumel=*/t.numel(), {}, /*preDivide=*/true);
}

c10::intrusive_ptr<c10d::Work> ProcessGroupFairring::allreduceFromGrads(
    at::Tensor bucket, std::vector<at::Tensor> grads, bool preDivide) {
  FRG_CHECK(bucket.layout() == at::kStrided);
  FRG_CHECK(bucket.is_cuda());
  FRG_CHECK(bucket.is_non_overlapping_and_dense());
  at::Tensor out = viewAsFlat(bucket);
  const int dtype = dtypeCode(out);
  TORCH_CHECK(dtype >= 0, "fairring: unsupported dtype ", out.scalar_type());
  FRG_CHECK(8 % out.element_size() == 0);
  int64_t total = 0;
  std::vector<frg_segment> segments;
  segments.reserve(grads.size());
  for (at::Tensor& gr : grads) {
    TORCH_CHECK(gr.is_cuda() && gr.device() == out.device() && gr.scalar_type() == out.scalar_type(),
                "fairring: a gradient must be a tensor of the bucket's type on the bucket's device");
    TORCH_CHECK(gr.layout() == at::kStrided && gr.is_non_overlapping_and_dense(),
                "fairring: a gradient must be dense");
    gr = viewAsFlat(gr);
    segments.push_back(frg_segment{gr.data_ptr(), gr.numel()});
    total += gr.numel();
  }
  TORCH_CHECK(total == out.numel(), "fairring: the gradients hold ", total,
              " elements, the bucket ", out.numel());
  TORCH_CHECK(!preDivide || at::isFloatingType(out.scalar_type()),
              "fairring: a pre-divided allreduce takes a floating-point bucket");

  std::lock_guard<std::mutex> g(mutex_);
  const c10::DeviceIndex device = out.device().index();
  frg_ctx* ctx = contextFor(device);
  const int size = getSize();
  const int rank = getRank();
  const int64_t n = out.numel();
  const std::vector<at::Tensor>& peers = peers_;
  TORCH_CHECK(static_cast<int>(peers.size()) == size - 1,
              "fairring: this build runs on one GPU without a transport; a group of size ",
              size, " needs ", size - 1, " simulated peer contributions, got ", peers.size());
  TORCH_CHECK(peers.empty() || !peersFromHost_,
              "fairring: an allreduce from gradients takes GPU-resident peers");
  for (const at::Tensor& p : peers) {
    TORCH_CHECK(p.scalar_type() == out.scalar_type() && p.numel() == n &&
                    p.device() == out.device(),
                "fairring: peer contribution must match the bucket's dtype, size and device");
  }
  peersUsed_ = true;
  std::vector<const void*> table;
  table.reserve(size);
  for (int r = 0, pi = 0; r < size; ++r) {
    table.push_back(r == rank ? nullptr : peers[pi].data_ptr());
    if (r != rank) ++pi;
  }
  recordOnPipelineStreams(device, /*copyStreamsToo=*/false, {&out}, &grads);

  const bool divide = !preDivide && fusedDivide_ && size > 1;
  const bool pow2 = (size & (size - 1)) == 0;
  int scaleMode = !divide ? FRG_SCALE_NONE : (pow2 ? FRG_SCALE_MUL : FRG_SCALE_DIV);
  float scale = !divide ? 1.0f : (pow2 ? 1.0f / static_cast<float>(size)
                                        : static_cast<float>(size));
  if (preDivide) {
    scaleMode = FRG_SCALE_PRE_MUL;
    scale = 1.0f / static_cast<float>(size);
  }
  const auto currentStream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(device);
  {
    const c10::Stream asStream = currentStream.unwrap();
    bool seen = false;
    for (const c10::Stream& st : peersUsedFrom_) seen = seen || st == asStream;
    if (!seen) peersUsedFrom_.push_back(asStream);
  }
  auto state = std::make_shared<OpState>();
  state->tensor = out;
  state->inputs = std::move(grads);
  state->inputs.insert(state->inputs.end(), peers.begin(), peers.end());
  state->device = device;
  auto* holder = new std::shared_ptr<OpState>(state);
  frg_work* handle = nullptr;
  const int rc = frg_allreduce_gathered(ctx, out.data_ptr(), table.data(), size, rank,
                                        segments.data(), static_cast<int>(segments.size()), n,
                                        dtype, FRG_SUM, scaleMode, scale, currentStream.stream(),
                                        &onEnqueued, holder, &handle);
  if (rc != FRG_OK) {
    delete holder;
    TORCH_CHECK(false, "fairring: ", frg_last_error());
  }
  return c10::make_intrusive<WorkFairring>(
      c10d::OpType::ALLREDUCE, std::move(state), handle,
      c10::intrusive_ptr<c10d::Backend>::unsafe_reclaim_from_nonowning(this), ctx);
}

c10::intrusive_ptr<c10d::Work> ProcessGroupFairring::allreduceCompressed(
    at::Tensor bucket, at::ScalarType wire, std::vector<at::Tensor> grads) {
  FRG_CHECK(bucket.layout() == at::kStrided);
  FRG_CHECK(bucket.is_cuda());
  FRG_CHECK(bucket.is_non_overlapping_and_dense());
  TORCH_CHECK(bucket.scalar_type() == at::kFloat,
              "fairring: the compression hooks take a float32 bucket, got ", bucket.scalar_type());
  TORCH_CHECK(wire == at::kBFloat16 || wire == at::kHalf,
              "fairring: the wire type must be bfloat16 or float16, got ", wire);
  at::Tensor t = viewAsFlat(bucket);
  // the bucket's own contribution, where it is still in the gradients it is assembled from
  std::vector<frg_segment> segments;
  segments.reserve(grads.size());
  int64_t held = 0;
  for (at::Tensor& gr : grads) {
    TORCH_CHECK(gr.is_cuda() && gr.device() == t.device() && gr.scalar_type() == at::kFloat,
                "fairring: a gradient must be a float32 tensor on the bucket's device");
    TORCH_CHECK(gr.layout() == at::kStrided && gr.is_non_overlapping_and_dense(),
                "fairring: a gradient must be dense");
    gr = viewAsFlat(gr);
    segments.push_back(frg_segment{gr.data_ptr(), gr.numel()});
    held += gr.numel();
  }
  TORCH_CHECK(grads.empty() || held == t.numel(), "fairring: the gradients hold ", held,
              " elements, the bucket ", t.numel());

  std::lock_guard<std::mutex> g(mutex_);
  const c10::DeviceIndex device = t.device().index();
  frg_ctx* ctx = contextFor(device);
  const int size = getSize();
  const int rank = getRank();
  const int64_t n = t.numel();
  const std::vector<at::Tensor>& peers = peers_;
  TORCH_CHECK(static_cast<int>(peers.size()) == size - 1,
              "fairring: this build runs on one GPU without a transport; a group of size ",
              size, " needs ", size - 1, " simulated peer contributions, got ", peers.size());
  for (const at::Tensor& p : peers) {
    TORCH_CHECK(p.is_cuda() && p.device() == t.device(),
                "fairring: a compressed peer contribution must be a dense tensor on the bucket's "
                "device");
    TORCH_CHECK(p.scalar_type() == wire && p.numel() == n,
                "fairring: a compressed peer contribution must hold ", n, " elements of ", wire);
  }
  peersUsed_ = true;
  std::vector<const void*> table;
  table.reserve(size);
  for (int r = 0, pi = 0; r < size; ++r) {
    table.push_back(r == rank ? t.data_ptr() : peers[pi].data_ptr());
    if (r != rank) ++pi;
  }
  recordOnPipelineStreams(device, /*copyStreamsToo=*/false, {&t}, grads.empty() ? nullptr : &grads);
  auto future = c10::make_intrusive<c10::ivalue::Future>(
      c10::ListType::ofTensors(), std::vector<c10::Device>{t.device()});
  hipStream_t current = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(device).stream();
  // the peers (and the gradients) are held until the operation is enqueued (see reduceCommon)
  std::vector<at::Tensor> keep = peers;
  keep.insert(keep.end(), grads.begin(), grads.end());
  auto* pending = new Pending{future, t, std::move(keep), device};
  // buffer.to(wire).div_(size): on the GPU a multiply by the reciprocal, in
  // the wire type's arithmetic
  const int wireCode = wire == at::kBFloat16 ? FRG_BF16 : FRG_F16;
  const int scaleMode = size > 1 ? FRG_SCALE_MUL : FRG_SCALE_NONE;
  const float scale = 1.0f / static_cast<float>(size);
  const int rc =
      segments.empty()
          ? frg_allreduce_compressed(ctx, t.data_ptr(), FRG_F32, table.data(), size, rank, n,
                                     wireCode, scaleMode, scale, current, &onDone, pending, nullptr)
          : frg_allreduce_compressed_gathered(ctx, t.data_ptr(), FRG_F32, table.data(), size, rank,
                                              segments.data(), static_cast<int>(segments.size()),
                                              n, wireCode, scaleMode, scale, current, &onDone,
                                              pending, nullptr);
  if (rc != FRG_OK) {
    delete pending;
    TORCH_CHECK(false, "fairring: ", frg_last_error());
  }
  return c10::make_intrusive<WorkFairring>(
      c10d::OpType::ALLREDUCE, std::move(future),
      c10::intrusive_ptr<c10d::Backend>::unsafe_reclaim_from_nonowning(this), ctx);
}

}  // namespace fairring
