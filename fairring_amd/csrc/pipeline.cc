#include "pipeline.h"

#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <stdexcept>

#include "ksum_kernels.h"
#include "pipeline_internal.h"

namespace frg {

namespace {

thread_local std::string tlsError;

}  // namespace

void setLastError(const std::string& msg) { tlsError = msg; }
const char* lastError() { return tlsError.c_str(); }

namespace {

// How long a thread polls for something it expects soon before it goes to sleep
// on a condition variable: the buckets of a backward pass arrive some tens to
// hundreds of microseconds apart, and waking a sleeping thread costs the caller
// a system call and the operation 20 to 30 microseconds.
constexpr int64_t kDefaultSpinMicros = 200;

// FAIRRING_SPIN_US overrides it (0: sleep at once), read once.
std::chrono::microseconds spinBeforeSleep() {
  static const std::chrono::microseconds v = [] {
    const char* e = std::getenv("FAIRRING_SPIN_US");
    const long long us = e != nullptr ? std::atoll(e) : kDefaultSpinMicros;
    return std::chrono::microseconds(us < 0 ? 0 : (us > 100000 ? 100000 : us));
  }();
  return v;
}

inline void cpuRelax() {
#if defined(__x86_64__) || defined(__i386__)
  __builtin_ia32_pause();
#else
  std::this_thread::yield();
#endif
}

// Polls `ready` for at most spinBeforeSleep(); true as soon as it holds.
template <typename F>
bool spinFor(F&& ready) {
  if (ready()) return true;
  const auto until = std::chrono::steady_clock::now() + spinBeforeSleep();
  for (;;) {
    for (int i = 0; i < 32; ++i) {
      if (ready()) return true;
      cpuRelax();
    }
    if (std::chrono::steady_clock::now() > until) return false;
  }
}

}  // namespace

void CommandQueue::push(Command c) {
  {
    std::unique_lock<std::mutex> lock(mutex_);
    entries_.push_back(std::move(c));
    pending_.fetch_add(1, std::memory_order_release);
  }
  cv_.notify_one();
}

void CommandQueue::enqueue(std::function<void()> fn) { push(Command{std::move(fn), nullptr}); }

void CommandQueue::enqueue(std::shared_ptr<QueuedOp> op) { push(Command{nullptr, std::move(op)}); }

CommandQueue::Command CommandQueue::dequeue() {
  spinFor([&] { return pending_.load(std::memory_order_acquire) > 0; });
  std::unique_lock<std::mutex> lock(mutex_);
  cv_.wait(lock, [&] { return !entries_.empty(); });
  Command c = std::move(entries_.front());
  entries_.pop_front();
  pending_.fetch_sub(1, std::memory_order_relaxed);
  return c;
}

std::vector<std::shared_ptr<QueuedOp>> CommandQueue::takeRun(
    const QueuedOp& first, const std::function<bool(const QueuedOp&, const QueuedOp&)>& continues,
    int atLeast, int atMost) {
  std::vector<std::shared_ptr<QueuedOp>> run;
  if (pending_.load(std::memory_order_acquire) < atLeast) return run;
  std::unique_lock<std::mutex> lock(mutex_);
  size_t n = 0;
  const QueuedOp* previous = &first;
  while (n < entries_.size() && static_cast<int>(n) < atMost && entries_[n].op &&
         continues(*previous, *entries_[n].op)) {
    previous = entries_[n].op.get();
    ++n;
  }
  if (static_cast<int>(n) < atLeast) return run;
  for (size_t i = 0; i < n; ++i) {
    run.push_back(std::move(entries_.front().op));
    entries_.pop_front();
  }
  pending_.fetch_sub(static_cast<int64_t>(n), std::memory_order_relaxed);
  return run;
}

namespace {

// The streams of every context of the process come from here and go back here
// when the context goes. A stream is never destroyed (a consumer may still hold
// an event that orders its own stream after it, fairring/machine.cc:162-175),
// so without reuse every context created would leave its streams behind, and
// the runtime maps streams onto a small number of hardware queues in the order
// they are created: a process that creates contexts one after the other would
// see its reduce streams land on other queues every time, now and then on the
// one its default stream uses (measured: the same bucket stream on the same
// buffers ran at 6.25 or 5.78 TB/s depending on nothing else). With reuse the
// first context's streams are every later context's streams.
class StreamPool {
 public:
  enum Kind { kReduce = 0, kCopy = 1 };

  // `n` idle streams of the kind on `device`, the longest-lived first; creates
  // what is missing (non-blocking, default priority). Throws HipFailure.
  std::vector<hipStream_t> acquire(int device, Kind kind, int n) {
    std::lock_guard<std::mutex> g(mu_);
    std::vector<Entry>& all = streams_[kind];
    std::vector<hipStream_t> out;
    for (Entry& e : all) {
      if (static_cast<int>(out.size()) == n) break;
      if (e.device == device && !e.busy) {
        e.busy = true;
        out.push_back(e.stream);
      }
    }
    while (static_cast<int>(out.size()) < n) {
      hipStream_t s;
      const hipError_t r = hipStreamCreateWithFlags(&s, hipStreamNonBlocking);
      if (r != hipSuccess) {
        (void)hipGetLastError();
        releaseLocked(kind, out);
        throw HipFailure(std::string("hipStreamCreateWithFlags: ") + hipGetErrorString(r));
      }
      all.push_back(Entry{s, device, true});
      out.push_back(s);
    }
    return out;
  }

  // The caller has drained them.
  void release(Kind kind, const std::vector<hipStream_t>& streams) {
    std::lock_guard<std::mutex> g(mu_);
    releaseLocked(kind, streams);
  }

 private:
  struct Entry {
    hipStream_t stream;
    int device;
    bool busy;
  };
  void releaseLocked(Kind kind, const std::vector<hipStream_t>& streams) {
    for (hipStream_t s : streams) {
      for (Entry& e : streams_[kind]) {
        if (e.stream == s) e.busy = false;
      }
    }
  }
  std::mutex mu_;
  std::vector<Entry> streams_[2];
};

StreamPool& streamPool() {
  static StreamPool* pool = new StreamPool();  // outlives every context and static destructor
  return *pool;
}

// An event for one record and the waits on it. Every record gets an event of
// its own, which is destroyed as soon as the waits on it have been enqueued (a
// wait that is pending keeps what it needs: the runtime releases the event's
// resources when it has fired). That is what the reference does with its
// at::cuda::CUDAEvent objects (fairring/device.cc:453-456), and it means that
// no event is ever recorded a second time, so nothing here depends on how a
// wait that has been enqueued but not yet executed treats a later record of
// its event. (Events used to be pooled and recorded again at once; creating
// and destroying one costs about a microsecond of host time.)
hipEvent_t newEvent() {
  hipEvent_t e;
  FRG_HIP_CHECK(hipEventCreateWithFlags(&e, hipEventDisableTiming));
  return e;
}

void retireEvent(hipEvent_t e) {
  if (e != nullptr) (void)hipEventDestroy(e);
}

}  // namespace

int Context::create(int device, const frg_options& o, Context** out, std::string* err) {
  const int64_t total = o.max_memory_allocated_in_bytes > 0 ? o.max_memory_allocated_in_bytes
                                                             : kDefaultTotalMemory;
  const int64_t padding = o.max_padding_allocated_in_bytes > 0
                              ? o.max_padding_allocated_in_bytes
                              : kDefaultPaddingMemory;
  const int64_t parallelism = o.min_parallelism > 0 ? o.min_parallelism : kDefaultParallelism;
  const int64_t machines = o.num_machines > 0 ? o.num_machines : 1;

  Layout layout;
  if (o.slice_size_in_bytes > 0) {
    // README regime: the pool holds TOTAL / SLICE slots of one slice each.
    if (o.slice_size_in_bytes % kAlignment != 0) {
      *err = "slice size must be a multiple of 8 bytes";
      return FRG_ERR_LAYOUT;
    }
    layout.sliceSizeInBytes = o.slice_size_in_bytes;
    layout.slotSizeInBytes = o.slice_size_in_bytes;
    layout.numStagingSlots = total / o.slice_size_in_bytes;
    layout.numPaddingSlots = layout.numStagingSlots;
    if (layout.numStagingSlots < 1) {
      *err = "FAIRRING_TOTAL_MEMORY holds less than one slice";
      return FRG_ERR_LAYOUT;
    }
  } else {
    const int rc = computeLayout(total, padding, parallelism, machines, 1, &layout);
    if (rc != 0) {
      *err = rc == 1 ? "min_parallelism exceeds the padding slots the padding memory allows"
                     : "padding memory alone exceeds the total staging memory";
      return FRG_ERR_LAYOUT;
    }
    if (layout.slotSizeInBytes < kAlignment) {
      *err = "staging memory too small for the requested parallelism";
      return FRG_ERR_LAYOUT;
    }
  }

  Context* c = new Context();
  c->device_ = device;
  c->layout_ = layout;
  c->numSlots_ = layout.numStagingSlots;
  c->slotBytes_ = layout.slotSizeInBytes;
  // Measured on MI355X (K = 8 fp32): launches of 12.5 MiB per contribution,
  // alternating over two streams, sustain 6.4 TB/s where one 25 MiB launch per
  // slice sustains 6.2: short launches keep the blocks of a grid in step, and
  // the second stream fills the ramp and drain of the first. Shorter launches
  // still (6 to 8 MiB) gain another 2 % in a bare launch loop but lose it again
  // to per-launch costs here.
  c->launchBytesByContribs_ = o.max_launch_bytes == 0;  // the default: see defaultLaunchShape
  c->maxLaunchBytes_ = o.max_launch_bytes == 0 ? kDefaultMaxLaunchBytes
                                               : (o.max_launch_bytes < 0 ? 0 : o.max_launch_bytes);
  c->maxLaunchBytes_ -= c->maxLaunchBytes_ % 16;  // keep every launch 16-byte congruent
  if (const char* v = std::getenv("FAIRRING_MERGE_OPERATIONS")) {
    const long long m = std::atoll(v);
    if (m >= 1 && m <= 1024) c->mergeOperations_ = static_cast<int>(m);
  }
  if (const char* v = std::getenv("FAIRRING_INLINE_BYTES")) {
    const long long b = std::atoll(v);
    if (b >= 0) c->inlineTrafficBytes_ = b;
  }
  if (const char* v = std::getenv("FAIRRING_CHAIN_SCRATCH_BYTES")) {
    const long long b = std::atoll(v);
    if (b >= 4096) c->carryScratchBytes_ = b / 4096 * 4096;
  }
  try {
    DeviceGuard g(device);
    int nStreams = o.num_reduce_streams > 0 ? o.num_reduce_streams : 2;
    if (nStreams > 8) nStreams = 8;
    // Default priority on purpose: all streams of the pipeline share one level.
    c->reduceStreams_ = streamPool().acquire(device, StreamPool::kReduce, nStreams);
    // The copy streams of the host-staged path are created when that path is
    // first used (copyStreams()): until then the context holds its reduce
    // streams only.
    c->numCopyStreams_ = o.num_copy_streams > 0 ? (o.num_copy_streams < 4 ? o.num_copy_streams : 4)
                                                : kDefaultStagingStreams;
    FRG_HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&c->stagingPool_),
                            static_cast<size_t>(c->numSlots_ * c->slotBytes_)));
    // The scratch of the launch chains, here rather than on first use: an
    // allocation that fails in the middle of training would only surface as an
    // asynchronous failure of some operation.
    FRG_HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&c->carryScratch_),
                            c->reduceStreams_.size() *
                                static_cast<size_t>(c->carryScratchBytes_ + 16)));
    prepareStaticScratch(device);  // for frg_reduce_slice_static; failures are left to that call
    c->streamLaunches_.assign(c->reduceStreams_.size(), 0);
    c->streamElems_.assign(c->reduceStreams_.size(), 0);
    c->history_.resize(c->reduceStreams_.size());
    c->orderedAfter_.assign(c->reduceStreams_.size(),
                            std::vector<int64_t>(c->reduceStreams_.size(), 0));
  } catch (const std::exception& e) {
    *err = e.what();
    // partially built: the destructor releases what exists and hands the
    // streams back (there is no command thread to join yet)
    delete c;
    return FRG_ERR_HIP;
  }

  c->thread_ = std::thread([c] {
    (void)hipSetDevice(c->device_);
    while (true) {
      CommandQueue::Command cmd = c->queue_.dequeue();
      if (cmd.op) {
        // Neighbouring operations that are already waiting run as one: what
        // limits a stream of buckets is the ragged ends of each, and a run of
        // them has only two.
        // Only a run of several: launches cut from ranges of ever-changing
        // length (one bucket, then two, then one) run slower than either kind.
        std::vector<std::shared_ptr<QueuedOp>> group{std::move(cmd.op)};
        if (c->mergeOperations_ > 1) {
          int direction = 0;
          int64_t bytes = group[0]->req.numel * elementSize(group[0]->req.dtype);
          std::vector<std::shared_ptr<QueuedOp>> more = c->queue_.takeRun(
              *group[0],
              [&](const QueuedOp& previous, const QueuedOp& next) {
                const int64_t nextBytes = next.req.numel * elementSize(next.req.dtype);
                if (bytes + nextBytes > kMaxMergedBytes ||
                    !c->adjoins(previous, next, bytes, &direction)) {
                  return false;
                }
                bytes += nextBytes;
                return true;
              },
              (c->mergeOperations_ < kMinMergedOperations ? c->mergeOperations_
                                                           : kMinMergedOperations) - 1,
              c->mergeOperations_ - 1);
          for (auto& op : more) group.push_back(std::move(op));
        }
        c->runGroup(group);
      } else if (cmd.fn) {
        cmd.fn();
      } else {
        return;
      }
    }
  });
  *out = c;
  return FRG_OK;
}

Context::~Context() {
  if (thread_.joinable()) {
    queue_.enqueue(std::function<void()>());
    thread_.join();
  }
  // Everything submitted has been enqueued; let it finish before the pool goes.
  int prev = 0;
  (void)hipGetDevice(&prev);
  (void)hipSetDevice(device_);
  for (hipStream_t s : reduceStreams_) (void)hipStreamSynchronize(s);
  for (hipStream_t s : copyStreams_) (void)hipStreamSynchronize(s);
  if (inlinePending_) {
    (void)(inlineRecorded_ ? hipEventSynchronize(inlineEvent_) : hipStreamSynchronize(nullptr));
  }
  if (inlineEvent_ != nullptr) (void)hipEventDestroy(inlineEvent_);
  if (stagingPool_) (void)hipFree(stagingPool_);
  if (carryScratch_) (void)hipFree(carryScratch_);
  for (auto& p : profEvents_) {
    (void)hipEventDestroy(p.begin);
    (void)hipEventDestroy(p.end);
  }
  for (auto& m : marks_) {
    for (hipEvent_t e : m.events) (void)hipEventDestroy(e);
  }
  // The streams are not destroyed: a consumer may still hold an event that
  // orders its own stream after one of them (fairring/machine.cc:162-175). They
  // are idle now and serve the next context of the process.
  streamPool().release(StreamPool::kReduce, reduceStreams_);
  streamPool().release(StreamPool::kCopy, copyStreams_);
  (void)hipSetDevice(prev);
}

std::vector<hipStream_t> Context::copyStreams() {
  std::lock_guard<std::mutex> g(copyMu_);
  if (copyStreams_.empty()) {
    DeviceGuard dg(device_);
    copyStreams_ = streamPool().acquire(device_, StreamPool::kCopy, numCopyStreams_);
  }
  return copyStreams_;
}

std::vector<hipStream_t> Context::streams() {
  std::vector<hipStream_t> v = reduceStreams_;
  std::lock_guard<std::mutex> g(copyMu_);
  v.insert(v.end(), copyStreams_.begin(), copyStreams_.end());
  return v;
}

hipEvent_t Context::takeEvent() { return newEvent(); }

void Context::giveEvent(hipEvent_t e) { retireEvent(e); }

// Retires the event `holder` names, if any, and puts a new one in its place:
// for the places that keep "the last record" around (a staging slot's free
// event, the event behind a launch on a caller's stream).
hipEvent_t Context::freshEvent(hipEvent_t* holder) {
  hipEvent_t e = newEvent();
  retireEvent(*holder);
  *holder = e;
  return e;
}

void Context::releaseWork(Work* w) {
  if (w->refs.fetch_sub(1) == 1) delete w;
}

bool Context::workEnqueued(Work* w) {
  std::lock_guard<std::mutex> g(w->mu);
  return w->enqueued;
}

namespace {

// Seconds after which a wait gives up and reports where the pipeline stands
// instead of blocking for good; 0 = wait without limit, as the reference does
// (fairring/process_group.cc:64-68). Starts from FAIRRING_WAIT_TIMEOUT_S.
std::atomic<double>& waitTimeout() {
  static std::atomic<double> seconds{[] {
    const char* v = std::getenv("FAIRRING_WAIT_TIMEOUT_S");
    const double s = v ? std::atof(v) : 0.0;
    return s > 0.0 ? s : 0.0;
  }()};
  return seconds;
}

double waitTimeoutSeconds() { return waitTimeout().load(); }

std::string progressReport(const Work* w) {
  const Progress& p = *w->progress;
  return "operation #" + std::to_string(w->seq) + "; context: " +
         std::to_string(p.submitted.load()) + " submitted, " + std::to_string(p.started.load()) +
         " started by the command thread, " + std::to_string(p.enqueued.load()) +
         " fully enqueued, " + std::to_string(p.launches.load()) + " kernel launches issued";
}

}  // namespace

void setWaitTimeout(double seconds) { waitTimeout().store(seconds > 0.0 ? seconds : 0.0); }

int Context::waitWork(Work* w, std::string* err) {
  const double limit = waitTimeoutSeconds();
  const auto deadline = std::chrono::steady_clock::now() +
                        std::chrono::duration_cast<std::chrono::steady_clock::duration>(
                            std::chrono::duration<double>(limit));
  // a small operation is enqueued within microseconds: poll before sleeping
  spinFor([&] { return w->enqueuedFlag.load(std::memory_order_acquire); });
  {
    std::unique_lock<std::mutex> lock(w->mu);
    if (limit > 0.0) {
      // against the system clock: that is pthread_cond_timedwait, which
      // ThreadSanitizer models (the steady-clock wait is not intercepted by
      // older versions of it, which then report a double lock)
      const auto wallDeadline =
          std::chrono::system_clock::now() +
          std::chrono::duration_cast<std::chrono::system_clock::duration>(
              std::chrono::duration<double>(limit));
      if (!w->cv.wait_until(lock, wallDeadline, [&] { return w->enqueued; })) {
        *err = "gave up after " + std::to_string(limit) +
               " s waiting for the command thread to enqueue " + progressReport(w);
        return FRG_ERR_NOT_READY;
      }
    } else {
      w->cv.wait(lock, [&] { return w->enqueued; });
    }
    if (w->status != FRG_OK) {
      *err = w->error;
      return w->status;
    }
  }
  try {
    DeviceGuard g(w->device);
    for (size_t i = 0; i < w->doneStreams.size(); ++i) {
      hipStream_t s = w->doneStreams[i];
      if (limit <= 0.0) {
        FRG_HIP_CHECK(hipStreamSynchronize(s));
        continue;
      }
      // poll, so that a stream that never drains ends in a message, not a stall
      int64_t spins = 0;
      for (;;) {
        const hipError_t q = hipStreamQuery(s);
        if (q == hipSuccess) break;
        if (q != hipErrorNotReady) FRG_HIP_CHECK(q);
        (void)hipGetLastError();
        if (std::chrono::steady_clock::now() > deadline) {
          *err = "gave up after " + std::to_string(limit) + " s waiting for stream " +
                 std::to_string(i) + " of " + std::to_string(w->doneStreams.size()) +
                 " to drain after " + progressReport(w);
          return FRG_ERR_NOT_READY;
        }
        if (++spins > 2000) std::this_thread::sleep_for(std::chrono::microseconds(50));
      }
    }
  } catch (const std::exception& e) {
    *err = e.what();
    return FRG_ERR_HIP;
  }
  return FRG_OK;
}

int Context::blockStream(Work* w, hipStream_t stream, std::string* err) {
  const double limit = waitTimeoutSeconds();
  // a small operation is enqueued within microseconds: poll before sleeping
  spinFor([&] { return w->enqueuedFlag.load(std::memory_order_acquire); });
  {
    std::unique_lock<std::mutex> lock(w->mu);
    if (limit > 0.0) {
      // the host's share of this call is the enqueue; it gives up like frg_work_wait
      const auto wallDeadline =
          std::chrono::system_clock::now() +
          std::chrono::duration_cast<std::chrono::system_clock::duration>(
              std::chrono::duration<double>(limit));
      if (!w->cv.wait_until(lock, wallDeadline, [&] { return w->enqueued; })) {
        *err = "gave up after " + std::to_string(limit) +
               " s waiting for the command thread to enqueue " + progressReport(w);
        return FRG_ERR_NOT_READY;
      }
    } else {
      w->cv.wait(lock, [&] { return w->enqueued; });
    }
    if (w->status != FRG_OK) {
      *err = w->error;
      return w->status;
    }
  }
  try {
    DeviceGuard g(w->device);
    Progress& p = *w->progress;
    for (size_t i = 0; i < w->doneStreams.size(); ++i) {
      hipStream_t s = w->doneStreams[i];
      if (s == stream) continue;
      const int idx = i < w->doneIndices.size() ? w->doneIndices[i] : -1;
      // The event goes behind whatever the stream holds now, this operation
      // included. The null stream remembers how far that is.
      const bool remember = stream == nullptr && idx >= 0 && idx < Progress::kMaxStreams;
      std::unique_lock<std::mutex> known(p.nullWaitMu, std::defer_lock);
      int64_t upTo = 0;
      if (remember) {
        known.lock();
        if (w->donePositions[i] <= p.nullStreamWaitsFor[idx]) continue;
        upTo = p.streamPosition[idx].load(std::memory_order_acquire);
      }
      hipEvent_t e = newEvent();
      hipError_t r = hipEventRecord(e, s);
      if (r == hipSuccess) r = hipStreamWaitEvent(stream, e, 0);
      retireEvent(e);
      FRG_HIP_CHECK(r);
      if (remember && upTo > p.nullStreamWaitsFor[idx]) p.nullStreamWaitsFor[idx] = upTo;
    }
  } catch (const std::exception& e) {
    *err = e.what();
    return FRG_ERR_HIP;
  }
  return FRG_OK;
}

// What was launched on a caller's stream is ahead of whatever comes from the
// same stream (it takes the producer's event, or finds that stream drained).
// Coming from another stream, the producer waits for it first.
void Context::orderAfterInline(hipStream_t producer) {
  std::lock_guard<std::mutex> g(inlineMu_);
  if (!inlinePending_ || inlineStream_ == producer) return;
  if (!inlineRecorded_) {
    // the null stream, which is always there to record on: behind whatever it
    // holds by now, the launch included
    FRG_HIP_CHECK(hipEventRecord(freshEvent(&inlineEvent_), nullptr));
    inlineRecorded_ = true;
  }
  if (hipEventQuery(inlineEvent_) == hipSuccess) {
    inlinePending_ = false;
    return;
  }
  (void)hipGetLastError();
  FRG_HIP_CHECK(hipStreamWaitEvent(producer, inlineEvent_, 0));
}

// Launches a small operation on the producer stream itself, if it is one the
// rule covers and the reduce streams have drained, marks the work and calls
// the completion callback (on this, the caller's, thread). Returns false when
// the operation is to go through the pipeline instead.
bool Context::tryInline(const Request& req, Work* work) {
  if (inlineTrafficBytes_ <= 0 || req.fromHost || req.compressed || !launchBytesByContribs_ ||
      !req.gathered.empty()) {
    return false;
  }
  const int total = static_cast<int>(req.contribs.size());
  if (total > kMaxContribsPerLaunch || req.numel <= 0) return false;
  const int64_t elsize = elementSize(req.dtype);
  if ((total + 1) * req.numel * elsize > inlineTrafficBytes_) return false;
  if (profiling_.load(std::memory_order_relaxed)) return false;  // its records are per reduce stream
  if (total == 1 && req.contribs[0] == req.out && req.scaleMode == FRG_SCALE_NONE) return false;
  // Asking a busy stream costs 12 us: after a "busy" nobody asks again for a while.
  const int64_t now = std::chrono::duration_cast<std::chrono::nanoseconds>(
                          std::chrono::steady_clock::now().time_since_epoch())
                          .count();
  if (now < inlineRetryAtNs_.load(std::memory_order_relaxed)) return false;
  // Found idle once, the reduce streams stay idle until the command thread takes
  // up another operation (nothing else gives them work that touches data), and
  // none is waiting or being dealt with now: no need to ask again. (Asking a
  // drained stream whose last packet was a wait marker costs 7 to 12 us each
  // time, not 0.1.)
  const int64_t dealtWith = pipelineOps_.load(std::memory_order_acquire);
  if (idleConfirmedAt_.load(std::memory_order_acquire) != dealtWith) {
    for (hipStream_t s : reduceStreams_) {
      if (hipStreamQuery(s) != hipSuccess) {
        (void)hipGetLastError();
        inlineRetryAtNs_.store(now + kInlineRetryNs, std::memory_order_relaxed);
        return false;
      }
    }
    idleConfirmedAt_.store(dealtWith, std::memory_order_release);
  }
  ReduceArgs a;
  a.out = req.out;
  a.contribs = req.contribs.data();
  a.K = total;
  a.n = req.numel;
  a.dtype = req.dtype;
  a.op = req.op;
  a.scale_mode = req.scaleMode;
  a.scale = req.scale;
  // From here on the operation is this function's; a failure is the work's
  // status, as it would be on the command thread.
  int status = FRG_OK;
  std::string error;
  try {
    std::lock_guard<std::mutex> g(inlineMu_);
    status = launchReduce(a, req.producerStream, &error);
    if (status == FRG_OK) {
      // The event that orders other streams after this launch. A stream of the
      // caller's may be gone by the time it is needed, so it is recorded now;
      // the null stream is always there, and a record on it now would make it
      // look busy to the next operation's idle check for no reason: it is
      // recorded when another stream turns up.
      inlineRecorded_ = req.producerStream != nullptr;
      if (inlineRecorded_) {
        // a new event every time: a stream may still be waiting for the last launch's
        FRG_HIP_CHECK(hipEventRecord(freshEvent(&inlineEvent_), req.producerStream));
      }
      inlineStream_ = req.producerStream;
      inlinePending_ = true;
      inlineExplainsBusy_ = true;
      work->doneStreams.assign(1, req.producerStream);
      work->doneIndices.assign(1, -1);
      work->donePositions.assign(1, -1);
      progress_->launches.fetch_add(1);
      progress_->onCallersStream.fetch_add(1);
    }
  } catch (const std::exception& e) {
    status = FRG_ERR_HIP;
    error = e.what();
  }
  if (status != FRG_OK) {
    std::fprintf(stderr, "[fairring] operation #%lld failed: %s\n",
                 static_cast<long long>(work->seq), error.c_str());
  }
  // every slice takes its turn in the slot rotation (fairring/device.cc:482)
  nextStagingSlot_ += numSlices(req.numel, layout_.sliceSizeInBytes, elsize);
  progress_->started.fetch_add(1);
  progress_->enqueued.fetch_add(1);
  {
    std::lock_guard<std::mutex> lock(work->mu);
    work->status = status;
    work->error = error;
    work->lastStream = req.producerStream;
    work->enqueued = true;
    work->enqueuedFlag.store(true, std::memory_order_release);
  }
  if (req.done) req.done(req.user, status, req.producerStream);
  return true;
}

int Context::submit(Request req, Work** workOut, std::string* err) {
  // Contract checks made on the caller's thread, before anything is queued.
  if (elementSize(req.dtype) == 0) {
    *err = "unsupported dtype";
    return FRG_ERR_UNSUPPORTED;
  }
  if (req.op != FRG_SUM && req.op != FRG_MAX) {  // fairring/machine.cc:181
    *err = "unsupported reduce op (only SUM and MAX)";
    return FRG_ERR_UNSUPPORTED;
  }
  if (req.contribs.empty() && !(req.fromHost && req.carry)) {
    *err = "at least one contribution is required";
    return FRG_ERR_INVALID;
  }
  if (req.numel < 0) {
    *err = "negative element count";
    return FRG_ERR_INVALID;
  }
  if (req.op == FRG_MAX && req.scaleMode != FRG_SCALE_NONE) {
    *err = "MAX takes no scale";
    return FRG_ERR_INVALID;
  }
  if (req.scaleMode < FRG_SCALE_NONE || req.scaleMode > FRG_SCALE_PRE_DIV) {
    *err = "bad scale mode";
    return FRG_ERR_INVALID;
  }
  if (req.scaleMode != FRG_SCALE_NONE && !isFloating(req.dtype)) {
    *err = "integer types take no scale";
    return FRG_ERR_INVALID;
  }
  if (req.fromHost && req.scaleMode >= FRG_SCALE_PRE_MUL) {
    // a server does not rescale what the machines deliver
    *err = "host-staged contributions take no pre-scale";
    return FRG_ERR_UNSUPPORTED;
  }
  if (req.compressed) {
    if (req.dtype != FRG_BF16 && req.dtype != FRG_F16) {
      *err = "the wire type must be bf16 or fp16";
      return FRG_ERR_UNSUPPORTED;
    }
    if (req.outDtype != FRG_F32 && req.outDtype != req.dtype) {
      *err = "the output must be fp32 or of the wire type";
      return FRG_ERR_UNSUPPORTED;
    }
    if (req.scaleMode > FRG_SCALE_DIV) {
      *err = "bad scale mode (NONE, MUL or DIV on the raw contribution)";
      return FRG_ERR_INVALID;
    }
    const int K = static_cast<int>(req.contribs.size());
    if (K > kMaxContribsPerLaunch) {
      *err = "at most 64 contributions with compression folded in";
      return FRG_ERR_INVALID;
    }
    if (req.rawIndex < -1 || req.rawIndex >= K) {
      *err = "raw_index out of range";
      return FRG_ERR_INVALID;
    }
  }
  if (!req.gathered.empty() || req.gatheredIndex >= 0) {
    const int K = static_cast<int>(req.contribs.size());
    if (req.fromHost) {
      *err = "a piecewise contribution goes with device-resident contributions";
      return FRG_ERR_UNSUPPORTED;
    }
    if (req.gatheredIndex < 0 || req.gatheredIndex >= K) {
      *err = "gathered_index out of range";
      return FRG_ERR_INVALID;
    }
    if (req.compressed && req.gatheredIndex != req.rawIndex) {
      // the gradients are what is still uncompressed
      *err = "with compression folded in, the piecewise contribution is the raw fp32 one";
      return FRG_ERR_INVALID;
    }
    int64_t sum = 0;
    for (const Request::Segment& g : req.gathered) {
      if (g.numel < 0 || (g.numel > 0 && g.ptr == nullptr)) {
        *err = "bad segment (negative length or null pointer)";
        return FRG_ERR_INVALID;
      }
      sum += g.numel;
    }
    if (sum != req.numel) {
      *err = "the segments hold " + std::to_string(sum) + " elements, the operation " +
             std::to_string(req.numel);
      return FRG_ERR_INVALID;
    }
    for (int k = 0; k < K; ++k) {
      if (k != req.gatheredIndex && req.contribs[static_cast<size_t>(k)] == req.out &&
          req.numel > 0) {
        *err = "the output of an operation with a piecewise contribution must not be another "
               "of its contributions";
        return FRG_ERR_INVALID;
      }
    }
    // the slot it leaves in the table is never read; give it a value that passes the checks
    req.contribs[static_cast<size_t>(req.gatheredIndex)] = req.out;
    if (req.numel > 0 && req.gathered.empty()) {
      *err = "no segments";
      return FRG_ERR_INVALID;
    }
  }
  if (kAlignment % elementSize(req.dtype) != 0) {  // fairring/device.cc:316
    *err = "element size must divide 8";
    return FRG_ERR_INVALID;
  }
  if (req.numel > 0) {
    if (req.out == nullptr) {
      *err = "null output";
      return FRG_ERR_INVALID;
    }
    for (const void* p : req.contribs) {
      if (p == nullptr) {
        *err = "null contribution";
        return FRG_ERR_INVALID;
      }
    }
  }

  {
    // The pipeline hands the launches to its own thread and streams: under HIP
    // graph capture that cannot be recorded into the caller's graph.
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(req.producerStream, &capture) != hipSuccess) {
      (void)hipGetLastError();
    } else if (capture != hipStreamCaptureStatusNone) {
      *err = "the producer stream is being captured into a HIP graph: the pipeline cannot be "
             "captured, issue frg_reduce_slice on the capturing stream instead";
      return FRG_ERR_UNSUPPORTED;
    }
  }

  Work* work = new Work();
  work->device = device_;
  work->progress = progress_;
  // nothing of the pipeline in flight, as far as the host can tell without asking
  const bool nothingQueued = progress_->enqueued.load() == progress_->submitted.load();
  work->seq = progress_->submitted.fetch_add(1);
  hipEvent_t initial = nullptr;
  try {
    DeviceGuard g(device_);
    orderAfterInline(req.producerStream);
    if (nothingQueued && tryInline(req, work)) {
      if (workOut) {
        work->refs.fetch_add(1);
        *workOut = work;
      }
      releaseWork(work);  // the share the command thread would have held
      return FRG_OK;
    }
    // Orders the pipeline after whatever produced the inputs
    // (fairring/device.cc:294-295). A producer stream that has already drained
    // has nothing to wait for, and no event is recorded on it: a record is a
    // packet on the producer's hardware queue, and two hundred of them per step
    // (one per bucket) are work for the command processor that the reduction's
    // own queues then wait behind.
    // Asking an idle stream costs 0.1 us, asking a busy one over 10 (the
    // runtime flushes its queue to find out) against 1 for the record: after a
    // "busy" the next operations from that stream record without asking.
    bool producerIdle = false;
    {
      if (busyProducer_.load(std::memory_order_relaxed) == req.producerStream &&
          busyProducerSkips_.load(std::memory_order_relaxed) > 0) {
        busyProducerSkips_.fetch_sub(1, std::memory_order_relaxed);
      } else {
        const hipError_t q = hipStreamQuery(req.producerStream);
        if (q == hipSuccess) {
          producerIdle = true;
          std::lock_guard<std::mutex> ig(inlineMu_);
          if (inlineStream_ == req.producerStream) {  // and with it what was launched there
            inlinePending_ = false;
            inlineExplainsBusy_ = false;
          }
        } else {
          (void)hipGetLastError();  // "not ready" (or a failure the record below will report)
          // (what keeps it busy may be a small operation of this context's own,
          // launched there a moment ago and gone by the next time: ask again then)
          bool ownLaunch = false;
          {
            std::lock_guard<std::mutex> ig(inlineMu_);
            ownLaunch = inlineExplainsBusy_ && inlineStream_ == req.producerStream;
            inlineExplainsBusy_ = false;  // once per launch
          }
          if (!ownLaunch) {
            busyProducer_.store(req.producerStream, std::memory_order_relaxed);
            busyProducerSkips_.store(kBusyProducerSkips, std::memory_order_relaxed);
          }
        }
      }
    }
    if (!producerIdle) {
      initial = takeEvent();
      FRG_HIP_CHECK(hipEventRecord(initial, req.producerStream));
    }
  } catch (const std::exception& e) {
    *err = e.what();
    if (initial) giveEvent(initial);
    releaseWork(work);
    // counted as dealt with: the counters stay level for what comes after
    progress_->started.fetch_add(1);
    progress_->enqueued.fetch_add(1);
    return FRG_ERR_HIP;
  }
  if (workOut) {
    work->refs.fetch_add(1);
    *workOut = work;
  }
  auto queued = std::make_shared<QueuedOp>();
  queued->req = std::move(req);
  queued->initial = initial;
  queued->work = work;
  queue_.enqueue(std::move(queued));
  return FRG_OK;
}

// Enqueues one launch and keeps the books around it: the running totals per
// reduce stream and, with per-launch profiling on, the timing events of the
// dispatch. Failures become exceptions that run() turns into the work's status.
template <typename Args>
void Context::launchAndCount(const Args& args, hipStream_t stream,
                             int (*enqueue)(const Args&, hipStream_t, std::string*)) {
  Args a = args;
  const bool prof = profiling_.load(std::memory_order_relaxed) && args.n > 0;
  if (prof) {
    FRG_HIP_CHECK(hipEventCreate(&a.startEvent));
    FRG_HIP_CHECK(hipEventCreate(&a.stopEvent));
  }
  std::string err;
  const int rc = enqueue(a, stream, &err);
  if (rc == FRG_OK && args.n > 0) {
    for (size_t i = 0; i < reduceStreams_.size(); ++i) {
      if (reduceStreams_[i] == stream) {
        streamLaunches_[i] += 1;
        streamElems_[i] += args.n;
      }
    }
    lastContribs_ = args.K;
    progress_->launches.fetch_add(1);
  }
  if (prof) {
    if (rc == FRG_OK) {
      std::lock_guard<std::mutex> g(profMu_);
      profEvents_.push_back(ProfRecord{a.startEvent, a.stopEvent, a.n, a.K, stream, 1});
    } else {
      (void)hipEventDestroy(a.startEvent);
      (void)hipEventDestroy(a.stopEvent);
    }
  }
  if (rc == FRG_ERR_HIP) throw HipFailure(err);
  if (rc != FRG_OK) throw ContractFailure(rc, err);
}

void Context::launch(const ReduceArgs& args, hipStream_t stream) {
  launchAndCount<ReduceArgs>(args, stream, &launchReduce);
}

void Context::launchCompressed(const CompressedArgs& args, hipStream_t stream) {
  launchAndCount<CompressedArgs>(args, stream, &launchCompressedReduce);
}

// One launch over several pieces; the books count its elements like any launch's.
void Context::launchSegments(const SegmentedArgs& args, hipStream_t stream) {
  SegmentedArgs a = args;
  int64_t elems = 0;
  for (int i = 0; i < args.numPieces; ++i) elems += args.pieces[i].n;
  const bool prof = profiling_.load(std::memory_order_relaxed) && elems > 0;
  if (prof) {
    FRG_HIP_CHECK(hipEventCreate(&a.startEvent));
    FRG_HIP_CHECK(hipEventCreate(&a.stopEvent));
  }
  std::string err;
  const int rc = launchSegmented(a, stream, &err);
  if (rc == FRG_OK && elems > 0) {
    for (size_t i = 0; i < reduceStreams_.size(); ++i) {
      if (reduceStreams_[i] == stream) {
        streamLaunches_[i] += 1;
        streamElems_[i] += elems;
      }
    }
    lastContribs_ = args.K;
    progress_->launches.fetch_add(1);
    progress_->segmentedLaunches.fetch_add(1);
  }
  if (prof) {
    if (rc == FRG_OK) {
      std::lock_guard<std::mutex> g(profMu_);
      profEvents_.push_back(ProfRecord{a.startEvent, a.stopEvent, elems, a.K, stream, 1});
    } else {
      (void)hipEventDestroy(a.startEvent);
      (void)hipEventDestroy(a.stopEvent);
    }
  }
  if (rc == FRG_ERR_HIP) throw HipFailure(err);
  if (rc != FRG_OK) throw ContractFailure(rc, err);
}

// Start of the allocation that holds `p` (what hipMalloc returned for it), or 0
// when the runtime does not know the pointer: physical memory is laid out from
// there, so that is where the 4 MiB multiples that matter to the launch
// partition are counted from. The last answer is kept: the buckets of a
// gradient mostly share an allocation.
uint64_t Context::allocationBase(const void* p) {
  const uint64_t a = reinterpret_cast<uint64_t>(p);
  if (a >= allocBase_ && a - allocBase_ < allocSize_) return allocBase_;
  hipDeviceptr_t base = nullptr;
  size_t size = 0;
  if (hipMemGetAddressRange(&base, &size, const_cast<void*>(p)) != hipSuccess || size == 0) {
    (void)hipGetLastError();
    return 0;
  }
  allocBase_ = reinterpret_cast<uint64_t>(base);
  allocSize_ = size;
  return allocBase_;
}

// ---- order between operations ----------------------------------------------

Context::OpSpans Context::spansOf(const Request& req) {
  OpSpans op;
  const uintptr_t wireSize = static_cast<uintptr_t>(elementSize(req.dtype));
  const uintptr_t outSize =
      req.compressed ? static_cast<uintptr_t>(elementSize(req.outDtype)) : wireSize;
  const uintptr_t n = static_cast<uintptr_t>(req.numel);
  const uintptr_t o = reinterpret_cast<uintptr_t>(req.out);
  op.write = Span{o, o + n * outSize};
  if (!req.fromHost) {  // host memory is not written by any operation of the pipeline
    op.reads.reserve(req.contribs.size());
    for (size_t k = 0; k < req.contribs.size(); ++k) {
      const uintptr_t p = reinterpret_cast<uintptr_t>(req.contribs[k]);
      if (p == o) continue;  // in place: covered by the write
      if (static_cast<int>(k) == req.gatheredIndex) continue;  // given piecewise, below
      const uintptr_t es = (req.compressed && static_cast<int>(k) == req.rawIndex) ? 4 : wireSize;
      op.reads.push_back(Span{p, p + n * es});
    }
    const uintptr_t segSize = req.compressed ? 4 : wireSize;  // the raw contribution is fp32
    for (const Request::Segment& g : req.gathered) {
      const uintptr_t p = reinterpret_cast<uintptr_t>(g.ptr);
      if (g.numel > 0) op.reads.push_back(Span{p, p + static_cast<uintptr_t>(g.numel) * segSize});
    }
  }
  return op;
}

// Two operations conflict when one writes what the other reads or writes.
bool Context::conflict(const OpSpans& a, const OpSpans& b) {
  auto overlap = [](const Span& x, const Span& y) { return x.lo < y.hi && y.lo < x.hi; };
  if (overlap(a.write, b.write)) return true;
  for (const Span& r : b.reads) {
    if (overlap(a.write, r)) return true;
  }
  for (const Span& r : a.reads) {
    if (overlap(r, b.write)) return true;
  }
  return false;
}

void Context::joinTail(size_t src, size_t target) {
  hipEvent_t e = takeEvent();
  hipError_t r = hipEventRecord(e, reduceStreams_[src]);
  if (r == hipSuccess) r = hipStreamWaitEvent(reduceStreams_[target], e, 0);
  giveEvent(e);
  FRG_HIP_CHECK(r);
  if (!history_[src].empty()) orderedAfter_[target][src] = history_[src].back().seq;
}

void Context::orderAfterConflicts(const OpSpans& op, const std::vector<size_t>& targets) {
  const size_t n = reduceStreams_.size();
  if (n < 2) return;
  for (size_t s = 0; s < n; ++s) {
    if (history_[s].empty()) continue;
    for (size_t t : targets) {
      if (t == s) continue;
      const int64_t seen = orderedAfter_[t][s];
      bool hit = false;
      // newest first: what conflicts is most often what was submitted last
      for (auto it = history_[s].rbegin(); it != history_[s].rend() && it->seq > seen; ++it) {
        if (conflict(op, *it)) {
          hit = true;
          break;
        }
      }
      if (!hit) continue;
      // What has already finished orders nothing: a stream that has drained is
      // behind everything and its history can go (a host-side question to the
      // runtime, asked only on a conflict; a join costs an event packet on
      // either stream).
      if (hipStreamQuery(reduceStreams_[s]) == hipSuccess) {
        for (size_t u = 0; u < n; ++u) orderedAfter_[u][s] = history_[s].back().seq;
        history_[s].clear();
        break;
      }
      (void)hipGetLastError();
      joinTail(s, t);
    }
  }
}

void Context::remember(OpSpans op, const std::vector<size_t>& targets) {
  const size_t n = reduceStreams_.size();
  if (n < 2 || op.write.lo == op.write.hi) return;
  op.seq = ++spanSeq_;
  for (size_t t : targets) {
    std::deque<OpSpans>& h = history_[t];
    h.push_back(op);
    // what every other stream already follows need not be kept
    int64_t followed = h.back().seq;
    for (size_t u = 0; u < n; ++u) {
      if (u != t && orderedAfter_[u][t] < followed) followed = orderedAfter_[u][t];
    }
    while (!h.empty() && h.front().seq <= followed) h.pop_front();
    if (h.size() > kMaxHistory) {
      // bounded memory and search: order every other stream after this one
      // (one event record, one wait per stream, once in kMaxHistory operations)
      for (size_t u = 0; u < n; ++u) {
        if (u != t) joinTail(t, u);
      }
      h.clear();
    }
  }
}

void Context::waitInitial(hipStream_t stream, hipEvent_t initialEvent, bool* fired) {
  if (initialEvent == nullptr) return;  // the producer stream was idle when the operation came in
  // Once the producer's event has fired no stream needs to wait for it: a
  // wait that is already satisfied still costs a barrier packet on the queue.
  if (!*fired) {
    if (hipEventQuery(initialEvent) == hipSuccess) {
      *fired = true;
    } else {
      (void)hipGetLastError();  // "not ready" is an answer, not a failure to keep
    }
  }
  if (!*fired) FRG_HIP_CHECK(hipStreamWaitEvent(stream, initialEvent, 0));
}

// Whether `next`, which was submitted right after `last`, continues it: the
// same reduction over buffers that lie directly below (direction -1) or above
// (+1) those of `last`, output and every contribution alike, so that the two
// are one elementwise operation over the joint range. `bytesSoFar`: the length
// of the run that ends in `last`; `*direction` is 0 until the first pair has
// set it.
bool Context::adjoins(const QueuedOp& last, const QueuedOp& next, int64_t bytesSoFar,
                      int* direction) {
  const Request& a = last.req;
  const Request& b = next.req;
  if (!launchBytesByContribs_ || a.fromHost || b.fromHost || a.compressed || b.compressed ||
      !a.gathered.empty() || !b.gathered.empty()) {
    return false;
  }
  if (a.dtype != b.dtype || a.op != b.op || a.scaleMode != b.scaleMode || a.scale != b.scale ||
      a.contribs.size() != b.contribs.size() || a.numel <= 0 || b.numel <= 0 ||
      a.contribs.size() > static_cast<size_t>(kMaxContribsPerLaunch)) {
    return false;
  }
  const uintptr_t elsize = static_cast<uintptr_t>(elementSize(a.dtype));
  const uintptr_t aBytes = static_cast<uintptr_t>(a.numel) * elsize;
  const uintptr_t bBytes = static_cast<uintptr_t>(b.numel) * elsize;
  const uintptr_t ao = reinterpret_cast<uintptr_t>(a.out);
  const uintptr_t bo = reinterpret_cast<uintptr_t>(b.out);
  int dir = 0;
  if (bo + bBytes == ao) dir = -1;
  if (ao + aBytes == bo) dir = +1;
  if (dir == 0 || (*direction != 0 && dir != *direction)) return false;
  for (size_t k = 0; k < a.contribs.size(); ++k) {
    const uintptr_t ap = reinterpret_cast<uintptr_t>(a.contribs[k]);
    const uintptr_t bp = reinterpret_cast<uintptr_t>(b.contribs[k]);
    if (dir < 0 ? bp + bBytes != ap : ap + aBytes != bp) return false;
    // Over the joint range a contribution is the output itself or apart from
    // it: operations of which one reads what another writes are not one. Every
    // operation of the run has the same distance between the two, so the
    // question is whether that distance is shorter than the run.
    const uintptr_t distance = ap > ao ? ap - ao : ao - ap;
    if (distance != 0 && distance < static_cast<uintptr_t>(bytesSoFar) + bBytes) return false;
  }
  if (allocationBase(a.out) != allocationBase(b.out)) return false;
  *direction = dir;
  return true;
}

// One operation, or several neighbours as one (see adjoins()): enqueues the
// launches, then marks every work and calls every callback, in submission order.
void Context::runGroup(const std::vector<std::shared_ptr<QueuedOp>>& group) {
  const size_t count = group.size();
  pipelineOps_.fetch_add(static_cast<int64_t>(count), std::memory_order_acq_rel);
  const int64_t firstSeq = nextSeq_;
  nextSeq_ += static_cast<int64_t>(count);
  progress_->started.fetch_add(static_cast<int64_t>(count));
  if (count > 1) progress_->merged.fetch_add(static_cast<int64_t>(count));
  int status = FRG_OK;
  std::string error;
  hipStream_t lastStream = reduceStreams_[0];
  std::vector<hipStream_t> used;
  try {
    const Request* req = &group[0]->req;
    Request joint;
    int64_t slices = -1;
    if (count > 1) {
      // the joint range starts where the lowest of them does
      const QueuedOp* lowest = group[0].get();
      const int64_t elsize = elementSize(req->dtype);
      slices = 0;
      int64_t numel = 0;
      for (const auto& op : group) {
        if (op->req.out < lowest->req.out) lowest = op.get();
        numel += op->req.numel;
        slices += numSlices(op->req.numel, layout_.sliceSizeInBytes, elsize);
      }
      joint = lowest->req;
      joint.numel = numel;
      joint.done = nullptr;
      joint.user = nullptr;
      req = &joint;
    }
    // what the producers recorded: of one stream's events the last covers the others
    std::vector<hipEvent_t> initials;
    std::vector<hipStream_t> producers;
    bool anyCallback = false;
    for (const auto& op : group) {
      anyCallback = anyCallback || op->req.done != nullptr;
      if (op->initial == nullptr) continue;
      size_t at = producers.size();
      for (size_t i = 0; i < producers.size(); ++i) {
        if (producers[i] == op->req.producerStream) at = i;
      }
      if (at == producers.size()) {
        producers.push_back(op->req.producerStream);
        initials.push_back(op->initial);
      } else {
        initials[at] = op->initial;
      }
    }
    used = req->fromHost ? runHostStaged(*req, initials.empty() ? nullptr : initials[0])
                         : (!req->gathered.empty() ? runGathered(*req, initials)
                                                   : runResident(*req, initials, slices));
    lastStream = used.back();
    if (anyCallback && used.size() > 1) {
      // The callback orders consumers after ONE stream (fairring/device.cc:337-340
      // marks the future under a guard of the last stream): join the others into it.
      for (size_t i = 0; i + 1 < used.size(); ++i) {
        hipEvent_t j = takeEvent();
        hipError_t r = hipEventRecord(j, used[i]);
        if (r == hipSuccess) r = hipStreamWaitEvent(lastStream, j, 0);
        giveEvent(j);
        FRG_HIP_CHECK(r);
      }
      used.assign(1, lastStream);
    }
    // Without a callback nothing needs a single stream, and the streams keep
    // running independently of each other.
  } catch (const ContractFailure& e) {
    status = e.code;
    error = e.what();
    used.clear();
  } catch (const std::exception& e) {
    status = FRG_ERR_HIP;
    error = e.what();
    used.clear();
  }
  if (status != FRG_OK) {
    std::fprintf(stderr, "[fairring] operation #%lld%s failed: %s\n",
                 static_cast<long long>(firstSeq), count > 1 ? " (and its neighbours)" : "",
                 error.c_str());
  }
  for (const auto& op : group) {
    Work* work = op->work;
    work->doneStreams = used;
    // where the operation stands on each of them, for waits that are remembered
    for (hipStream_t s : used) {
      int idx = -1;
      for (size_t i = 0; i < reduceStreams_.size(); ++i) {
        if (reduceStreams_[i] == s) idx = static_cast<int>(i);
      }
      int64_t position = -1;
      if (idx >= 0 && idx < Progress::kMaxStreams) {
        position = progress_->streamPosition[idx].fetch_add(1, std::memory_order_acq_rel) + 1;
      }
      work->doneIndices.push_back(idx);
      work->donePositions.push_back(position);
    }
    if (op->initial != nullptr) giveEvent(op->initial);
    progress_->enqueued.fetch_add(1);
    {
      std::lock_guard<std::mutex> g(work->mu);
      work->status = status;
      work->error = error;
      work->lastStream = lastStream;
      work->enqueued = true;
      work->enqueuedFlag.store(true, std::memory_order_release);
    }
    work->cv.notify_all();
    if (op->req.done) op->req.done(op->req.user, status, lastStream);
    releaseWork(work);
  }
}

int Context::synchronize(std::string* err) {
  // A marker through the queue: everything submitted before it is enqueued
  // once it runs.
  std::mutex mu;
  std::condition_variable cv;
  bool reached = false;
  queue_.enqueue([&] {
    std::lock_guard<std::mutex> g(mu);
    reached = true;
    cv.notify_all();
  });
  {
    std::unique_lock<std::mutex> lock(mu);
    cv.wait(lock, [&] { return reached; });
  }
  try {
    DeviceGuard g(device_);
    for (hipStream_t s : reduceStreams_) FRG_HIP_CHECK(hipStreamSynchronize(s));
    for (hipStream_t s : copyStreams_) FRG_HIP_CHECK(hipStreamSynchronize(s));
    std::lock_guard<std::mutex> ig(inlineMu_);
    if (inlinePending_) {  // what went to a caller's stream
      FRG_HIP_CHECK(inlineRecorded_ ? hipEventSynchronize(inlineEvent_)
                                    : hipStreamSynchronize(nullptr));
      inlinePending_ = false;
    }
  } catch (const std::exception& e) {
    *err = e.what();
    return FRG_ERR_HIP;
  }
  return FRG_OK;
}

void Context::setProfiling(bool perLaunch) { profiling_.store(perLaunch); }

int Context::profileMark(std::string* err) {
  std::mutex mu;
  std::condition_variable cv;
  bool reached = false;
  int status = FRG_OK;
  queue_.enqueue([&] {
    Mark m;
    try {
      for (hipStream_t s : reduceStreams_) {
        hipEvent_t e;
        FRG_HIP_CHECK(hipEventCreate(&e));
        m.events.push_back(e);
        FRG_HIP_CHECK(hipEventRecord(e, s));
      }
      m.launches = streamLaunches_;
      m.elems = streamElems_;
      std::lock_guard<std::mutex> g(profMu_);
      marks_.push_back(std::move(m));
    } catch (const std::exception& e) {
      for (hipEvent_t ev : m.events) (void)hipEventDestroy(ev);
      status = FRG_ERR_HIP;
      *err = e.what();
    }
    std::lock_guard<std::mutex> g(mu);
    reached = true;
    cv.notify_all();
  });
  std::unique_lock<std::mutex> lock(mu);
  cv.wait(lock, [&] { return reached; });
  return status;
}

int Context::launchRecords(frg_launch_record* recs, int capacity, int* count, std::string* err) {
  const int rc = synchronize(err);
  if (rc != FRG_OK) return rc;
  std::vector<ProfRecord> evs;
  std::vector<Mark> marks;
  {
    std::lock_guard<std::mutex> g(profMu_);
    evs.swap(profEvents_);
    marks.swap(marks_);
  }
  int n = 0;
  int status = FRG_OK;
  auto elapsed = [&](hipEvent_t from, hipEvent_t to) {
    float t = 0.f;
    const hipError_t r = hipEventElapsedTime(&t, from, to);
    if (r != hipSuccess && status == FRG_OK) {
      status = FRG_ERR_HIP;
      *err = std::string("hipEventElapsedTime: ") + hipGetErrorString(r);
    }
    return t;
  };
  auto emit = [&](float b, float e, int64_t numel, int contribs, int si, int64_t launches) {
    if (n < capacity && recs) {
      recs[n] = frg_launch_record{b, e, numel, contribs, si, static_cast<int32_t>(launches), 0};
    }
    ++n;
  };
  // regions between consecutive marks, one record per stream that ran anything
  for (size_t m = 0; m + 1 < marks.size(); ++m) {
    for (size_t si = 0; si < marks[m].events.size(); ++si) {
      const int64_t launches = marks[m + 1].launches[si] - marks[m].launches[si];
      if (launches <= 0) continue;
      emit(elapsed(marks[0].events[0], marks[m].events[si]),
           elapsed(marks[0].events[0], marks[m + 1].events[si]),
           marks[m + 1].elems[si] - marks[m].elems[si], lastContribs_, static_cast<int>(si),
           launches);
    }
  }
  // per-launch records
  for (auto& p : evs) {
    int si = 0;
    for (size_t i = 0; i < reduceStreams_.size(); ++i) {
      if (reduceStreams_[i] == p.stream) si = static_cast<int>(i);
    }
    emit(elapsed(evs.front().begin, p.begin), elapsed(evs.front().begin, p.end), p.numel,
         p.numContribs, si, 1);
  }
  for (auto& p : evs) {
    (void)hipEventDestroy(p.begin);
    (void)hipEventDestroy(p.end);
  }
  for (auto& m : marks) {
    for (hipEvent_t e : m.events) (void)hipEventDestroy(e);
  }
  if (count) *count = n;
  return status;
}

int Context::kernelTimes(float* ms, int capacity, int* count, std::string* err) {
  std::vector<frg_launch_record> recs(static_cast<size_t>(capacity > 0 ? capacity : 0));
  int n = 0;
  const int rc = launchRecords(recs.data(), capacity, &n, err);
  for (int i = 0; i < n && i < capacity && ms; ++i) ms[i] = recs[i].end_ms - recs[i].begin_ms;
  if (count) *count = n;
  return rc;
}

}  // namespace frg
