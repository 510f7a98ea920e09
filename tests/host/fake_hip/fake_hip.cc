// See hip/hip_runtime.h in this directory. Test infrastructure only.
#include <atomic>
#include <hip/hip_runtime.h>

#include <chrono>
#include <condition_variable>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <functional>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <thread>
#include <utility>
#include <vector>

namespace {

using Clock = std::chrono::steady_clock;

struct Record {
  std::mutex mu;
  std::condition_variable cv;
  bool done = false;
  Clock::time_point when;
};

std::mutex gCallMu;
std::map<std::string, long> gCalls;
std::map<std::string, long> gFailAt;  // api -> absolute call number that fails

// Counts the call and says whether this one is the injected failure.
bool enter(const char* api) {
  std::lock_guard<std::mutex> g(gCallMu);
  const long n = ++gCalls[api];
  auto it = gFailAt.find(api);
  if (it != gFailAt.end() && it->second == n) {
    gFailAt.erase(it);
    return true;
  }
  return false;
}

thread_local int tlsDevice = 0;
thread_local hipError_t tlsLastError = hipSuccess;

hipError_t ret(hipError_t e) {
  if (e != hipSuccess) tlsLastError = e;
  return e;
}

}  // namespace

// A hardware queue: packets of every stream mapped onto it run strictly in the
// order they were written, one at a time, so a wait packet holds up everything
// behind it whatever stream that belongs to (the barrier bit of an in-order AQL
// queue). With fake_hip_set_hw_queues(0) every stream has a queue of its own.
struct HwQueue {
  std::mutex mu;
  std::condition_variable cv;
  std::deque<std::pair<FakeStream*, std::function<void()>>> packets;
  bool stop = false;
  std::thread worker;

  HwQueue();
  ~HwQueue() {
    {
      std::lock_guard<std::mutex> g(mu);
      stop = true;
    }
    cv.notify_all();
    worker.join();
  }
};

struct FakeStream {
  std::mutex mu;
  std::condition_variable cv;
  long submitted = 0;
  long finished = 0;
  bool blocking = false;  // takes part in the null stream's implicit synchronisation
  HwQueue* queue = nullptr;
  bool ownsQueue = false;

  FakeStream(HwQueue* shared, bool blockingStream) : blocking(blockingStream) {
    if (shared != nullptr) {
      queue = shared;
    } else {
      queue = new HwQueue();
      ownsQueue = true;
    }
  }

  ~FakeStream() {
    drain();
    if (ownsQueue) delete queue;
  }

  void push(std::function<void()> fn) {
    {
      std::lock_guard<std::mutex> g(mu);
      ++submitted;
    }
    {
      std::lock_guard<std::mutex> g(queue->mu);
      queue->packets.emplace_back(this, std::move(fn));
    }
    queue->cv.notify_all();
  }

  void drain() {
    std::unique_lock<std::mutex> lock(mu);
    const long target = submitted;
    cv.wait(lock, [&] { return finished >= target; });
  }

  bool idle() {
    std::lock_guard<std::mutex> lock(mu);
    return finished >= submitted;
  }
};

HwQueue::HwQueue() {
  worker = std::thread([this] {
    while (true) {
      std::pair<FakeStream*, std::function<void()>> p;
      {
        std::unique_lock<std::mutex> lock(mu);
        cv.wait(lock, [&] { return stop || !packets.empty(); });
        if (packets.empty()) return;
        p = std::move(packets.front());
        packets.pop_front();
      }
      p.second();
      {
        std::lock_guard<std::mutex> g(p.first->mu);
        ++p.first->finished;
      }
      p.first->cv.notify_all();
    }
  });
}

struct FakeEvent {
  std::mutex mu;
  std::shared_ptr<Record> current;  // the latest record, if any
};

namespace {

std::mutex gTopologyMu;
std::vector<HwQueue*> gSharedQueues;  // empty: a queue per stream
size_t gNextQueue = 0;
FakeStream* gDefaultStream = nullptr;
std::vector<FakeStream*> gBlockingStreams;  // live streams created without hipStreamNonBlocking
std::vector<FakeStream*> gAllStreams;       // every live stream but the null stream

HwQueue* pickQueueLocked() {
  if (gSharedQueues.empty()) return nullptr;
  return gSharedQueues[gNextQueue++ % gSharedQueues.size()];
}

FakeStream* defaultStream() {
  std::lock_guard<std::mutex> g(gTopologyMu);
  if (gDefaultStream == nullptr) {
    // lives until the topology is changed, like the null stream
    gDefaultStream = new FakeStream(pickQueueLocked(), /*blockingStream=*/true);
  }
  return gDefaultStream;
}

FakeStream* resolve(hipStream_t s) { return s ? s : defaultStream(); }

std::shared_ptr<Record> recordOn(FakeStream* s) {
  auto r = std::make_shared<Record>();
  s->push([r] {
    {
      std::lock_guard<std::mutex> g(r->mu);
      r->done = true;
      r->when = Clock::now();
    }
    r->cv.notify_all();
  });
  return r;
}

void waitOn(FakeStream* s, std::shared_ptr<Record> r) {
  s->push([r] {
    std::unique_lock<std::mutex> lock(r->mu);
    r->cv.wait(lock, [&] { return r->done; });
  });
}

// How a stream wait binds to its event: to the record the event held when the
// wait was enqueued (what the HIP runtime does, the default), or, as a probe,
// to whatever record the event holds when the wait packet is executed.
std::atomic<int> gLatestRecordWaits{0};
std::mutex gGraveyardMu;
std::vector<FakeEvent*> gGraveyard;  // destroyed events a late-binding wait may still read

bool recordDone(const std::shared_ptr<Record>& r) {
  std::lock_guard<std::mutex> g(r->mu);
  return r->done;
}

// The legacy null stream: work submitted to it starts after everything
// submitted so far to the blocking streams, and work submitted to a blocking
// stream starts after everything submitted so far to the null stream. Streams
// created with hipStreamNonBlocking stay out of it.
void implicitSync(FakeStream* target) {
  std::vector<FakeStream*> others;
  FakeStream* null = nullptr;
  {
    std::lock_guard<std::mutex> g(gTopologyMu);
    null = gDefaultStream;
    if (target == null) {
      others = gBlockingStreams;
    } else if (target->blocking && null != nullptr) {
      others.push_back(null);
    }
  }
  for (FakeStream* o : others) {
    if (o != target && !o->idle()) waitOn(target, recordOn(o));
  }
}

// Every submission of real work goes through here.
void submit(hipStream_t stream, std::function<void()> fn) {
  FakeStream* s = resolve(stream);
  implicitSync(s);
  s->push(std::move(fn));
}

}  // namespace

void fake_hip_enqueue(hipStream_t stream, void (*fn)(void*), void* arg) {
  submit(stream, [fn, arg] { fn(arg); });
}

extern "C" {

hipError_t hipGetDeviceCount(int* count) {
  if (enter("hipGetDeviceCount")) return ret(hipErrorUnknown);
  *count = 1;
  return hipSuccess;
}

hipError_t hipGetDevice(int* device) {
  enter("hipGetDevice");
  *device = tlsDevice;
  return hipSuccess;
}

hipError_t hipSetDevice(int device) {
  enter("hipSetDevice");
  if (device != 0) return ret(hipErrorInvalidDevice);
  tlsDevice = device;
  return hipSuccess;
}

hipError_t hipDeviceGetAttribute(int* value, hipDeviceAttribute_t, int) {
  enter("hipDeviceGetAttribute");
  *value = 4;
  return hipSuccess;
}

hipError_t hipGetLastError(void) {
  const hipError_t e = tlsLastError;
  tlsLastError = hipSuccess;
  return e;
}

const char* hipGetErrorString(hipError_t e) {
  switch (e) {
    case hipSuccess:
      return "no error";
    case hipErrorNotReady:
      return "not ready";
    case hipErrorOutOfMemory:
      return "out of memory";
    case hipErrorInvalidValue:
      return "invalid value";
    default:
      return "injected failure";
  }
}

hipError_t hipStreamCreateWithFlags(hipStream_t* stream, unsigned int flags) {
  if (enter("hipStreamCreateWithFlags")) return ret(hipErrorUnknown);
  const bool blocking = (flags & hipStreamNonBlocking) == 0;
  std::lock_guard<std::mutex> g(gTopologyMu);
  *stream = new FakeStream(pickQueueLocked(), blocking);
  if (blocking) gBlockingStreams.push_back(*stream);
  gAllStreams.push_back(*stream);
  return hipSuccess;
}

hipError_t hipStreamDestroy(hipStream_t stream) {
  enter("hipStreamDestroy");
  if (stream == nullptr) return ret(hipErrorInvalidValue);
  {
    std::lock_guard<std::mutex> g(gTopologyMu);
    for (std::vector<FakeStream*>* list : {&gBlockingStreams, &gAllStreams}) {
      for (size_t i = 0; i < list->size(); ++i) {
        if ((*list)[i] == stream) {
          list->erase(list->begin() + static_cast<long>(i));
          break;
        }
      }
    }
  }
  delete stream;  // drains it first
  return hipSuccess;
}

hipError_t hipStreamSynchronize(hipStream_t stream) {
  if (enter("hipStreamSynchronize")) return ret(hipErrorUnknown);
  resolve(stream)->drain();
  return hipSuccess;
}

hipError_t hipStreamWaitEvent(hipStream_t stream, hipEvent_t event, unsigned int) {
  if (enter("hipStreamWaitEvent")) return ret(hipErrorUnknown);
  std::shared_ptr<Record> r;
  {
    std::lock_guard<std::mutex> g(event->mu);
    r = event->current;  // snapshot: later records of the event do not matter
  }
  if (!r) return hipSuccess;
  FakeStream* s = resolve(stream);
  if (gLatestRecordWaits.load()) {
    // a wait on a record that has fired is no packet at all, as in the runtime
    if (recordDone(r)) return hipSuccess;
    implicitSync(s);
    s->push([event] {
      std::shared_ptr<Record> latest;
      {
        std::lock_guard<std::mutex> g(event->mu);
        latest = event->current;
      }
      if (!latest) return;
      std::unique_lock<std::mutex> lock(latest->mu);
      latest->cv.wait(lock, [&] { return latest->done; });
    });
    return hipSuccess;
  }
  implicitSync(s);
  waitOn(s, r);
  return hipSuccess;
}

hipError_t hipEventCreateWithFlags(hipEvent_t* event, unsigned int) {
  if (enter("hipEventCreate")) return ret(hipErrorUnknown);
  *event = new FakeEvent();
  return hipSuccess;
}

hipError_t hipEventCreate(hipEvent_t* event) { return hipEventCreateWithFlags(event, 0); }

hipError_t hipEventDestroy(hipEvent_t event) {
  enter("hipEventDestroy");
  if (gLatestRecordWaits.load()) {
    // a wait that binds late still reads the event: it is kept, with its last record
    std::lock_guard<std::mutex> g(gGraveyardMu);
    gGraveyard.push_back(event);
    return hipSuccess;
  }
  delete event;  // pending waits hold their own reference to the record
  return hipSuccess;
}

hipError_t hipEventRecord(hipEvent_t event, hipStream_t stream) {
  if (enter("hipEventRecord")) return ret(hipErrorUnknown);
  FakeStream* s = resolve(stream);
  implicitSync(s);
  // the packet is written and the event updated as one step, as the runtime
  // does under the event's lock
  std::lock_guard<std::mutex> g(event->mu);
  event->current = recordOn(s);
  return hipSuccess;
}

hipError_t hipStreamQuery(hipStream_t stream) {
  enter("hipStreamQuery");
  return resolve(stream)->idle() ? hipSuccess : ret(hipErrorNotReady);
}

static std::atomic<int> gCapturing{0};

void fake_hip_set_capturing(int on) { gCapturing = on; }

hipError_t hipStreamIsCapturing(hipStream_t /*stream*/, hipStreamCaptureStatus* status) {
  enter("hipStreamIsCapturing");
  *status = gCapturing.load() ? hipStreamCaptureStatusActive : hipStreamCaptureStatusNone;
  return hipSuccess;
}

hipError_t hipEventQuery(hipEvent_t event) {
  enter("hipEventQuery");
  std::shared_ptr<Record> r;
  {
    std::lock_guard<std::mutex> g(event->mu);
    r = event->current;
  }
  if (!r) return hipSuccess;
  std::lock_guard<std::mutex> g(r->mu);
  return r->done ? hipSuccess : ret(hipErrorNotReady);
}

hipError_t hipEventSynchronize(hipEvent_t event) {
  if (enter("hipEventSynchronize")) return ret(hipErrorUnknown);
  std::shared_ptr<Record> r;
  {
    std::lock_guard<std::mutex> g(event->mu);
    r = event->current;
  }
  if (!r) return hipSuccess;
  std::unique_lock<std::mutex> lock(r->mu);
  r->cv.wait(lock, [&] { return r->done; });
  return hipSuccess;
}

hipError_t hipEventElapsedTime(float* ms, hipEvent_t start, hipEvent_t stop) {
  enter("hipEventElapsedTime");
  std::shared_ptr<Record> a, b;
  {
    std::lock_guard<std::mutex> g(start->mu);
    a = start->current;
  }
  {
    std::lock_guard<std::mutex> g(stop->mu);
    b = stop->current;
  }
  if (!a || !b) return ret(hipErrorInvalidValue);
  Clock::time_point ta, tb;
  {
    std::lock_guard<std::mutex> g(a->mu);
    if (!a->done) return ret(hipErrorNotReady);
    ta = a->when;
  }
  {
    std::lock_guard<std::mutex> g(b->mu);
    if (!b->done) return ret(hipErrorNotReady);
    tb = b->when;
  }
  *ms = std::chrono::duration<float, std::milli>(tb - ta).count();
  return hipSuccess;
}

static std::mutex gAllocMu;
static std::map<uintptr_t, size_t> gAllocs;  // what hipMalloc handed out

hipError_t hipMalloc(void** ptr, size_t size) {
  if (enter("hipMalloc")) return ret(hipErrorOutOfMemory);
  // device allocations start on a page boundary
  *ptr = nullptr;
  if (posix_memalign(ptr, 4096, size ? size : 1) != 0) return ret(hipErrorOutOfMemory);
  std::lock_guard<std::mutex> g(gAllocMu);
  gAllocs[reinterpret_cast<uintptr_t>(*ptr)] = size ? size : 1;
  return hipSuccess;
}

hipError_t hipFree(void* ptr) {
  enter("hipFree");
  {
    std::lock_guard<std::mutex> g(gAllocMu);
    gAllocs.erase(reinterpret_cast<uintptr_t>(ptr));
  }
  std::free(ptr);
  return hipSuccess;
}

hipError_t hipMemGetAddressRange(hipDeviceptr_t* base, size_t* size, hipDeviceptr_t ptr) {
  enter("hipMemGetAddressRange");
  const uintptr_t a = reinterpret_cast<uintptr_t>(ptr);
  std::lock_guard<std::mutex> g(gAllocMu);
  auto it = gAllocs.upper_bound(a);
  if (it == gAllocs.begin()) return ret(hipErrorInvalidValue);
  --it;
  if (a - it->first >= it->second) return ret(hipErrorInvalidValue);
  *base = reinterpret_cast<void*>(it->first);
  *size = it->second;
  return hipSuccess;
}

hipError_t hipMemcpyAsync(void* dst, const void* src, size_t bytes, hipMemcpyKind,
                          hipStream_t stream) {
  if (enter("hipMemcpyAsync")) return ret(hipErrorUnknown);
  submit(stream, [dst, src, bytes] { std::memcpy(dst, src, bytes); });
  return hipSuccess;
}

void fake_hip_occupy(hipStream_t stream, int ms) {
  submit(stream, [ms] { std::this_thread::sleep_for(std::chrono::milliseconds(ms)); });
}

void fake_hip_set_hw_queues(int n) {
  FakeStream* old = nullptr;
  {
    std::lock_guard<std::mutex> g(gTopologyMu);
    old = gDefaultStream;
    gDefaultStream = nullptr;
  }
  if (old != nullptr) old->drain();  // left alive: an event may still point into it
  std::lock_guard<std::mutex> g(gTopologyMu);
  for (FakeStream* s : gAllStreams) s->drain();
  for (HwQueue* q : gSharedQueues) delete q;  // idle: everything mapped onto them is drained
  gSharedQueues.clear();
  gNextQueue = 0;
  for (int i = 0; i < n; ++i) gSharedQueues.push_back(new HwQueue());
  // the streams that exist move onto the new queues in the order they were created
  for (FakeStream* s : gAllStreams) {
    if (s->ownsQueue) delete s->queue;
    HwQueue* shared = pickQueueLocked();
    s->ownsQueue = shared == nullptr;
    s->queue = shared != nullptr ? shared : new HwQueue();
  }
}

void fake_hip_set_latest_record_waits(int on) { gLatestRecordWaits = on; }

void fake_hip_fail_call(const char* api, int nth) {
  std::lock_guard<std::mutex> g(gCallMu);
  gFailAt[api] = gCalls[api] + nth;
}

long fake_hip_calls(const char* api) {
  std::lock_guard<std::mutex> g(gCallMu);
  return gCalls[api];
}

}  // extern "C"
