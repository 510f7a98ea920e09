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

struct FakeStream {
  std::mutex mu;
  std::condition_variable cv;
  std::deque<std::function<void()>> tasks;
  long submitted = 0;
  long finished = 0;
  bool stop = false;
  std::thread worker;

  FakeStream() {
    worker = std::thread([this] {
      while (true) {
        std::function<void()> fn;
        {
          std::unique_lock<std::mutex> lock(mu);
          cv.wait(lock, [&] { return stop || !tasks.empty(); });
          if (tasks.empty()) return;
          fn = std::move(tasks.front());
          tasks.pop_front();
        }
        fn();
        {
          std::lock_guard<std::mutex> g(mu);
          ++finished;
        }
        cv.notify_all();
      }
    });
  }

  ~FakeStream() {
    {
      std::lock_guard<std::mutex> g(mu);
      stop = true;
    }
    cv.notify_all();
    worker.join();
  }

  void push(std::function<void()> fn) {
    {
      std::lock_guard<std::mutex> g(mu);
      tasks.push_back(std::move(fn));
      ++submitted;
    }
    cv.notify_all();
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

struct FakeEvent {
  std::mutex mu;
  std::shared_ptr<Record> current;  // the latest record, if any
};

namespace {

FakeStream* defaultStream() {
  static FakeStream* s = new FakeStream();  // lives for the process, like the null stream
  return s;
}

FakeStream* resolve(hipStream_t s) { return s ? s : defaultStream(); }

}  // namespace

void fake_hip_enqueue(hipStream_t stream, void (*fn)(void*), void* arg) {
  resolve(stream)->push([fn, arg] { fn(arg); });
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

hipError_t hipStreamCreateWithFlags(hipStream_t* stream, unsigned int) {
  if (enter("hipStreamCreateWithFlags")) return ret(hipErrorUnknown);
  *stream = new FakeStream();
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
  resolve(stream)->push([r] {
    std::unique_lock<std::mutex> lock(r->mu);
    r->cv.wait(lock, [&] { return r->done; });
  });
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
  delete event;  // pending waits hold their own reference to the record
  return hipSuccess;
}

hipError_t hipEventRecord(hipEvent_t event, hipStream_t stream) {
  if (enter("hipEventRecord")) return ret(hipErrorUnknown);
  auto r = std::make_shared<Record>();
  {
    std::lock_guard<std::mutex> g(event->mu);
    event->current = r;
  }
  resolve(stream)->push([r] {
    {
      std::lock_guard<std::mutex> g(r->mu);
      r->done = true;
      r->when = Clock::now();
    }
    r->cv.notify_all();
  });
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

hipError_t hipMalloc(void** ptr, size_t size) {
  if (enter("hipMalloc")) return ret(hipErrorOutOfMemory);
  *ptr = std::malloc(size ? size : 1);
  return *ptr ? hipSuccess : ret(hipErrorOutOfMemory);
}

hipError_t hipFree(void* ptr) {
  enter("hipFree");
  std::free(ptr);
  return hipSuccess;
}

hipError_t hipMemcpyAsync(void* dst, const void* src, size_t bytes, hipMemcpyKind,
                          hipStream_t stream) {
  if (enter("hipMemcpyAsync")) return ret(hipErrorUnknown);
  resolve(stream)->push([dst, src, bytes] { std::memcpy(dst, src, bytes); });
  return hipSuccess;
}

void fake_hip_occupy(hipStream_t stream, int ms) {
  resolve(stream)->push([ms] { std::this_thread::sleep_for(std::chrono::milliseconds(ms)); });
}

void fake_hip_fail_call(const char* api, int nth) {
  std::lock_guard<std::mutex> g(gCallMu);
  gFailAt[api] = gCalls[api] + nth;
}

long fake_hip_calls(const char* api) {
  std::lock_guard<std::mutex> g(gCallMu);
  return gCalls[api];
}

}  // extern "C"
