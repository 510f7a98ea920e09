// A CPU stand-in for the few HIP runtime calls the slice pipeline makes, so
// that its host logic (slicing, stream/event choreography, slot reuse, error
// paths) can run on a machine without a GPU and under ThreadSanitizer.
// Test infrastructure only: the shipped library is never built against it.
//
// Semantics kept: a stream is an in-order queue; an event record is a point in
// its stream; a stream wait snapshots the event's record at the time of the
// call; "device memory" is host memory. By default every stream is drained by a
// thread of its own. fake_hip_set_hw_queues(n) instead maps the streams (those
// that exist, in the order they were created, and those created afterwards; the
// null stream included) round-robin onto n hardware queues, each
// an in-order queue shared by its streams: a wait packet holds up every stream
// behind it in that queue, as on a GPU whose process has fewer hardware queues
// than streams. The null stream synchronises implicitly with streams created
// without hipStreamNonBlocking, as the legacy default stream does.
#pragma once

#include <stddef.h>
#include <stdint.h>

typedef int hipError_t;
enum {
  hipSuccess = 0,
  hipErrorInvalidValue = 1,
  hipErrorOutOfMemory = 2,
  hipErrorInvalidDevice = 101,
  hipErrorNotReady = 600,
  hipErrorUnknown = 999
};

struct FakeStream;
struct FakeEvent;
typedef FakeStream* hipStream_t;
typedef FakeEvent* hipEvent_t;

enum hipMemcpyKind {
  hipMemcpyHostToHost = 0,
  hipMemcpyHostToDevice = 1,
  hipMemcpyDeviceToHost = 2,
  hipMemcpyDeviceToDevice = 3
};

enum hipDeviceAttribute_t { hipDeviceAttributeMultiprocessorCount = 0 };

#define hipStreamNonBlocking 0x01
#define hipEventDisableTiming 0x02

extern "C" {
hipError_t hipGetDeviceCount(int* count);
hipError_t hipGetDevice(int* device);
hipError_t hipSetDevice(int device);
hipError_t hipDeviceGetAttribute(int* value, hipDeviceAttribute_t attr, int device);
hipError_t hipGetLastError(void);
const char* hipGetErrorString(hipError_t e);

hipError_t hipStreamCreateWithFlags(hipStream_t* stream, unsigned int flags);
hipError_t hipStreamDestroy(hipStream_t stream);
hipError_t hipStreamSynchronize(hipStream_t stream);
hipError_t hipStreamQuery(hipStream_t stream);
typedef enum hipStreamCaptureStatus {
  hipStreamCaptureStatusNone = 0,
  hipStreamCaptureStatusActive = 1,
  hipStreamCaptureStatusInvalidated = 2
} hipStreamCaptureStatus;
hipError_t hipStreamIsCapturing(hipStream_t stream, hipStreamCaptureStatus* status);
hipError_t hipStreamWaitEvent(hipStream_t stream, hipEvent_t event, unsigned int flags);

hipError_t hipEventCreate(hipEvent_t* event);
hipError_t hipEventCreateWithFlags(hipEvent_t* event, unsigned int flags);
hipError_t hipEventDestroy(hipEvent_t event);
hipError_t hipEventRecord(hipEvent_t event, hipStream_t stream);
hipError_t hipEventQuery(hipEvent_t event);
hipError_t hipEventSynchronize(hipEvent_t event);
hipError_t hipEventElapsedTime(float* ms, hipEvent_t start, hipEvent_t stop);

typedef void* hipDeviceptr_t;
hipError_t hipMalloc(void** ptr, size_t size);
// Only memory that came from hipMalloc is known; everything else fails.
hipError_t hipMemGetAddressRange(hipDeviceptr_t* base, size_t* size, hipDeviceptr_t ptr);
hipError_t hipFree(void* ptr);
hipError_t hipMemcpyAsync(void* dst, const void* src, size_t bytes, hipMemcpyKind kind,
                          hipStream_t stream);

// ---- hooks for tests ------------------------------------------------------
// Occupies `stream` (nullptr = the default stream) for `ms` milliseconds.
void fake_hip_occupy(hipStream_t stream, int ms);
// Every stream, existing or yet to be created, shares `n` in-order hardware
// queues (0: a queue per stream, the default). Call it while no work is in flight.
void fake_hip_set_hw_queues(int n);
// A probe of how much the pipeline leans on the binding of a stream wait: with
// 1, a wait on an event that has not fired binds to the record the event holds
// when the wait packet is executed, not to the one it held when
// hipStreamWaitEvent was called (0, the default, and what the HIP runtime
// does). A caller that re-records an event while a wait on it is still pending
// then sees that wait follow the new record. Call it while no work is in flight.
void fake_hip_set_latest_record_waits(int on);
// Makes hipStreamIsCapturing report a capture in progress on every stream (1) or none (0).
void fake_hip_set_capturing(int on);
// Makes the `nth` next call (1 = the very next) of the named API fail once.
void fake_hip_fail_call(const char* api, int nth);
// Calls made so far to the named API.
long fake_hip_calls(const char* api);
}

// C++ only: run `fn(arg)` as one unit of work on a stream (how the test build's
// stand-in for the reduction kernel gets onto the fake streams).
void fake_hip_enqueue(hipStream_t stream, void (*fn)(void*), void* arg);
