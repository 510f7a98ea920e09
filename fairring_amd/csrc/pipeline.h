// The per-GPU slice pipeline: streams, events, the fixed staging pool and the
// command thread (the role of DeviceFairring, fairring/device.h:22-117).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <condition_variable>
#include <deque>
#include <functional>
#include <memory>
#include <mutex>
#include <string>
#include <thread>
#include <utility>
#include <vector>

#include "../../include/fairring_hip.h"
#include "layout.h"

namespace frg {

struct QueuedOp;  // a submitted operation on its way to the command thread
constexpr int64_t kMaxMergedBytes = 512ll << 20;
constexpr int kMinMergedOperations = 4;

// Unbounded FIFO drained by one thread: closures, and operations, which the
// thread may look ahead at (it runs neighbouring ones that are already waiting
// as one). An entry with neither is the shutdown token (fairring/utils.h:329-351,
// fairring/device.cc:275-283).
class CommandQueue {
 public:
  struct Command {
    std::function<void()> fn;
    std::shared_ptr<QueuedOp> op;
  };
  void enqueue(std::function<void()> fn);
  void enqueue(std::shared_ptr<QueuedOp> op);
  // Polls for a short while before it sleeps: a sleeping thread takes tens of
  // microseconds to wake, which is most of what a small operation costs.
  Command dequeue();
  // Takes the run of operations at the head of which each continues the one
  // before (`continues(previous, next)`, the first against `first`), at most
  // `atMost` of them, but only if there are at least `atLeast`; never waits.
  std::vector<std::shared_ptr<QueuedOp>> takeRun(
      const QueuedOp& first, const std::function<bool(const QueuedOp&, const QueuedOp&)>& continues,
      int atLeast, int atMost);

 private:
  void push(Command c);
  std::mutex mutex_;
  std::condition_variable cv_;
  std::deque<Command> entries_;
  std::atomic<int64_t> pending_{0};  // entries enqueued and not yet taken
};

// Progress counters of a context, shared with the works it hands out so that a
// wait that gives up can say where things stand (a work may outlive its
// context's handle).
struct Progress {
  std::atomic<int64_t> submitted{0};  // operations accepted by submit()
  std::atomic<int64_t> started{0};    // operations the command thread has begun
  std::atomic<int64_t> enqueued{0};   // operations whose GPU work is all enqueued
  std::atomic<int64_t> launches{0};   // kernel launches issued
  std::atomic<int64_t> onCallersStream{0};  // operations launched by submit() on the producer stream
  std::atomic<int64_t> merged{0};           // operations run together with others that were waiting
  std::atomic<int64_t> segmentedLaunches{0};  // launches that covered pieces of several operations
  // Per reduce stream: how many operations it has been given, and up to which
  // of them the device's null stream already waits (the null stream is never
  // destroyed, so what it was once told to wait for stays waited for: a step's
  // worth of Work.wait() calls on it costs one event per reduce stream, not
  // one per operation).
  static constexpr int kMaxStreams = 8;
  std::atomic<int64_t> streamPosition[kMaxStreams] = {};
  std::mutex nullWaitMu;
  int64_t nullStreamWaitsFor[kMaxStreams] = {};
};

// Completion state of one submitted operation (what the reference keeps in an
// ivalue::Future, fairring/device.cc:303-307,337-348).
struct Work {
  std::mutex mu;
  std::condition_variable cv;
  bool enqueued = false;  // the command thread is done with it
  std::atomic<bool> enqueuedFlag{false};  // the same, for a waiter that polls first
  int status = FRG_OK;
  std::string error;
  // The streams the operation's work ended on. No event is recorded per
  // operation (an event record is a packet on the stream, between two launches
  // that would otherwise run back to back: one per 25 MiB bucket cost a stream
  // of buckets 4 %): waiting is done against the streams themselves, which are
  // in order, so it covers the operation and whatever was enqueued on them up
  // to the moment of the wait. donePositions[i] counts the operations
  // doneStreams[i] had been given when this one was (Progress::streamPosition),
  // for reduce streams; -1 for a caller's stream.
  std::vector<hipStream_t> doneStreams;
  std::vector<int> doneIndices;        // which reduce stream, -1 for a caller's
  std::vector<int64_t> donePositions;
  hipStream_t lastStream = nullptr;
  int device = 0;
  int64_t seq = 0;  // position among the context's operations
  std::shared_ptr<Progress> progress;
  std::atomic<int> refs{1};
};

class Context {
 public:
  static int create(int device, const frg_options& opts, Context** out, std::string* err);
  ~Context();

  const Layout& layout() const { return layout_; }
  int device() const { return device_; }
  const Progress& progress() const { return *progress_; }
  // The reduce streams, then the copy streams that exist so far.
  std::vector<hipStream_t> streams();
  // The copy streams of the host-staged path, created on first use: a context
  // that only reduces resident tensors holds its reduce streams and no more.
  // Throws on a HIP failure.
  std::vector<hipStream_t> copyStreams();

  struct Request {
    void* out = nullptr;
    std::vector<const void*> contribs;
    int64_t numel = 0;
    int dtype = FRG_F32;
    int op = FRG_SUM;
    int scaleMode = FRG_SCALE_NONE;
    float scale = 1.0f;
    bool fromHost = false;
    bool carry = false;  // host-staged only: `out` already holds the first term
    // Compression hooks folded in: `dtype` is the wire type, contribution
    // `rawIndex` is raw fp32, the output is of `outDtype`.
    bool compressed = false;
    int outDtype = FRG_F32;
    int rawIndex = -1;
    // Contribution `gatheredIndex` is not one buffer but these pieces, in the
    // order they lie in the output (a bucket's own gradients, still in the
    // tensors autograd left them in); contribs[gatheredIndex] is ignored.
    struct Segment {
      const void* ptr = nullptr;
      int64_t numel = 0;
    };
    std::vector<Segment> gathered;
    int gatheredIndex = -1;
    hipStream_t producerStream = nullptr;
    frg_done_fn done = nullptr;
    void* user = nullptr;
  };

  // Validates, records the initial event on the producer stream, hands the
  // request to the command thread and returns. `*work` may be null.
  int submit(Request req, Work** work, std::string* err);

  int synchronize(std::string* err);
  void setProfiling(bool perLaunch);
  int profileMark(std::string* err);
  int kernelTimes(float* ms, int capacity, int* count, std::string* err);
  int launchRecords(frg_launch_record* recs, int capacity, int* count, std::string* err);

  static void releaseWork(Work* w);
  // Host blocks until the operation is enqueued and its GPU work is done.
  static int waitWork(Work* w, std::string* err);
  // `stream` waits for the operation; the host only waits for the enqueue.
  static int blockStream(Work* w, hipStream_t stream, std::string* err);
  static bool workEnqueued(Work* w);

 private:
  Context() = default;

  void runGroup(const std::vector<std::shared_ptr<QueuedOp>>& group);
  bool adjoins(const QueuedOp& last, const QueuedOp& next, int64_t bytesSoFar, int* direction);
  // Both return the streams the operation's work ended on, the last one used
  // at the back.
  // `initialEvents`: what the producers recorded (one operation: at most one);
  // `slices` >= 0 overrides the count of slices the operation advances the
  // slot cursor by (several operations run as one keep their own counts).
  std::vector<hipStream_t> runResident(const Request& req,
                                       const std::vector<hipEvent_t>& initialEvents,
                                       int64_t slices);
  std::vector<hipStream_t> runHostStaged(const Request& req, hipEvent_t initialEvent);
  std::vector<hipStream_t> runGathered(const Request& req,
                                       const std::vector<hipEvent_t>& initialEvents);
  void launchSegments(const struct SegmentedArgs& args, hipStream_t stream);
  // Makes `stream` wait for `initialEvent` unless that event has already fired.
  void waitInitial(hipStream_t stream, hipEvent_t initialEvent, bool* fired);
  template <typename Args>
  void launchAndCount(const Args& args, hipStream_t stream,
                      int (*enqueue)(const Args&, hipStream_t, std::string*));
  void launch(const struct ReduceArgs& args, hipStream_t stream);
  void launchCompressed(const struct CompressedArgs& args, hipStream_t stream);
  std::vector<hipStream_t> runGatheredCompressed(const Request& req,
                                                 const std::vector<hipEvent_t>& initialEvents);
  void chainThroughScratch(const Request& req, const std::vector<const void*>& ptrs, int64_t off,
                           int64_t len, size_t streamIdx, bool acc);
  char* scratchFor(size_t streamIdx, const void* like, bool acc, int64_t elsize);
  hipEvent_t takeEvent();
  void giveEvent(hipEvent_t e);
  hipEvent_t freshEvent(hipEvent_t* holder);

  // ---- order between operations ------------------------------------------
  // Operations are dealt to the reduce streams so that neighbours overlap, but
  // a caller sees one pipeline: an operation that touches memory an earlier one
  // on another stream wrote (or writes what that one read) must run after it,
  // as it would on the reference's single chain of streams
  // (fairring/device.cc:291-353). The command thread keeps, per reduce stream,
  // the address ranges of the operations enqueued there that some other stream
  // is not yet ordered after; a new operation is checked against them and its
  // streams wait on the tails of the streams it conflicts with: one event
  // record and wait per conflict, nothing for independent buckets.
  struct Span {
    uintptr_t lo = 0;
    uintptr_t hi = 0;
  };
  struct OpSpans {
    int64_t seq = 0;
    Span write;
    std::vector<Span> reads;
  };
  static OpSpans spansOf(const Request& req);
  static bool conflict(const OpSpans& a, const OpSpans& b);
  // Makes every stream in `targets` wait for what `op` conflicts with on the
  // other reduce streams.
  void orderAfterConflicts(const OpSpans& op, const std::vector<size_t>& targets);
  // Makes `target` wait for everything enqueued on reduce stream `src` so far.
  void joinTail(size_t src, size_t target);
  void remember(OpSpans op, const std::vector<size_t>& targets);
  static constexpr size_t kMaxHistory = 32;  // operations remembered per stream
  std::vector<std::deque<OpSpans>> history_;         // per reduce stream, oldest first
  std::vector<std::vector<int64_t>> orderedAfter_;   // [t][s]: t follows s's history up to this seq
  int64_t spanSeq_ = 0;

  int device_ = 0;
  Layout layout_;
  int64_t numSlots_ = 0;
  int64_t slotBytes_ = 0;
  int64_t maxLaunchBytes_ = 0;   // per contribution and launch; 0 = whole slice
  bool launchBytesByContribs_ = false;  // no size was asked for: it follows the contribution count
  uint64_t allocationBase(const void* p);
  uint64_t allocBase_ = 0;  // the allocation looked up last
  uint64_t allocSize_ = 0;
  // The last partition computed (the buckets of a gradient repeat).
  std::vector<LaunchPart> plan_;
  int64_t planBytes_ = -1;
  uint64_t planOutOffset_ = 0, planFirst_ = 0;
  int planContribs_ = -1;
  bool planAlignShort_ = false;
  // Short operations in a row that were cheap to align (layout.h::planDefaultLaunches).
  static constexpr int kAlignAfterStreak = 4;
  int cheapStreak_ = 0;
  int64_t nextLaunch_ = 0;       // deals launches (or whole operations) to the reduce streams
  // An operation of at most this many launches stays on one reduce stream
  // (with every operation dealing its launches over both, a stream of buckets
  // through the process group ran at 5,372 GB/s against 6,069).
  static constexpr int oneStreamLaunches_ = kOneStreamLaunches;
  // The producer stream that last answered "busy", and how many more of its
  // operations record their event without asking again (any thread may submit).
  static constexpr int kBusyProducerSkips = 15;
  std::atomic<hipStream_t> busyProducer_{nullptr};
  std::atomic<int> busyProducerSkips_{0};
  // Small operations on the caller's stream. With nothing of the pipeline in
  // flight, an operation of one launch that moves at most this many bytes is
  // launched by submit() itself on the producer stream: handing it to the
  // reduce streams costs two cross-stream waits of 6 to 13 us of host time each
  // (producer -> reduce stream, reduce stream -> consumer), several times what
  // the kernel takes. FAIRRING_INLINE_BYTES overrides it (0: never).
  // Operations waiting in the queue whose buffers continue one another's (the
  // buckets of one gradient, handed over faster than they run) are run as one
  // operation over the whole range: at least kMinMergedOperations, at most this
  // many at a time (FAIRRING_MERGE_OPERATIONS; 1: never) and kMaxMergedBytes of
  // output.
  int mergeOperations_ = 16;
  int64_t inlineTrafficBytes_ = 16ll << 20;
  // After a reduce stream answered "busy" the rule is not tried again before this time.
  static constexpr int64_t kInlineRetryNs = 200 * 1000;
  std::atomic<int64_t> inlineRetryAtNs_{0};
  // Operations the command thread has taken up, and the value of that count
  // when the reduce streams were last found idle.
  std::atomic<int64_t> pipelineOps_{0};
  std::atomic<int64_t> idleConfirmedAt_{-1};
  // The last such launch: an event recorded behind it and the stream it went
  // to (kept for comparison only, never used after the call that set it).
  // Whatever is submitted from another stream is ordered after that event.
  std::mutex inlineMu_;
  hipEvent_t inlineEvent_ = nullptr;
  hipStream_t inlineStream_ = nullptr;
  bool inlinePending_ = false;
  bool inlineExplainsBusy_ = false;  // the idle check has not been answered since that launch
  bool inlineRecorded_ = false;  // inlineEvent_ stands behind that launch (else: the null stream, not yet recorded)
  bool tryInline(const Request& req, Work* work);
  void orderAfterInline(hipStream_t producer);

  std::vector<hipStream_t> reduceStreams_;
  // The staging streams of the host-staged path: each owns groups of slots, copies into them
  // and runs the folds that read them; while one folds, the other's copies keep the link busy.
  std::vector<hipStream_t> copyStreams_;
  static constexpr int kDefaultStagingStreams = 1;
  int numCopyStreams_ = kDefaultStagingStreams;
  std::mutex copyMu_;  // guards the creation of copyStreams_

  char* stagingPool_ = nullptr;            // numSlots_ x slotBytes_ of device memory
  // Allocated with the context, one region per reduce stream: carries the partial
  // result of a chain of launches that must not, or not yet, land in `out`
  // (reduced in place into a late contribution; bf16 / fp16 sums, kept in fp32).
  // 8 MiB per stream by default: with 1 MiB a 100-way bf16 sum ran at 2.4 TB/s
  // (launches of a quarter of a million elements), with 8 MiB at 5.8, with 16 MiB
  // the same. FAIRRING_CHAIN_SCRATCH_BYTES overrides it when the context is
  // created (the tests use it to walk the piece loop on small tensors).
  static constexpr int64_t kDefaultCarryScratchBytes = 8 * 1024 * 1024;
  int64_t carryScratchBytes_ = kDefaultCarryScratchBytes;
  char* carryScratch_ = nullptr;
  std::atomic<int64_t> nextStagingSlot_{0};  // round-robin cursor (fairring/device.cc:482)
  int64_t nextSeq_ = 0;          // operation counter for log lines
  std::shared_ptr<Progress> progress_ = std::make_shared<Progress>();


  std::atomic<bool> profiling_{false};  // per-launch dispatch timestamps
  std::mutex profMu_;
  struct ProfRecord {
    hipEvent_t begin;
    hipEvent_t end;
    int64_t numel;
    int numContribs;
    hipStream_t stream;
    int launches;
  };
  std::vector<ProfRecord> profEvents_;
  // marks: one timing event per reduce stream plus the running totals then
  struct Mark {
    std::vector<hipEvent_t> events;
    std::vector<int64_t> launches;
    std::vector<int64_t> elems;
  };
  std::vector<Mark> marks_;
  std::vector<int64_t> streamLaunches_;  // running totals per reduce stream (command thread)
  std::vector<int64_t> streamElems_;
  int lastContribs_ = 0;

  CommandQueue queue_;
  std::thread thread_;
};

// Looks up the static scratch of frg_reduce_slice_static on `device` ahead of
// the first call (static_scratch.hip).
void prepareStaticScratch(int device);

// Process-wide limit of frg_work_wait in seconds (0: none).
void setWaitTimeout(double seconds);

void setLastError(const std::string& msg);
const char* lastError();

// What submit() hands to the command thread.
struct QueuedOp {
  Context::Request req;
  hipEvent_t initial = nullptr;  // recorded on the producer stream, or null if that was idle
  Work* work = nullptr;
};

}  // namespace frg
