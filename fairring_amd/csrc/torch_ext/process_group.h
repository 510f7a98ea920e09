// c10d backend "fairring" for PyTorch-ROCm on MI355X: the allreduce entry point
// of the reference's ProcessGroupFairring (fairring/process_group.h:22-189),
// re-targeted at the c10d::Backend / c10d::Work interfaces of current PyTorch
// and driven through the C ABI of include/fairring_hip.h.
//
// One GPU, no transport: the contributions that peers would deliver are handed
// in through setSimulatedPeerContributions() (not part of the reference), and
// an allreduce on a group of size > 1 without them fails loudly.
#pragma once

#include <torch/csrc/distributed/c10d/Backend.hpp>
#include <torch/csrc/distributed/c10d/Store.hpp>
#include <torch/csrc/distributed/c10d/Work.hpp>
#include <torch/torch.h>

#include <atomic>
#include <map>
#include <memory>
#include <mutex>

#include "../../../include/fairring_hip.h"

namespace fairring {

constexpr const char* kPgName = "fairring";

class ProcessGroupFairring : public c10d::Backend {
 public:
  // fairring/process_group.h:24-50, fairring/process_group.cc:35-75
  // What an operation in flight shares between its Work and the pipeline's
  // completion callback.
  struct OpState;

  class WorkFairring : public c10d::Work {
   public:
    // A work that is its future (already completed, or completed by a callback
    // of its own). `group` and `ctx` (optional) let a wait that gives up say
    // where the pipeline stands; the work keeps the group, and so the context,
    // alive.
    WorkFairring(c10d::OpType opType, c10::intrusive_ptr<c10::ivalue::Future> future,
                 c10::intrusive_ptr<c10d::Backend> group = {}, frg_ctx* ctx = nullptr);
    // A work over the pipeline's own handle: wait() orders the caller's stream
    // after the operation through that handle, and the device-aware future
    // (an event created, recorded and waited for per operation) is only made if
    // getFuture() asks for it. Takes over `handle`.
    WorkFairring(c10d::OpType opType, std::shared_ptr<OpState> state, frg_work* handle,
                 c10::intrusive_ptr<c10d::Backend> group, frg_ctx* ctx);
    ~WorkFairring() override;

    bool isCompleted() override;
    bool isSuccess() const override;
    std::exception_ptr exception() const override;
    std::vector<at::Tensor> result() override;
    void synchronize() override;
    bool wait(std::chrono::milliseconds timeout = kNoTimeout) override;
    void abort() override;
    c10::intrusive_ptr<c10::ivalue::Future> getFuture() override;

   private:
    void awaitCompletion();
    void awaitFuture();
    const c10::intrusive_ptr<c10::ivalue::Future> future_;  // null with a handle
    const std::shared_ptr<OpState> state_;
    frg_work* const handle_ = nullptr;
    const c10::intrusive_ptr<c10d::Backend> group_;
    frg_ctx* const ctx_;
  };

  // fairring/process_group.h:52-77, plus the README's slice size
  class OptionsFairring : public c10d::Backend::Options {
   public:
    explicit OptionsFairring(int64_t maxMemoryAllocatedInBytes,
                             int64_t maxPaddingAllocatedInBytes, int64_t minParallelism,
                             bool isHighPriorityStream = false,
                             std::chrono::milliseconds timeout = kBackendDefaultTimeout,
                             int64_t sliceSizeInBytes = 0);
    ~OptionsFairring() override;

    static c10::intrusive_ptr<OptionsFairring> create(
        int64_t maxMemoryAllocatedInBytes, int64_t maxPaddingAllocatedInBytes,
        int64_t minParallelism, bool isHighPriorityStream = false,
        std::chrono::milliseconds timeout = kBackendDefaultTimeout,
        int64_t sliceSizeInBytes = 0);

    const int64_t maxMemoryAllocatedInBytes;
    const int64_t maxPaddingAllocatedInBytes;
    const int64_t minParallelism;
    // Accepted for compatibility; every stream of the pipeline is created at
    // the default priority.
    const bool isHighPriorityStream;
    const int64_t sliceSizeInBytes;
  };

  ProcessGroupFairring(const c10::intrusive_ptr<c10d::Store>& store, int rank, int size,
                       c10::intrusive_ptr<OptionsFairring> options);
  ~ProcessGroupFairring() override;

  const std::string getBackendName() const override;

  // fairring/process_group.cc:131-155
  c10::intrusive_ptr<c10d::Work> allreduce(
      std::vector<at::Tensor>& data,
      const c10d::AllreduceOptions& opts = c10d::AllreduceOptions()) override;

  // fairring/process_group.cc:283-364: the server-side sum with a separate
  // output. One GPU: only this rank's output chunk is produced.
  c10::intrusive_ptr<c10d::Work> reduce_scatter(
      std::vector<at::Tensor>& outputTensors,
      std::vector<std::vector<at::Tensor>>& inputTensors,
      const c10d::ReduceScatterOptions& opts = c10d::ReduceScatterOptions()) override;

  c10::intrusive_ptr<c10d::Work> _reduce_scatter_base(
      at::Tensor& outputBuffer, at::Tensor& inputBuffer,
      const c10d::ReduceScatterOptions& opts = c10d::ReduceScatterOptions()) override;

  // The collectives that move data without reducing it need a transport (the
  // reference runs them on NCCL: fairring/process_group.cc:124-129,173-251,
  // 423-440). Here they exist for a group of one, where nothing moves, so that
  // DistributedDataParallel can be built on the backend as it is; for a larger
  // group they raise.
  c10::intrusive_ptr<c10d::Work> broadcast(
      std::vector<at::Tensor>& data,
      const c10d::BroadcastOptions& opts = c10d::BroadcastOptions()) override;
  c10::intrusive_ptr<c10d::Work> allgather(
      std::vector<std::vector<at::Tensor>>& outputTensors, std::vector<at::Tensor>& inputTensors,
      const c10d::AllgatherOptions& opts = c10d::AllgatherOptions()) override;
  c10::intrusive_ptr<c10d::Work> _allgather_base(
      at::Tensor& outputBuffer, at::Tensor& inputBuffer,
      const c10d::AllgatherOptions& opts = c10d::AllgatherOptions()) override;
  c10::intrusive_ptr<c10d::Work> barrier(
      const c10d::BarrierOptions& opts = c10d::BarrierOptions()) override;

  // Not in the reference. The contributions of the other size-1 ranks, in rank
  // order with this rank left out; GPU tensors on the caller's device or
  // pinned CPU tensors (then they are staged through the pool; refused unless
  // FAIRRING_PINNED_PEERS is set in the environment). For allreduce
  // each has the tensor's size; for the reduce-scatter forms each is either a
  // peer's whole flat input (size * n elements, its chunk for this rank is
  // taken) or just the n elements it would send here. Used by every operation
  // until replaced; an empty list clears them.
  void setSimulatedPeerContributions(std::vector<at::Tensor> peers);

  // Not in the reference. When on, SUM results are divided by the group size
  // inside the reduction (DDP otherwise pre-divides each gradient).
  void setFusedDivide(bool on);

  // Not in the reference: the allreduce with one of torch's DDP communication
  // hooks folded in (torch:distributed/algorithms/ddp_comm_hooks/default_hooks.py).
  //
  // allreducePreDivided: allreduce_hook (:18-54). Every rank's bucket is scaled
  // by 1/size before the sum; here the scaling of all contributions happens
  // inside the reduction and the peers hand in their unscaled buckets.
  c10::intrusive_ptr<c10d::Work> allreducePreDivided(at::Tensor bucket);
  // allreduceCompressed: bf16_compress_hook / fp16_compress_hook (:57-134).
  // `bucket` is this rank's fp32 gradient bucket, the simulated peers hand in
  // their buckets already compressed (tensors of `wire`, scaled by 1/size);
  // this rank's bucket is compressed in registers, the sum is rounded to
  // `wire` once and written back widened into `bucket`.
  // With `grads`, the bucket's own contribution is read from those tensors (in
  // bucket order) instead of from the bucket (frg_allreduce_compressed_gathered).
  c10::intrusive_ptr<c10d::Work> allreduceCompressed(at::Tensor bucket, at::ScalarType wire,
                                                     std::vector<at::Tensor> grads = {});
  // allreduceFromGrads: the allreduce of a bucket together with the copy that
  // fills it. With DDP's default (gradient_as_bucket_view=False) the reducer
  // copies every gradient to its place in the bucket just before the allreduce
  // (torch:csrc/distributed/c10d/reducer.cpp, copy_grad_to_bucket; with no hook
  // registered that copy multiplies by 1/size as well). Here this rank's
  // contribution is read from `grads`, the gradient tensors in the order they
  // lie in `bucket` (dense, their sizes adding up to the bucket's), and the
  // reduced bucket is written once: the bucket is never read. With `preDivide`
  // every contribution is scaled by 1/size before the sum (the peers hand in
  // unscaled buckets), as in allreducePreDivided.
  c10::intrusive_ptr<c10d::Work> allreduceFromGrads(at::Tensor bucket,
                                                    std::vector<at::Tensor> grads,
                                                    bool preDivide);

  // {slot size, slice size, padding slots, staging slots} once initialised.
  std::vector<int64_t> layout();

  // Not in the reference: the measurement hooks of the pipeline behind the
  // group (frg_profile_mark / frg_launch_records / frg_synchronize of the first
  // device's context), so that a benchmark can time the kernel through this
  // surface. A record is (begin ms, end ms, elements, contributions, reduce
  // stream, launches).
  void profileMark();
  std::vector<std::tuple<double, double, int64_t, int, int, int>> launchRecords();
  void synchronizeAll();

 private:
  frg_ctx* contextFor(c10::DeviceIndex device);
  void requireGroupOfOne(const char* what) const;
  c10::intrusive_ptr<c10d::Work> completedWork(c10d::OpType opType,
                                               std::vector<at::Tensor> tensors);
  c10::intrusive_ptr<c10d::Work> reduceCommon(c10d::OpType opType,
                                              const c10d::ReduceOp& reduceOp, at::Tensor own,
                                              at::Tensor out, int64_t chunkOffset,
                                              int64_t peerNumel,
                                              std::vector<at::Tensor> keepAlive,
                                              bool preDivide = false);

  c10::intrusive_ptr<c10d::Store> store_;
  c10::intrusive_ptr<OptionsFairring> options_;
  std::mutex mutex_;
  std::map<c10::DeviceIndex, frg_ctx*> contexts_;  // built lazily (process_group.cc:140-152)
  // The pipeline's reduce streams per device as c10 streams, and its copy
  // streams, which exist from the first host-staged operation on.
  std::map<c10::DeviceIndex, std::vector<c10::Stream>> streams_;
  std::map<c10::DeviceIndex, std::vector<c10::Stream>> copyStreams_;
  const std::vector<c10::Stream>& copyStreamsFor(c10::DeviceIndex device, frg_ctx* ctx);
  static constexpr int kNumReduceStreams = 2;
  static constexpr int kNumCopyStreams = 0;  // the library's default
  void recordOnPipelineStreams(c10::DeviceIndex device, bool copyStreamsToo,
                               std::initializer_list<const at::Tensor*> tensors,
                               const std::vector<at::Tensor>* more);
  std::vector<at::Tensor> peers_;     // flat views, checked when they were set
  bool peersFromHost_ = false;
  bool peersUsed_ = false;             // by an operation since they were set
  // The callers' streams those operations came from: a small operation runs on
  // its caller's stream, so that stream reads the peers' tensors too.
  std::vector<c10::Stream> peersUsedFrom_;
  bool fusedDivide_ = false;
};

}  // namespace fairring
