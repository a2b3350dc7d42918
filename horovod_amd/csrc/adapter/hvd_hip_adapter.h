// hvd_hip_adapter.h -- the host side above the C ABI: C++ classes shaped like
// the reference's op layer for this path, calling nothing but include/hvdhip.h.
//
// These are the bodies a Horovod maintainer would put behind the existing
// declarations (names, argument meaning and error behaviour are the
// reference's):
//   GPUContext          ops/gpu_operations.h:44-106, impl ops/cuda_operations.cc:28-210
//   GPUOpContext        ops/gpu_operations.h:108-137, ops/gpu_operations.cc:27-106
//   ThreadPool          common/thread_pool.h:27-43 (the finalizer threads, one per stream slot,
//                       common/operations.cc:449)
//   Status              common/common.h:192-212
//   FusionBufferManager common/fusion_buffer_manager.{h,cc}; PersistentBuffer common/common.h:321-325
//   GPUAllreduce hooks  ops/gpu_operations.h:139-172, ops/gpu_operations.cc:118-339
//   Adasum dispatch     ops/adasum/adasum.h:101-140,344-410
//   FuseResponses       common/controller.cc:793-866
// Errors become std::logic_error("<op> failed: <text>") exactly as
// GPUContext::ErrorCheck does (ops/cuda_operations.cc:82-86).
//
// The reference's own headers cannot be included here (they pull in Eigen,
// Boost and FlatBuffers), so the few types the hooks touch are restated in
// minimal form: DataType, TensorTableEntry (tensor/output pointer, size,
// dtype, device), Event.
#ifndef HVD_HIP_ADAPTER_H
#define HVD_HIP_ADAPTER_H

#include <condition_variable>
#include <cstddef>
#include <cstdint>
#include <deque>
#include <functional>
#include <list>
#include <map>
#include <memory>
#include <mutex>
#include <queue>
#include <string>
#include <thread>
#include <unordered_map>
#include <utility>
#include <vector>

#include "hvdhip.h"

namespace horovod {
namespace common {

// common/message.h:30-41
enum DataType {
  HOROVOD_UINT8 = 0, HOROVOD_INT8 = 1, HOROVOD_UINT16 = 2, HOROVOD_INT16 = 3, HOROVOD_INT32 = 4,
  HOROVOD_INT64 = 5, HOROVOD_FLOAT16 = 6, HOROVOD_FLOAT32 = 7, HOROVOD_FLOAT64 = 8, HOROVOD_BOOL = 9
};
std::size_t DataType_Size(DataType value);            // common/message.cc:66-92
const std::string& DataType_Name(DataType value);     // common/message.cc:40-64

typedef void* gpuStream_t;
#define CPU_DEVICE_ID (-1)  // common/common.h:150

// Activity names of the stages on this path, common/common.h:73-105.
#define WAIT_FOR_DATA "WAIT_FOR_DATA"
#define QUEUE "QUEUE"
#define MEMCPY_IN_FUSION_BUFFER "MEMCPY_IN_FUSION_BUFFER"
#define MEMCPY_OUT_FUSION_BUFFER "MEMCPY_OUT_FUSION_BUFFER"
#define NCCL_ALLREDUCE "NCCL_ALLREDUCE"

// common/common.h:181-189
struct Event {
  std::shared_ptr<void*> event;
  gpuStream_t stream = nullptr;
};

// common/common.h:157,192-212
enum StatusType { OK, UNKNOWN_ERROR, PRECONDITION_ERROR, ABORTED, INVALID_ARGUMENT, IN_PROGRESS };
class Status {
public:
  Status() {}
  static Status OK() { return Status(); }
  static Status UnknownError(const std::string& message) { return Status(UNKNOWN_ERROR, message); }
  static Status InProgress() { return Status(IN_PROGRESS, ""); }
  bool ok() const { return type_ == StatusType::OK; }
  bool in_progress() const { return type_ == IN_PROGRESS; }
  StatusType type() const { return type_; }
  const std::string& reason() const { return reason_; }
  // With asynchronous completion: recorded behind the response on its stream; the framework's
  // callback makes its own stream wait for it (horovod/torch/mpi_ops_v2.cc:110-116).
  Event event;

private:
  Status(StatusType type, std::string reason) : type_(type), reason_(std::move(reason)) {}
  StatusType type_ = StatusType::OK;
  std::string reason_;
};
typedef std::function<void(const Status&)> StatusCallback;

// The part of TensorTableEntry (common/common.h:341-374) that the hooks read:
// tensor->data()/size()/dtype(), output->data(), device, callback.
struct TensorTableEntry {
  std::string tensor_name;
  const void* tensor_data = nullptr;
  void* output_data = nullptr;
  int64_t num_elements = 0;
  DataType dtype = HOROVOD_FLOAT32;
  int device = 0;
  int64_t tensor_size() const { return num_elements * (int64_t)DataType_Size(dtype); }
  // Not in the reference: the dtype the entry travels in.  HOROVOD_FLOAT16 with FLOAT32 tensors
  // folds Compression.fp16 (horovod/torch/compression.py:46-64) into packing and unpacking;
  // left at its default the entry travels as it is.
  int buffer_dtype = -1;
  DataType wire_dtype() const { return buffer_dtype < 0 ? dtype : (DataType)buffer_dtype; }
  // ReadyEventList (common/common.h:262-300): events the framework recorded behind whatever produces
  // the tensor; empty when the data is ready at enqueue time.
  std::vector<void*> ready_events;
  // Called from a finalizer thread once the response has completed (or, with asynchronous
  // completion, once its last work has been queued); may be empty (common/common.cc:202-208).
  StatusCallback callback;
  void FinishWithCallback(const Status& status) const {
    if (callback) callback(status);
  }
};

// The finalizer threads: the background thread hands the wait for a response's events to one of
// them and goes on to launch the next response on the next stream slot.  Same surface as the
// reference's pool (create / execute / reset), plus wait_idle() so that a harness can tell when
// everything handed over has run.  reset() runs what is still queued before the threads end, so a
// response whose wait was queued always gets its callbacks.
class ThreadPool {
public:
  ThreadPool() {}
  ~ThreadPool();
  ThreadPool(const ThreadPool&) = delete;
  ThreadPool& operator=(const ThreadPool&) = delete;
  void create(int num_threads);
  void execute(std::function<void(void)> f);
  void reset();
  void wait_idle();
  int size() const { return (int)threads_.size(); }

private:
  void loop();
  std::mutex mutex_;
  std::condition_variable work_;   // a task was queued, or the pool is stopping
  std::condition_variable idle_;   // a task finished
  std::deque<std::function<void(void)>> queue_;
  std::vector<std::thread> threads_;
  int busy_ = 0;
  bool stopping_ = false;
};

// common/common.h:321-325: memory that the framework allocated and keeps alive while anybody holds it.
class PersistentBuffer {
public:
  virtual const void* AccessData() const = 0;
  virtual ~PersistentBuffer() = default;
};

// One fusion buffer per (device, stream slot), allocated through the framework at first use and again
// when the fusion threshold has changed (common/fusion_buffer_manager.cc:21-50).  The reference keys
// the buffers by framework as well; one process of this adapter serves one framework.  Handing out
// shared ownership is the point: a response in flight keeps the buffer it was packed into alive until
// its finalizer has run, whatever the threshold does meanwhile (ops/gpu_operations.cc:64-67).
class FusionBufferManager {
public:
  // Stands for OpContext::AllocatePersistent (common/common.h:327-339) of the entry's framework.
  typedef std::function<std::shared_ptr<PersistentBuffer>(int64_t size, int device)> Allocator;
  Status InitializeBuffer(int64_t threshold, int device, const Allocator& allocate, int stream_id,
                          std::function<void()> on_start_init, std::function<void()> on_end_init);
  // The buffer of (device, stream slot), or null.
  std::shared_ptr<PersistentBuffer> GetBuffer(int device, int stream_id);

private:
  std::map<std::pair<int, int>, std::pair<std::shared_ptr<PersistentBuffer>, int64_t>> tensor_fusion_buffers_;
};

class GPUContext {
public:
  GPUContext();
  ~GPUContext();

  // One stream per (stream slot, device), created lazily (ops/gpu_operations.cc:30-39).
  std::vector<std::unordered_map<int, gpuStream_t>> streams;
  // Completion of queued responses (ops/gpu_operations.h:65); created with one thread per stream
  // slot by whoever owns the context (common/operations.cc:449).  Left without threads,
  // FinalizeGPUQueue runs the completion on the calling thread.
  ThreadPool finalizer_thread_pool;

  void ErrorCheck(std::string op_name, int gpu_result);
  void RecordEvent(std::queue<std::pair<std::string, Event>>& event_queue, std::string name, gpuStream_t& stream);
  Event RecordEvent(gpuStream_t& stream);
  void ReleaseEvent(Event event);
  // Synchronises every queued event (or polls it when elastic is set, calling
  // error_check_callback between polls), then recycles it.
  void WaitForEvents(std::queue<std::pair<std::string, Event>>& event_queue,
                     const std::function<void()>& error_check_callback = nullptr, bool elastic = false,
                     std::vector<std::string>* timeline_activities = nullptr);
  void ClearEvents(std::queue<std::pair<std::string, Event>>& event_queue);
  void StreamCreate(gpuStream_t* stream);
  void StreamSynchronize(gpuStream_t stream);
  int GetDevice();
  void SetDevice(int device);
  void MemcpyAsyncD2D(void* dst, const void* src, size_t count, gpuStream_t stream);
  void MemcpyAsyncH2D(void* dst, const void* src, size_t count, gpuStream_t stream);
  void MemcpyAsyncD2H(void* dst, const void* src, size_t count, gpuStream_t stream);
  void ScaleBufferImpl(const void* fused_input_data, void* buffer_data, int64_t num_elements,
                       double scale_factor, DataType dtype, gpuStream_t stream);
};

// The slice of HorovodGlobalState the hooks read (common/global_state.h).
struct GlobalState {
  int current_nccl_stream = 0;
  int num_nccl_streams = 1;
  bool batch_d2d_memcopies = true;
  bool enable_async_completion = false;
  bool elastic_enabled = false;
  // Timeline::Initialized(): when set, the ops enqueue a named event after every stage
  // (ops/nccl_operations.cc:173-175,195-197,203-205) and the completed activity names are
  // appended to timeline_activities as the events are waited for.
  bool timeline_initialized = false;
  std::vector<std::string> timeline_activities;  // appended to by finalizer threads, under timeline_mutex
  std::mutex timeline_mutex;
  // One fusion buffer per (device, stream slot); the memory is the framework's.
  FusionBufferManager fusion_buffer;
};

class GPUOpContext {
public:
  GPUOpContext(GPUContext* context, GlobalState* global_state);
  void InitGPU(const std::vector<TensorTableEntry>& entries);
  void InitGPUQueue(const std::vector<TensorTableEntry>& entries);
  // Records the completion event, hands the wait for the queued events and the entries'
  // callbacks to a finalizer thread (ops/gpu_operations.cc:50-99), rotates the stream slot and
  // returns Status::InProgress() at once, so that the caller can launch the next response on
  // the next slot while this one runs.
  Status FinalizeGPUQueue(std::vector<TensorTableEntry>& entries,
                          const std::function<void()>& error_check_callback = nullptr);
  std::queue<std::pair<std::string, Event>> event_queue;
  gpuStream_t* stream = nullptr;
  // Whether the response's last kernel should carry the completion event itself
  // (hvdhip_fusion_unpack_record) instead of FinalizeGPUQueue recording one behind it: only when
  // that event is the one thing FinalizeGPUQueue would record (no timeline, no asynchronous completion).
  bool RecordsWithLastKernel() const;
  // Takes an event from the pool, unrecorded, and queues it as the completion event ("" as in
  // ops/gpu_operations.cc:82); the caller hands it to the launch that records it.
  void* QueueCompletionEvent();

private:
  bool completion_queued_ = false;
  GPUContext* gpu_context_;
  GlobalState* global_state_;
};

class GPUAllreduce {
public:
  GPUAllreduce(GPUContext* context, GlobalState* global_state);
  ~GPUAllreduce();

  // ops/gpu_operations.cc:110-115: this op takes the response when its tensors live on a GPU.
  bool Enabled(const std::vector<TensorTableEntry>& entries) const { return entries[0].device != CPU_DEVICE_ID; }

  // The op sequence of NCCLAllreduce::Execute (ops/nccl_operations.cc:156-214) with the
  // collective replaced by a local sum with `peers` (device buffers laid out like the
  // fusion buffer, or like the single tensor).  Returns Status::InProgress() as soon as the
  // response is queued; every entry's callback is called once it has completed.
  Status Execute(std::vector<TensorTableEntry>& entries, double prescale_factor, double postscale_factor,
                 const std::vector<const void*>& peers);

  // NCCLAllreduce::WaitForData (ops/nccl_operations.cc:140-154): the op's stream waits for the
  // entries' ready events, each once, with no host synchronisation; with the timeline on, the host
  // polls them instead (HorovodOp::WaitForData, ops/collective_operations.cc:35-62).
  void WaitForData(std::vector<TensorTableEntry>& entries);

  void MemcpyInFusionBuffer(const std::vector<TensorTableEntry>& entries, const void*& fused_input_data,
                            void*& buffer_data, size_t& buffer_len);
  void MemcpyOutFusionBuffer(const void* buffer_data, std::vector<TensorTableEntry>& entries);
  void ScaleMemcpyInFusionBuffer(const std::vector<TensorTableEntry>& entries, const void*& fused_input_data,
                                 void*& buffer_data, size_t& buffer_len, double scale_factor);
  void ScaleMemcpyOutFusionBuffer(void* buffer_data, size_t buffer_len, double scale_factor,
                                  std::vector<TensorTableEntry>& entries);
  void MemcpyEntryInFusionBuffer(const std::vector<TensorTableEntry>& entries, const TensorTableEntry& e,
                                 void* buffer_data_at_offset);
  void MemcpyEntryOutFusionBuffer(const std::vector<TensorTableEntry>& entries,
                                  const void* buffer_data_at_offset, TensorTableEntry& e);
  void ScaleBuffer(double scale_factor, const std::vector<TensorTableEntry>& entries,
                   const void* fused_input_data, void* buffer_data, int64_t num_elements);

  size_t cached_plans() const { return plans_.size(); }

private:
  // Execute after InitGPU / InitGPUQueue: everything from WaitForData to FinalizeGPUQueue.
  Status Queue(std::vector<TensorTableEntry>& entries, double prescale_factor, double postscale_factor,
               const std::vector<const void*>& peers);
  // Fused tensor sets repeat every step (the reference caches responses,
  // common/response_cache.cc:126-235): one resident plan per distinct entry list.
  hvdhip_fusion_plan* PlanFor(const std::vector<TensorTableEntry>& entries);
  gpuStream_t Stream(const std::vector<TensorTableEntry>& entries);

  GPUContext* gpu_context_;
  GlobalState* global_state_;
  GPUOpContext gpu_op_context_;
  // At most kMaxPlans resident plans, least recently used first out, so that a framework
  // that hands over fresh tensor addresses every step cannot grow the cache without bound.
  static constexpr size_t kMaxPlans = 128;
  std::map<std::vector<uint64_t>, hvdhip_fusion_plan*> plans_;
  std::list<std::vector<uint64_t>> plan_order_;  // front = most recently used
};

// The fusion-buffer hooks of the allgather op (ops/collective_operations.cc:200-275,
// GPU overrides ops/gpu_operations.cc:350-363).  The reference issues one async copy per
// entry (pack) and per (entry, rank) component (unpack); here each direction is one
// batched launch.  The collective itself (every rank's slab arriving in the buffer) is
// outside this class.
class GPUAllgather {
public:
  GPUAllgather(GPUContext* context, GlobalState* global_state);
  // AllgatherOp::SetDisplacements
  static void SetDisplacements(const int* recvcounts, int*& displcmnts, int global_size);
  // AllgatherOp::SetEntryComponentOffsets; the matrices are [entry][rank]
  static void SetEntryComponentOffsets(size_t num_entries, const int64_t* const* entry_component_sizes,
                                       const int* recvcounts, int64_t**& entry_component_offsets,
                                       int global_size);
  void MemcpyInFusionBuffer(const std::vector<TensorTableEntry>& entries, const int* displcmnts, int rank,
                            int element_size, void*& buffer_data);
  void MemcpyOutFusionBuffer(const int64_t* const* entry_component_offsets,
                             const int64_t* const* entry_component_sizes, const void* buffer_data,
                             int element_size, int global_size, std::vector<TensorTableEntry>& entries);

private:
  GPUContext* gpu_context_;
  GlobalState* global_state_;
};

// Adasum<Comm>'s dispatch hooks and pairwise reduce, run on the device instead of the
// host (the reference copies the shard to host first, ops/adasum_gpu_operations.cc:200-211).
class AdasumGPU {
public:
  explicit AdasumGPU(GPUContext* context);
  ~AdasumGPU();
  void DispatchComputeDotAndNormSqrds(const void* a, const void* b, DataType horovod_datatype, int count,
                                      double& dotProduct, double& anormsq, double& bnormsq,
                                      gpuStream_t stream);
  void DispatchScaledAdd(DataType horovod_datatype, int count, double acoeff, void* a, double bcoeff,
                         void* b, gpuStream_t stream);
  // FusedPairwiseReduceWithComm (ops/adasum/adasum.h:344-410) for one process: per-layer
  // triples, coefficients and scaled add without leaving the device.  normAndDots, if not
  // null, receives 3 doubles per layer.
  void FusedPairwiseReduce(void* a, const void* b, DataType horovod_datatype,
                           const std::vector<int>& tensor_counts, std::vector<double>* normAndDots,
                           gpuStream_t stream);

private:
  GPUContext* gpu_context_;
  static constexpr size_t kMaxAdasumPlans = 128;
  std::map<std::pair<std::pair<int, const void*>, std::vector<int>>, hvdhip_adasum_plan*> plans_;  // (dtype, stream), counts
};

// Controller::FuseResponses (common/controller.cc:793-866) for allreduce responses of one
// dtype and one pair of scale factors: returns groups of entry indices.
std::vector<std::vector<int>> FuseResponses(const std::vector<int64_t>& tensor_bytes,
                                            int64_t fusion_threshold_bytes, bool batch_d2d_memcopies);
// The same with mixed responses: keys[i] stands for everything that has to be equal for two
// responses to fuse (response type, devices, dtype, prescale and postscale factor,
// common/controller.cc:831-836); responses with different keys never share a group.
std::vector<std::vector<int>> FuseResponses(const std::vector<int64_t>& tensor_bytes,
                                            const std::vector<int>& keys, int64_t fusion_threshold_bytes,
                                            bool batch_d2d_memcopies);

}  // namespace common
}  // namespace horovod

#endif  // HVD_HIP_ADAPTER_H
