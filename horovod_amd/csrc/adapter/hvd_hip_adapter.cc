// hvd_hip_adapter.cc -- see hvd_hip_adapter.h.  Host code; links only libhvdhip.so.
#include "hvd_hip_adapter.h"

#include <algorithm>
#include <chrono>
#include <stdexcept>
#include <thread>
#include <unordered_set>

namespace horovod {
namespace common {

std::size_t DataType_Size(DataType value) {
  int64_t s = hvdhip_dtype_size((int)value);
  if (s < 0) throw std::logic_error("Type " + DataType_Name(value) + " is not supported.");
  return (std::size_t)s;
}

const std::string& DataType_Name(DataType value) {
  static const std::string names[] = {"uint8", "int8", "uint16", "int16", "int32", "int64",
                                      "float16", "float32", "float64", "bool"};
  static const std::string unknown("<unknown>");
  return ((int)value >= 0 && (int)value <= 9) ? names[(int)value] : unknown;
}

// ---------------------------------------------------------------- ThreadPool

ThreadPool::~ThreadPool() { reset(); }

void ThreadPool::create(int num_threads) {
  reset();
  {
    std::lock_guard<std::mutex> guard(mutex_);
    stopping_ = false;
  }
  for (int i = 0; i < num_threads; ++i) threads_.emplace_back([this] { loop(); });
}

void ThreadPool::execute(std::function<void(void)> f) {
  {
    std::lock_guard<std::mutex> guard(mutex_);
    queue_.push_back(std::move(f));
  }
  work_.notify_one();
}

void ThreadPool::loop() {
  std::unique_lock<std::mutex> lock(mutex_);
  for (;;) {
    work_.wait(lock, [this] { return stopping_ || !queue_.empty(); });
    if (queue_.empty()) return;  // stopping, and nothing left to run
    std::function<void(void)> task = std::move(queue_.front());
    queue_.pop_front();
    ++busy_;
    lock.unlock();
    task();
    task = nullptr;  // what the task captured goes before the pool reads as idle
    lock.lock();
    --busy_;
    idle_.notify_all();
  }
}

void ThreadPool::wait_idle() {
  std::unique_lock<std::mutex> lock(mutex_);
  if (threads_.empty()) return;
  idle_.wait(lock, [this] { return queue_.empty() && busy_ == 0; });
}

void ThreadPool::reset() {
  {
    std::lock_guard<std::mutex> guard(mutex_);
    stopping_ = true;
  }
  work_.notify_all();
  for (auto& t : threads_) t.join();
  threads_.clear();
}

// -------------------------------------------------------- FusionBufferManager

Status FusionBufferManager::InitializeBuffer(int64_t threshold, int device, const Allocator& allocate, int stream_id,
                                             std::function<void()> on_start_init, std::function<void()> on_end_init) {
  auto& slot = tensor_fusion_buffers_[std::make_pair(device, stream_id)];
  if (slot.second != threshold) {
    // another threshold: this manager lets go of the buffer; responses in flight still hold it
    slot.first.reset();
    slot.second = 0;
  }
  if (slot.first) return Status::OK();
  if (on_start_init) on_start_init();
  slot.first = allocate(threshold, device);
  if (on_end_init) on_end_init();
  if (!slot.first) return Status::UnknownError("the framework could not allocate the fusion buffer");
  slot.second = threshold;
  return Status::OK();
}

std::shared_ptr<PersistentBuffer> FusionBufferManager::GetBuffer(int device, int stream_id) {
  auto it = tensor_fusion_buffers_.find(std::make_pair(device, stream_id));
  return it == tensor_fusion_buffers_.end() ? nullptr : it->second.first;
}

static void* SlotBuffer(GlobalState* state, int device) {
  auto buffer = state->fusion_buffer.GetBuffer(device, state->current_nccl_stream);
  if (!buffer) throw std::logic_error("no fusion buffer has been initialised for this device and stream slot");
  return const_cast<void*>(buffer->AccessData());
}

// ---------------------------------------------------------------- GPUContext

GPUContext::GPUContext() {}
// The reference keeps its streams for the life of the process; a context that can be created
// and dropped many times (tests, benchmarks) gives them back, after the finalizer threads have
// run what was handed to them.
GPUContext::~GPUContext() {
  finalizer_thread_pool.reset();
  for (auto& per_device : streams)
    for (auto& kv : per_device)
      if (kv.second) hvdhip_stream_destroy(kv.second);
}

void GPUContext::ErrorCheck(std::string op_name, int gpu_result) {
  if (gpu_result != 0) {
    std::string detail = hvdhip_last_error();
    throw std::logic_error(op_name + " failed: " + hvdhip_error_string(gpu_result) +
                           (detail.empty() ? "" : " (" + detail + ")"));
  }
}

static Event AcquireEvent(GPUContext* ctx, gpuStream_t stream) {
  void* ev = nullptr;
  ctx->ErrorCheck("GetGpuEvent", hvdhip_event_acquire(stream, &ev));
  Event event;
  event.event = std::make_shared<void*>(ev);
  event.stream = stream;
  return event;
}

void GPUContext::RecordEvent(std::queue<std::pair<std::string, Event>>& event_queue, std::string name,
                             gpuStream_t& stream) {
  Event event = AcquireEvent(this, stream);
  ErrorCheck("hipEventRecord", hvdhip_event_record(*event.event, event.stream));
  event_queue.emplace(name, event);
}

Event GPUContext::RecordEvent(gpuStream_t& stream) {
  Event event = AcquireEvent(this, stream);
  ErrorCheck("hipEventRecord", hvdhip_event_record(*event.event, event.stream));
  return event;
}

void GPUContext::ReleaseEvent(Event event) {
  ErrorCheck("ReleaseGpuEvent", hvdhip_event_release(event.stream, *event.event));
}

void GPUContext::WaitForEvents(std::queue<std::pair<std::string, Event>>& event_queue,
                               const std::function<void()>& error_check_callback, bool elastic,
                               std::vector<std::string>* timeline_activities) {
  while (!event_queue.empty()) {
    std::string name = event_queue.front().first;
    Event event = event_queue.front().second;
    event_queue.pop();
    if (elastic) {
      // ops/cuda_operations.cc:116-132: poll, checking for asynchronous errors in between
      while (true) {
        int done = 0;
        int rc = hvdhip_event_query(*event.event, &done);
        if (rc != 0) {
          hvdhip_event_release(event.stream, *event.event);  // a failed wait still gives its event back
          throw std::logic_error(std::string("hipEventQuery failed: ") + hvdhip_error_string(rc));
        }
        if (done) break;
        if (error_check_callback) error_check_callback();
        std::this_thread::yield();
      }
    } else {
      int rc = hvdhip_event_synchronize(*event.event);
      if (rc != 0) {
        hvdhip_event_release(event.stream, *event.event);
        throw std::logic_error(std::string("hipEventSynchronize failed: ") + hvdhip_error_string(rc));
      }
      if (error_check_callback) error_check_callback();
    }
    // timeline.ActivityStartAll(entries, name) ... ActivityEndAll(entries) bracket the wait
    if (name != "" && timeline_activities) timeline_activities->push_back(name);  // the caller's own vector
    ErrorCheck("ReleaseGpuEvent", hvdhip_event_release(event.stream, *event.event));
  }
}

void GPUContext::ClearEvents(std::queue<std::pair<std::string, Event>>& event_queue) {
  while (!event_queue.empty()) {
    Event event = event_queue.front().second;
    event_queue.pop();
    ErrorCheck("ReleaseGpuEvent", hvdhip_event_release(event.stream, *event.event));
  }
}

void GPUContext::StreamCreate(gpuStream_t* stream) { ErrorCheck("hipStreamCreate", hvdhip_stream_create(stream)); }
void GPUContext::StreamSynchronize(gpuStream_t stream) {
  ErrorCheck("hipStreamSynchronize", hvdhip_stream_synchronize(stream));
}
int GPUContext::GetDevice() {
  int device = 0;
  ErrorCheck("hipGetDevice", hvdhip_get_device(&device));
  return device;
}
void GPUContext::SetDevice(int device) { ErrorCheck("hipSetDevice", hvdhip_set_device(device)); }
void GPUContext::MemcpyAsyncD2D(void* dst, const void* src, size_t count, gpuStream_t stream) {
  ErrorCheck("hipMemcpyAsync", hvdhip_memcpy_async(dst, src, count, HVDHIP_MEMCPY_D2D, stream));
}
void GPUContext::MemcpyAsyncH2D(void* dst, const void* src, size_t count, gpuStream_t stream) {
  ErrorCheck("hipMemcpyAsync", hvdhip_memcpy_async(dst, src, count, HVDHIP_MEMCPY_H2D, stream));
}
void GPUContext::MemcpyAsyncD2H(void* dst, const void* src, size_t count, gpuStream_t stream) {
  ErrorCheck("hipMemcpyAsync", hvdhip_memcpy_async(dst, src, count, HVDHIP_MEMCPY_D2H, stream));
}
void GPUContext::ScaleBufferImpl(const void* fused_input_data, void* buffer_data, int64_t num_elements,
                                 double scale_factor, DataType dtype, gpuStream_t stream) {
  int rc = hvdhip_scale_buffer(fused_input_data, buffer_data, num_elements, scale_factor, (int)dtype, stream);
  if (rc == HVDHIP_ERR_UNSUPPORTED_DTYPE)  // ops/cuda/cuda_kernels.cu:182-185
    throw std::logic_error("Type " + DataType_Name(dtype) + " not supported by ScaleBufferCudaImpl.");
  ErrorCheck("ScaleBufferImpl", rc);
}

// -------------------------------------------------------------- GPUOpContext

GPUOpContext::GPUOpContext(GPUContext* context, GlobalState* global_state)
    : gpu_context_(context), global_state_(global_state) {}

void GPUOpContext::InitGPU(const std::vector<TensorTableEntry>& entries) {
  auto& first_entry = entries[0];
  gpu_context_->SetDevice(first_entry.device);
  if (gpu_context_->streams.size() < (size_t)global_state_->num_nccl_streams)
    gpu_context_->streams.resize((size_t)global_state_->num_nccl_streams);
  gpuStream_t& s = gpu_context_->streams[(size_t)global_state_->current_nccl_stream][first_entry.device];
  if (s == nullptr) gpu_context_->StreamCreate(&s);
}

void GPUOpContext::InitGPUQueue(const std::vector<TensorTableEntry>& entries) {
  event_queue = std::queue<std::pair<std::string, Event>>();
  stream = &gpu_context_->streams[(size_t)global_state_->current_nccl_stream][entries[0].device];
  if (global_state_->timeline_initialized) gpu_context_->RecordEvent(event_queue, QUEUE, *stream);
  completion_queued_ = false;
}

bool GPUOpContext::RecordsWithLastKernel() const {
  return stream != nullptr && !global_state_->timeline_initialized && !global_state_->enable_async_completion;
}

void* GPUOpContext::QueueCompletionEvent() {
  Event event = AcquireEvent(gpu_context_, *stream);
  event_queue.emplace("", event);
  completion_queued_ = true;
  return *event.event;
}

Status GPUOpContext::FinalizeGPUQueue(std::vector<TensorTableEntry>& entries,
                                      const std::function<void()>& error_check_callback) {
  // A completion marker on the stream instead of a blocking stream synchronisation on this thread.
  if (!global_state_->enable_async_completion && !completion_queued_)
    gpu_context_->RecordEvent(event_queue, "", *stream);

  // Everything the completion needs travels by value: this context is reused by the next response
  // while a finalizer thread still works on this one.
  GPUContext* gpu_context = gpu_context_;
  GlobalState* global_state = global_state_;
  const int device = entries[0].device;
  const bool elastic = global_state_->elastic_enabled;
  const bool async_completion = global_state_->enable_async_completion;
  const bool timeline = global_state_->timeline_initialized;
  gpuStream_t current_stream = *stream;
  auto events = event_queue;
  // a claim on the slot's fusion buffer, so that its memory outlives this response whatever happens
  // to the fusion threshold meanwhile (ops/gpu_operations.cc:64-67); dropped when the task is done
  auto fusion_buffer = global_state_->fusion_buffer.GetBuffer(device, global_state_->current_nccl_stream);
  auto finalize = [gpu_context, global_state, device, elastic, async_completion, timeline, current_stream, events,
                   entries, error_check_callback, fusion_buffer]() mutable {
    Status status = Status::OK();
    try {
      gpu_context->SetDevice(device);  // ops/gpu_operations.cc:75: the thread has no device of its own yet
      if (!async_completion || timeline) {
        // with the timeline on, events are waited for on the host for accurate timings (ops/gpu_operations.cc:77-80)
        std::vector<std::string> activities;
        gpu_context->WaitForEvents(events, error_check_callback, elastic, &activities);
        if (!activities.empty()) {
          std::lock_guard<std::mutex> guard(global_state->timeline_mutex);
          for (auto& a : activities) global_state->timeline_activities.push_back(a);
        }
      } else {
        gpu_context->ClearEvents(events);
        status.event = gpu_context->RecordEvent(current_stream);  // the framework's stream waits for this one
      }
    } catch (const std::exception& e) {
      // an exception must not leave a finalizer thread; the entries learn of it as the reference's
      // background loop reports a failed op (common/operations.cc:291-305)
      Event recorded = status.event;
      status = Status::UnknownError(e.what());
      status.event = recorded;
      try {
        gpu_context->ClearEvents(events);  // the events behind the one that failed go back to the pool
      } catch (const std::exception&) {
      }
    }
    for (auto& e : entries) e.FinishWithCallback(status);
    fusion_buffer.reset();
    if (status.event.event) {
      try {
        gpu_context->ReleaseEvent(status.event);
      } catch (const std::exception&) {
      }
    }
  };
  if (gpu_context_->finalizer_thread_pool.size() > 0)
    gpu_context_->finalizer_thread_pool.execute(std::move(finalize));
  else
    finalize();

  global_state_->current_nccl_stream = (global_state_->current_nccl_stream + 1) % global_state_->num_nccl_streams;
  return Status::InProgress();
}

// -------------------------------------------------------------- GPUAllreduce

GPUAllreduce::GPUAllreduce(GPUContext* context, GlobalState* global_state)
    : gpu_context_(context), global_state_(global_state), gpu_op_context_(context, global_state) {}

GPUAllreduce::~GPUAllreduce() {
  for (auto& kv : plans_) hvdhip_fusion_plan_destroy(kv.second);
}

gpuStream_t GPUAllreduce::Stream(const std::vector<TensorTableEntry>& entries) {
  return gpu_context_->streams[(size_t)global_state_->current_nccl_stream][entries[0].device];
}

hvdhip_fusion_plan* GPUAllreduce::PlanFor(const std::vector<TensorTableEntry>& entries) {
  std::vector<uint64_t> key;
  key.reserve(3 * entries.size() + 1);
  key.push_back((uint64_t)entries[0].dtype | ((uint64_t)entries[0].wire_dtype() << 8));
  for (auto& e : entries) {
    key.push_back((uint64_t)(uintptr_t)e.tensor_data);
    key.push_back((uint64_t)(uintptr_t)e.output_data);
    key.push_back((uint64_t)e.num_elements);
  }
  auto it = plans_.find(key);
  if (it != plans_.end()) {
    plan_order_.remove(key);
    plan_order_.push_front(key);
    return it->second;
  }
  if (plans_.size() >= kMaxPlans) {
    // destroying a plan waits for the device, so no queued kernel can still read its tables
    auto victim = plans_.find(plan_order_.back());
    hvdhip_fusion_plan_destroy(victim->second);
    plans_.erase(victim);
    plan_order_.pop_back();
  }
  std::vector<const void*> tensors;
  std::vector<void*> outputs;
  std::vector<int64_t> counts;
  for (auto& e : entries) {
    tensors.push_back(e.tensor_data);
    outputs.push_back(e.output_data);
    counts.push_back(e.num_elements);
  }
  hvdhip_fusion_plan* plan = nullptr;
  gpu_context_->ErrorCheck("hvdhip_fusion_plan_create",
                           hvdhip_fusion_plan_create(tensors.data(), outputs.data(), counts.data(), (int)entries.size(),
                                                     (int)entries[0].dtype, (int)entries[0].wire_dtype(), &plan));
  plans_[key] = plan;
  plan_order_.push_front(key);
  return plan;
}

void GPUAllreduce::MemcpyInFusionBuffer(const std::vector<TensorTableEntry>& entries,
                                        const void*& fused_input_data, void*& buffer_data, size_t& buffer_len) {
  ScaleMemcpyInFusionBuffer(entries, fused_input_data, buffer_data, buffer_len, 1.0);
}

void GPUAllreduce::ScaleMemcpyInFusionBuffer(const std::vector<TensorTableEntry>& entries,
                                             const void*& fused_input_data, void*& buffer_data,
                                             size_t& buffer_len, double scale_factor) {
  buffer_data = SlotBuffer(global_state_, entries[0].device);  // ops/gpu_operations.cc:122-124
  const bool converting = entries[0].wire_dtype() != entries[0].dtype;
  if (converting && !global_state_->batch_d2d_memcopies)
    throw std::logic_error("A fusion buffer of another dtype than the tensors needs HOROVOD_BATCH_D2D_MEMCOPIES.");
  if (global_state_->batch_d2d_memcopies) {
    hvdhip_fusion_plan* plan = PlanFor(entries);
    // cast, then scale the half: the order (and roundings) of compress() followed by the fp16 ScaleBuffer
    int rc = hvdhip_fusion_pack(plan, buffer_data, scale_factor,
                                converting ? HVDHIP_PACK_CAST_THEN_SCALE : HVDHIP_PACK_DEFAULT, Stream(entries));
    if (rc == HVDHIP_ERR_UNSUPPORTED_DTYPE)  // ops/cuda/cuda_kernels.cu:317-319
      throw std::logic_error("Type " + DataType_Name(entries[0].dtype) +
                             " not supported by BatchedScaledD2DMemcpyCudaImpl.");
    gpu_context_->ErrorCheck("BatchedScaledD2DMemcpyCudaImpl", rc);
    buffer_len = (size_t)hvdhip_fusion_plan_buffer_len(plan);
  } else {
    // ops/gpu_operations.cc:209-222: one async copy per entry at unpadded offsets, then a whole-buffer scale
    int64_t offset = 0;
    for (auto& e : entries) {
      MemcpyEntryInFusionBuffer(entries, e, (uint8_t*)buffer_data + offset);
      offset += e.tensor_size();
    }
    buffer_len = (size_t)offset;
    if (scale_factor != 1.0)
      ScaleBuffer(scale_factor, entries, buffer_data, buffer_data,
                  (int64_t)(buffer_len / DataType_Size(entries[0].dtype)));
  }
  fused_input_data = buffer_data;
}

void GPUAllreduce::MemcpyOutFusionBuffer(const void* buffer_data, std::vector<TensorTableEntry>& entries) {
  ScaleMemcpyOutFusionBuffer(const_cast<void*>(buffer_data), 0, 1.0, entries);
}

void GPUAllreduce::ScaleMemcpyOutFusionBuffer(void* buffer_data, size_t buffer_len, double scale_factor,
                                              std::vector<TensorTableEntry>& entries) {
  if (global_state_->batch_d2d_memcopies) {
    hvdhip_fusion_plan* plan = PlanFor(entries);
    // The unpack is the response's last kernel: it takes the completion event along.
    int rc = gpu_op_context_.RecordsWithLastKernel()
                 ? hvdhip_fusion_unpack_record(plan, buffer_data, scale_factor, Stream(entries),
                                               gpu_op_context_.QueueCompletionEvent())
                 : hvdhip_fusion_unpack(plan, buffer_data, scale_factor, Stream(entries));
    if (rc == HVDHIP_ERR_UNSUPPORTED_DTYPE)
      throw std::logic_error("Type " + DataType_Name(entries[0].dtype) +
                             " not supported by BatchedScaledD2DMemcpyCudaImpl.");
    gpu_context_->ErrorCheck("BatchedScaledD2DMemcpyCudaImpl", rc);
  } else {
    if (scale_factor != 1.0)
      ScaleBuffer(scale_factor, entries, buffer_data, buffer_data,
                  (int64_t)(buffer_len / DataType_Size(entries[0].dtype)));
    int64_t offset = 0;
    for (auto& e : entries) {
      MemcpyEntryOutFusionBuffer(entries, (uint8_t*)buffer_data + offset, e);
      offset += e.tensor_size();
    }
  }
}

void GPUAllreduce::MemcpyEntryInFusionBuffer(const std::vector<TensorTableEntry>& entries,
                                             const TensorTableEntry& e, void* buffer_data_at_offset) {
  gpu_context_->MemcpyAsyncD2D(buffer_data_at_offset, e.tensor_data, (size_t)e.tensor_size(), Stream(entries));
}

void GPUAllreduce::MemcpyEntryOutFusionBuffer(const std::vector<TensorTableEntry>& entries,
                                              const void* buffer_data_at_offset, TensorTableEntry& e) {
  gpu_context_->MemcpyAsyncD2D(e.output_data, buffer_data_at_offset, (size_t)e.tensor_size(), Stream(entries));
}

void GPUAllreduce::ScaleBuffer(double scale_factor, const std::vector<TensorTableEntry>& entries,
                               const void* fused_input_data, void* buffer_data, int64_t num_elements) {
  gpu_context_->ScaleBufferImpl(fused_input_data, buffer_data, num_elements, scale_factor, entries[0].dtype,
                                Stream(entries));
}

void GPUAllreduce::WaitForData(std::vector<TensorTableEntry>& entries) {
  if (global_state_->timeline_initialized) {
    // the normal CPU syncing path: poll until every entry's events have completed
    bool waited = false;
    for (auto& e : entries) {
      for (void* ev : e.ready_events) {
        waited = true;
        for (;;) {
          int done = 0;
          gpu_context_->ErrorCheck("hipEventQuery", hvdhip_event_query(ev, &done));
          if (done) break;
          std::this_thread::sleep_for(std::chrono::nanoseconds(100));
        }
      }
    }
    if (waited) {
      std::lock_guard<std::mutex> guard(global_state_->timeline_mutex);
      global_state_->timeline_activities.push_back(WAIT_FOR_DATA);
    }
    return;
  }
  // entries that were produced together share an event: wait for each one once
  std::unordered_set<void*> event_set;
  for (auto& e : entries)
    for (void* ev : e.ready_events) event_set.insert(ev);
  for (void* ev : event_set)
    gpu_context_->ErrorCheck("hipStreamWaitEvent", hvdhip_stream_wait_event(*gpu_op_context_.stream, ev));
}

Status GPUAllreduce::Execute(std::vector<TensorTableEntry>& entries, double prescale_factor,
                             double postscale_factor, const std::vector<const void*>& peers) {
  gpu_op_context_.InitGPU(entries);
  gpu_op_context_.InitGPUQueue(entries);
  try {
    return Queue(entries, prescale_factor, postscale_factor, peers);
  } catch (...) {
    // the op failed while it was being queued (the caller reports it, common/operations.cc:291-305):
    // the events taken for it so far go back to their pool
    try {
      gpu_context_->ClearEvents(gpu_op_context_.event_queue);
    } catch (const std::exception&) {
    }
    throw;
  }
}

Status GPUAllreduce::Queue(std::vector<TensorTableEntry>& entries, double prescale_factor,
                           double postscale_factor, const std::vector<const void*>& peers) {
  auto& first_entry = entries[0];
  WaitForData(entries);
  const void* fused_input_data;
  void* buffer_data;
  size_t buffer_len;
  const bool timeline = global_state_->timeline_initialized;
  const DataType wire = first_entry.wire_dtype();
  const bool fused = entries.size() > 1 || wire != first_entry.dtype;  // a lone entry still needs the buffer to convert
  if (fused) {
    ScaleMemcpyInFusionBuffer(entries, fused_input_data, buffer_data, buffer_len, prescale_factor);
    if (timeline) gpu_context_->RecordEvent(gpu_op_context_.event_queue, MEMCPY_IN_FUSION_BUFFER, *gpu_op_context_.stream);
  } else {
    // ops/nccl_operations.cc:176-186: no fusion buffer, tensor -> output
    fused_input_data = first_entry.tensor_data;
    buffer_data = first_entry.output_data;
    buffer_len = (size_t)first_entry.tensor_size();
    int64_t num_elements = first_entry.num_elements;
    if (prescale_factor != 1.0) {
      ScaleBuffer(prescale_factor, entries, fused_input_data, buffer_data, num_elements);
      fused_input_data = buffer_data;
    } else if (fused_input_data != buffer_data) {
      gpu_context_->MemcpyAsyncD2D(buffer_data, fused_input_data, buffer_len, Stream(entries));
    }
  }
  // The collective (ncclAllReduce(sum), ops/nccl_operations.cc:190-193) on one GPU.
  if (!peers.empty()) {
    int64_t num_elements = (int64_t)(buffer_len / DataType_Size(wire));
    size_t done = 0;
    while (done < peers.size()) {
      int k = (int)std::min<size_t>(16, peers.size() - done);
      gpu_context_->ErrorCheck("hvdhip_reduce_sum_k",
                               hvdhip_reduce_sum_k(buffer_data, peers.data() + done, k, num_elements, (int)wire,
                                                   Stream(entries)));
      done += (size_t)k;
    }
  }
  if (timeline) gpu_context_->RecordEvent(gpu_op_context_.event_queue, NCCL_ALLREDUCE, *gpu_op_context_.stream);
  if (fused) {
    ScaleMemcpyOutFusionBuffer(buffer_data, buffer_len, postscale_factor, entries);
    if (timeline) gpu_context_->RecordEvent(gpu_op_context_.event_queue, MEMCPY_OUT_FUSION_BUFFER, *gpu_op_context_.stream);
  } else if (postscale_factor != 1.0) {
    ScaleBuffer(postscale_factor, entries, buffer_data, buffer_data, first_entry.num_elements);
  }
  return gpu_op_context_.FinalizeGPUQueue(entries);
}

// --------------------------------------------------------------- GPUAllgather

GPUAllgather::GPUAllgather(GPUContext* context, GlobalState* global_state)
    : gpu_context_(context), global_state_(global_state) {}

void GPUAllgather::SetDisplacements(const int* recvcounts, int*& displcmnts, int global_size) {
  for (int rc = 0; rc < global_size; ++rc)
    displcmnts[rc] = rc == 0 ? 0 : displcmnts[rc - 1] + recvcounts[rc - 1];
}

void GPUAllgather::SetEntryComponentOffsets(size_t num_entries, const int64_t* const* entry_component_sizes,
                                            const int* recvcounts, int64_t**& entry_component_offsets,
                                            int global_size) {
  int64_t rank_displacement = 0;
  for (int rc = 0; rc < global_size; ++rc) {
    for (size_t ec = 0; ec < num_entries; ++ec)
      entry_component_offsets[ec][rc] =
          ec == 0 ? rank_displacement : entry_component_offsets[ec - 1][rc] + entry_component_sizes[ec - 1][rc];
    rank_displacement += recvcounts[rc];
  }
}

void GPUAllgather::MemcpyInFusionBuffer(const std::vector<TensorTableEntry>& entries, const int* displcmnts,
                                        int rank, int element_size, void*& buffer_data) {
  auto& first_entry = entries[0];
  buffer_data = SlotBuffer(global_state_, first_entry.device);
  std::vector<void*> out;
  std::vector<const void*> in;
  std::vector<size_t> sizes;
  int64_t offset = (int64_t)displcmnts[rank] * element_size;
  for (auto& e : entries) {
    out.push_back((uint8_t*)buffer_data + offset);
    in.push_back(e.tensor_data);
    sizes.push_back((size_t)e.tensor_size());
    offset += e.tensor_size();
  }
  gpu_context_->ErrorCheck("hvdhip_batched_d2d_memcpy",
                           hvdhip_batched_d2d_memcpy(out.data(), in.data(), sizes.data(), (int)sizes.size(),
                                                     gpu_context_->streams[(size_t)global_state_->current_nccl_stream][first_entry.device]));
}

void GPUAllgather::MemcpyOutFusionBuffer(const int64_t* const* entry_component_offsets,
                                         const int64_t* const* entry_component_sizes, const void* buffer_data,
                                         int element_size, int global_size,
                                         std::vector<TensorTableEntry>& entries) {
  std::vector<void*> out;
  std::vector<const void*> in;
  std::vector<size_t> sizes;
  for (size_t ec = 0; ec < entries.size(); ++ec) {
    int64_t copy_offset = 0;
    for (int rc = 0; rc < global_size; ++rc) {
      const int64_t entry_offset = entry_component_offsets[ec][rc] * element_size;
      const int64_t entry_size = entry_component_sizes[ec][rc] * element_size;
      out.push_back((uint8_t*)entries[ec].output_data + copy_offset);
      in.push_back((const uint8_t*)buffer_data + entry_offset);
      sizes.push_back((size_t)entry_size);
      copy_offset += entry_size;
    }
  }
  gpu_context_->ErrorCheck("hvdhip_batched_d2d_memcpy",
                           hvdhip_batched_d2d_memcpy(out.data(), in.data(), sizes.data(), (int)sizes.size(),
                                                     gpu_context_->streams[(size_t)global_state_->current_nccl_stream][entries[0].device]));
}

// ------------------------------------------------------------------ AdasumGPU

AdasumGPU::AdasumGPU(GPUContext* context) : gpu_context_(context) {}
AdasumGPU::~AdasumGPU() {
  for (auto& kv : plans_) hvdhip_adasum_plan_destroy(kv.second);
}

static void CheckAdasumType(DataType t, const char* what) {
  // ops/adasum/adasum.h:118-121,136-139
  if (t != HOROVOD_FLOAT16 && t != HOROVOD_FLOAT32 && t != HOROVOD_FLOAT64)
    throw std::logic_error(std::string("Unsupported data type in ") + what + ".");
}

void AdasumGPU::DispatchComputeDotAndNormSqrds(const void* a, const void* b, DataType horovod_datatype,
                                               int count, double& dotProduct, double& anormsq,
                                               double& bnormsq, gpuStream_t stream) {
  CheckAdasumType(horovod_datatype, "ComputeDotAndNormSqrds");
  gpu_context_->ErrorCheck("hvdhip_adasum_dot_and_norm_sqrds",
                           hvdhip_adasum_dot_and_norm_sqrds(a, b, (int)horovod_datatype, count, &dotProduct,
                                                            &anormsq, &bnormsq, stream));
}

void AdasumGPU::DispatchScaledAdd(DataType horovod_datatype, int count, double acoeff, void* a,
                                  double bcoeff, void* b, gpuStream_t stream) {
  CheckAdasumType(horovod_datatype, "ScaledAdd");
  gpu_context_->ErrorCheck("hvdhip_adasum_dispatch_scaled_add",
                           hvdhip_adasum_dispatch_scaled_add((int)horovod_datatype, count, acoeff, a, bcoeff, b,
                                                             stream));
}

void AdasumGPU::FusedPairwiseReduce(void* a, const void* b, DataType horovod_datatype,
                                    const std::vector<int>& tensor_counts, std::vector<double>* normAndDots,
                                    gpuStream_t stream) {
  CheckAdasumType(horovod_datatype, "FusedPairwiseReduce");
  // a plan owns the partial sums of the combine in flight, so streams do not share one
  auto key = std::make_pair(std::make_pair((int)horovod_datatype, (const void*)stream), tensor_counts);
  hvdhip_adasum_plan* plan;
  auto it = plans_.find(key);
  if (it == plans_.end()) {
    if (plans_.size() >= kMaxAdasumPlans) {
      // layer layouts repeat from step to step; a caller that keeps producing new ones starts over
      // (destroying a plan waits for the device, so nothing queued can still use it)
      for (auto& kv : plans_) hvdhip_adasum_plan_destroy(kv.second);
      plans_.clear();
    }
    plan = nullptr;
    gpu_context_->ErrorCheck("hvdhip_adasum_plan_create",
                             hvdhip_adasum_plan_create(tensor_counts.data(), (int)tensor_counts.size(),
                                                       (int)horovod_datatype, &plan));
    plans_[key] = plan;
  } else {
    plan = it->second;
  }
  gpu_context_->ErrorCheck("hvdhip_adasum_combine", hvdhip_adasum_combine(plan, a, b, stream));
  if (normAndDots) {
    normAndDots->resize(3 * tensor_counts.size());
    gpu_context_->ErrorCheck("hvdhip_adasum_read", hvdhip_adasum_read(plan, normAndDots->data(), nullptr, stream));
  }
}

// -------------------------------------------------------------- FuseResponses

std::vector<std::vector<int>> FuseResponses(const std::vector<int64_t>& tensor_bytes,
                                            int64_t fusion_threshold_bytes, bool batch_d2d_memcopies) {
  return FuseResponses(tensor_bytes, std::vector<int>(tensor_bytes.size(), 0), fusion_threshold_bytes,
                       batch_d2d_memcopies);
}

std::vector<std::vector<int>> FuseResponses(const std::vector<int64_t>& tensor_bytes,
                                            const std::vector<int>& keys, int64_t fusion_threshold_bytes,
                                            bool batch_d2d_memcopies) {
  auto padded = [&](int64_t s) { return batch_d2d_memcopies ? 16 * ((s + 15) / 16) : s; };
  const int n = (int)tensor_bytes.size();
  std::vector<int> group_of((size_t)n, -1);
  std::vector<std::vector<int>> groups;
  for (int head = 0; head < n; ++head) {
    if (group_of[(size_t)head] != -1) continue;
    const int g = (int)groups.size();
    groups.push_back({head});
    group_of[(size_t)head] = g;
    int64_t tensor_size = padded(tensor_bytes[(size_t)head]);
    int64_t skipped_size = 0;
    for (int j = head + 1; j < n; ++j) {
      if (group_of[(size_t)j] != -1) continue;
      const int64_t new_tensor_size = padded(tensor_bytes[(size_t)j]);
      if (keys[(size_t)j] == keys[(size_t)head] && tensor_size + new_tensor_size <= fusion_threshold_bytes) {
        tensor_size += new_tensor_size;
        group_of[(size_t)j] = g;
        groups[(size_t)g].push_back(j);
      } else {
        // look ahead past a response that does not fit or does not match, while the batch
        // plus everything skipped still fits (common/controller.cc:839-856)
        skipped_size += new_tensor_size;
        if (tensor_size + skipped_size > fusion_threshold_bytes) break;
      }
    }
  }
  return groups;
}

}  // namespace common
}  // namespace horovod
