// adapter_capi.cc -- a small C surface over the adapter classes so that the
// Python tests and the benchmark can drive them (exceptions are turned into a message buffer).
//
// The harness plays the part of Horovod's background thread: the caller's thread queues one
// response after the other with GPUAllreduce::Execute, which returns as soon as the kernels
// are launched; the adapter's finalizer threads wait for each response's events and call
// the entries' callbacks, which the harness counts per response.
#include <chrono>
#include <condition_variable>
#include <cstring>
#include <deque>
#include <mutex>
#include <stdexcept>

#include "hvd_hip_adapter.h"

using namespace horovod::common;

namespace {
double now_s() {
  return std::chrono::duration<double>(std::chrono::steady_clock::now().time_since_epoch()).count();
}

// One queued response as the harness sees it.
struct Op {
  int pending = 0;           // entries whose callback has not run yet
  bool failed = false;
  std::string reason;
  double queued_at = 0;      // Execute was called
  double returned_at = 0;    // Execute returned (kernels launched, completion handed over)
  double completed_at = 0;   // the last entry's callback ran
};

// A response whose entries are kept between calls, so that a benchmark loop pays for the
// launch and not for rebuilding the entry list.
struct Prepared {
  std::vector<TensorTableEntry> entries;
};

struct Harness {
  GPUContext context;
  GlobalState state;
  GPUAllreduce* allreduce = nullptr;
  AdasumGPU* adasum = nullptr;
  std::mutex mu;
  std::condition_variable done;
  std::deque<Op> ops;  // index = ticket; a deque so that queued entries stay where they are
  int completed = 0;
  std::vector<Prepared> prepared;
  bool borrowed_streams = false;  // the streams belong to the caller: not to be destroyed with the context
  std::vector<void*> next_ready_events;  // for the entries of the next response queued
};

// Memory that the caller of this harness allocated (a torch tensor in the tests): nothing to free.
class CallerBuffer : public PersistentBuffer {
public:
  explicit CallerBuffer(void* p) : p_(p) {}
  const void* AccessData() const override { return p_; }

private:
  void* p_;
};

int report(const std::exception& e, char* err, size_t errlen) {
  if (err && errlen) {
    std::strncpy(err, e.what(), errlen - 1);
    err[errlen - 1] = 0;
  }
  return -1;
}

int report(const std::string& reason, char* err, size_t errlen) {
  if (err && errlen) {
    std::strncpy(err, reason.c_str(), errlen - 1);
    err[errlen - 1] = 0;
  }
  return -1;
}

// Queues one response and returns its ticket.
int queue_response(Harness* h, std::vector<TensorTableEntry>& entries, double prescale, double postscale,
                   const void* const* peers, int npeers) {
  int ticket;
  {
    std::lock_guard<std::mutex> guard(h->mu);
    ticket = (int)h->ops.size();
    h->ops.emplace_back();
    h->ops.back().pending = (int)entries.size();
    h->ops.back().queued_at = now_s();
  }
  for (auto& e : entries) {
    e.ready_events = h->next_ready_events;
    e.callback = [h, ticket](const Status& status) {
      // what a framework's callback does with asynchronous completion: its own stream (here the
      // null stream) waits for the event (horovod/torch/mpi_ops_v2.cc:110-116)
      if (status.event.event) hvdhip_stream_wait_event(nullptr, *status.event.event);
      std::lock_guard<std::mutex> guard(h->mu);
      Op& op = h->ops[(size_t)ticket];
      if (!status.ok() && !op.failed) {
        op.failed = true;
        op.reason = status.reason();
      }
      if (--op.pending == 0) {
        op.completed_at = now_s();
        ++h->completed;
        h->done.notify_all();
      }
    };
  }
  h->next_ready_events.clear();
  std::vector<const void*> p(peers, peers + npeers);
  try {
    h->allreduce->Execute(entries, prescale, postscale, p);
  } catch (...) {
    // nothing was handed to a finalizer thread: the response is over, with no callbacks to come
    std::lock_guard<std::mutex> guard(h->mu);
    Op& op = h->ops[(size_t)ticket];
    op.pending = 0;
    op.failed = true;
    op.completed_at = now_s();
    ++h->completed;
    throw;
  }
  std::lock_guard<std::mutex> guard(h->mu);
  h->ops[(size_t)ticket].returned_at = now_s();
  return ticket;
}

int wait_ticket(Harness* h, int ticket, char* err, size_t errlen) {
  std::unique_lock<std::mutex> lock(h->mu);
  if (ticket < 0 || (size_t)ticket >= h->ops.size()) return report(std::string("unknown ticket"), err, errlen);
  h->done.wait(lock, [&] { return h->ops[(size_t)ticket].pending == 0; });
  const Op& op = h->ops[(size_t)ticket];
  return op.failed ? report(op.reason, err, errlen) : 0;
}

void fill_entries(std::vector<TensorTableEntry>& entries, const void* const* tensors, void* const* outputs,
                  const int64_t* counts, int n, int dtype, int buffer_dtype) {
  entries.resize((size_t)n);
  for (int i = 0; i < n; ++i) {
    entries[(size_t)i].tensor_name = "t" + std::to_string(i);
    entries[(size_t)i].tensor_data = tensors[i];
    entries[(size_t)i].output_data = outputs[i];
    entries[(size_t)i].num_elements = counts[i];
    entries[(size_t)i].dtype = (DataType)dtype;
    entries[(size_t)i].buffer_dtype = buffer_dtype;
    entries[(size_t)i].device = 0;
  }
}
}  // namespace

extern "C" {

// finalizer_threads: threads that wait for queued responses (the reference creates one per stream
// slot, common/operations.cc:449); 0 runs every completion on the calling thread.
void* hvd_adapter_create_ex(int num_streams, int batch_d2d_memcopies, int enable_async_completion, int elastic,
                            void* const* fusion_buffers, int finalizer_threads) {
  Harness* h = new Harness();
  h->state.num_nccl_streams = num_streams;
  h->state.batch_d2d_memcopies = batch_d2d_memcopies != 0;
  h->state.enable_async_completion = enable_async_completion != 0;
  h->state.elastic_enabled = elastic != 0;
  for (int i = 0; i < num_streams; ++i) {
    void* p = fusion_buffers[i];
    // the size plays no part when the caller owns the memory; any one value keeps the buffer for good
    h->state.fusion_buffer.InitializeBuffer(64 << 20, 0, [p](int64_t, int) { return std::make_shared<CallerBuffer>(p); }, i,
                                            nullptr, nullptr);
  }
  h->context.streams.resize((size_t)num_streams);
  if (finalizer_threads > 0) h->context.finalizer_thread_pool.create(finalizer_threads);
  h->allreduce = new GPUAllreduce(&h->context, &h->state);
  h->adasum = new AdasumGPU(&h->context);
  return h;
}

void* hvd_adapter_create(int num_streams, int batch_d2d_memcopies, int enable_async_completion, int elastic,
                         void* const* fusion_buffers) {
  return hvd_adapter_create_ex(num_streams, batch_d2d_memcopies, enable_async_completion, elastic, fusion_buffers,
                               num_streams);
}

// Hands the context one existing stream per stream slot (device 0) instead of letting it create its
// own at first use, as gpu_context.streams is filled by whoever gets there first in the reference
// (ops/gpu_operations.cc:30-39).  Streams map onto a few hardware queues in the order they are
// created; a process that wants two slots to overlap creates their streams early and hands them over.
// The streams stay the caller's.
int hvd_adapter_use_streams(void* handle, void* const* streams) {
  Harness* h = static_cast<Harness*>(handle);
  for (int slot = 0; slot < h->state.num_nccl_streams; ++slot) h->context.streams[(size_t)slot][0] = streams[slot];
  h->borrowed_streams = true;
  return 0;
}

void hvd_adapter_destroy(void* handle) {
  Harness* h = static_cast<Harness*>(handle);
  if (!h) return;
  h->context.finalizer_thread_pool.reset();  // the callbacks of queued responses run before the harness goes
  delete h->allreduce;
  delete h->adasum;
  if (h->borrowed_streams) {
    for (auto& per_device : h->context.streams) {
      for (auto& kv : per_device) hvdhip_stream_synchronize(kv.second);
      per_device.clear();
    }
  }
  delete h;  // the context's destructor gives its streams back
}

int hvd_adapter_allreduce_wire(void* handle, const void* const* tensors, void* const* outputs,
                               const int64_t* counts, int n, int dtype, int buffer_dtype, double prescale,
                               double postscale, const void* const* peers, int npeers, char* err, size_t errlen);

int hvd_adapter_allreduce(void* handle, const void* const* tensors, void* const* outputs, const int64_t* counts,
                          int n, int dtype, double prescale, double postscale, const void* const* peers,
                          int npeers, char* err, size_t errlen) {
  return hvd_adapter_allreduce_wire(handle, tensors, outputs, counts, n, dtype, -1, prescale, postscale, peers,
                                    npeers, err, errlen);
}

// Queues one response and returns its ticket (>= 0) as soon as GPUAllreduce::Execute has
// returned, or -1 with the exception's text.  buffer_dtype: the dtype of the fusion buffer and of
// the peers' buffers (-1: that of the tensors).
int hvd_adapter_allreduce_async(void* handle, const void* const* tensors, void* const* outputs,
                                const int64_t* counts, int n, int dtype, int buffer_dtype, double prescale,
                                double postscale, const void* const* peers, int npeers, char* err, size_t errlen) {
  Harness* h = static_cast<Harness*>(handle);
  try {
    std::vector<TensorTableEntry> entries;
    fill_entries(entries, tensors, outputs, counts, n, dtype, buffer_dtype);
    return queue_response(h, entries, prescale, postscale, peers, npeers);
  } catch (const std::exception& e) {
    return report(e, err, errlen);
  }
}

// The same, waiting for the response's callbacks before it returns: 0, or -1 with the text of
// the exception or of the failed Status.
int hvd_adapter_allreduce_wire(void* handle, const void* const* tensors, void* const* outputs,
                               const int64_t* counts, int n, int dtype, int buffer_dtype, double prescale,
                               double postscale, const void* const* peers, int npeers, char* err, size_t errlen) {
  int ticket = hvd_adapter_allreduce_async(handle, tensors, outputs, counts, n, dtype, buffer_dtype, prescale,
                                           postscale, peers, npeers, err, errlen);
  if (ticket < 0) return -1;
  return wait_ticket(static_cast<Harness*>(handle), ticket, err, errlen);
}

// Keeps a response's entry list in the harness; returns its id.
int hvd_adapter_prepare(void* handle, const void* const* tensors, void* const* outputs, const int64_t* counts,
                        int n, int dtype, int buffer_dtype) {
  Harness* h = static_cast<Harness*>(handle);
  h->prepared.emplace_back();
  fill_entries(h->prepared.back().entries, tensors, outputs, counts, n, dtype, buffer_dtype);
  return (int)h->prepared.size() - 1;
}

// Queues a prepared response; returns its ticket or -1.
int hvd_adapter_execute_prepared(void* handle, int id, double prescale, double postscale,
                                 const void* const* peers, int npeers, char* err, size_t errlen) {
  Harness* h = static_cast<Harness*>(handle);
  try {
    if (id < 0 || (size_t)id >= h->prepared.size()) throw std::logic_error("unknown prepared response");
    return queue_response(h, h->prepared[(size_t)id].entries, prescale, postscale, peers, npeers);
  } catch (const std::exception& e) {
    return report(e, err, errlen);
  }
}

// The framework's ready events (hipEvent_t) for every entry of the next response queued: what the
// entries' ReadyEventList would hold.  All entries get the same events, as tensors produced by one
// backward pass do.
int hvd_adapter_next_ready_events(void* handle, void* const* events, int n) {
  Harness* h = static_cast<Harness*>(handle);
  h->next_ready_events.assign(events, events + n);
  return 0;
}

int hvd_adapter_wait(void* handle, int ticket, char* err, size_t errlen) {
  return wait_ticket(static_cast<Harness*>(handle), ticket, err, errlen);
}

// Waits for every response queued so far; -1 with the first failure's text if one failed.
int hvd_adapter_wait_all(void* handle, char* err, size_t errlen) {
  Harness* h = static_cast<Harness*>(handle);
  std::unique_lock<std::mutex> lock(h->mu);
  h->done.wait(lock, [&] { return h->completed == (int)h->ops.size(); });
  for (const Op& op : h->ops)
    if (op.failed) return report(op.reason, err, errlen);
  return 0;
}

// Responses whose callbacks have all run.
int hvd_adapter_completed(void* handle) {
  Harness* h = static_cast<Harness*>(handle);
  std::lock_guard<std::mutex> guard(h->mu);
  return h->completed;
}

// Steady-clock seconds at which Execute was called for the ticket, returned, and the last callback
// ran (0 while that has not happened).
int hvd_adapter_op_times(void* handle, int ticket, double* queued_at, double* returned_at, double* completed_at) {
  Harness* h = static_cast<Harness*>(handle);
  std::lock_guard<std::mutex> guard(h->mu);
  if (ticket < 0 || (size_t)ticket >= h->ops.size()) return -1;
  const Op& op = h->ops[(size_t)ticket];
  *queued_at = op.queued_at;
  *returned_at = op.returned_at;
  *completed_at = op.completed_at;
  return 0;
}

// Forgets the finished responses' bookkeeping (tickets start again at 0); all must have completed.
int hvd_adapter_reset_tickets(void* handle) {
  Harness* h = static_cast<Harness*>(handle);
  std::lock_guard<std::mutex> guard(h->mu);
  if (h->completed != (int)h->ops.size()) return -1;
  h->ops.clear();
  h->completed = 0;
  return 0;
}

// Switches the timeline hooks on or off.
void hvd_adapter_set_timeline(void* handle, int on) {
  static_cast<Harness*>(handle)->state.timeline_initialized = on != 0;
}

// Copies the activity names waited for so far, separated by ',', and clears them.
int hvd_adapter_timeline(void* handle, char* out, size_t outlen) {
  Harness* h = static_cast<Harness*>(handle);
  std::string s;
  std::lock_guard<std::mutex> guard(h->state.timeline_mutex);
  for (auto& a : h->state.timeline_activities) s += (s.empty() ? "" : ",") + a;
  h->state.timeline_activities.clear();
  std::strncpy(out, s.c_str(), outlen - 1);
  out[outlen - 1] = 0;
  return 0;
}

int hvd_adapter_state(void* handle, int* current_stream, int* cached_plans) {
  Harness* h = static_cast<Harness*>(handle);
  *current_stream = h->state.current_nccl_stream;
  *cached_plans = (int)h->allreduce->cached_plans();
  return 0;
}

int hvd_adapter_adasum_pairwise(void* handle, void* a, const void* b, int dtype, const int* counts, int nlayers,
                                double* normdots, char* err, size_t errlen) {
  Harness* h = static_cast<Harness*>(handle);
  try {
    gpuStream_t s = nullptr;
    if (h->context.streams.empty()) h->context.streams.resize(1);
    gpuStream_t& slot = h->context.streams[0][0];
    if (!slot) h->context.StreamCreate(&slot);
    s = slot;
    std::vector<int> tc(counts, counts + nlayers);
    std::vector<double> nd;
    h->adasum->FusedPairwiseReduce(a, b, (DataType)dtype, tc, &nd, s);
    if (normdots) std::memcpy(normdots, nd.data(), nd.size() * sizeof(double));
    h->context.StreamSynchronize(s);
    return 0;
  } catch (const std::exception& e) {
    return report(e, err, errlen);
  }
}

int hvd_adapter_adasum_dispatch(void* handle, void* a, void* b, int dtype, int count, double* out3, double acoeff,
                                double bcoeff, char* err, size_t errlen) {
  Harness* h = static_cast<Harness*>(handle);
  try {
    if (h->context.streams.empty()) h->context.streams.resize(1);
    gpuStream_t& s = h->context.streams[0][0];
    if (!s) h->context.StreamCreate(&s);
    h->adasum->DispatchComputeDotAndNormSqrds(a, b, (DataType)dtype, count, out3[0], out3[1], out3[2], s);
    h->adasum->DispatchScaledAdd((DataType)dtype, count, acoeff, a, bcoeff, b, s);
    h->context.StreamSynchronize(s);
    return 0;
  } catch (const std::exception& e) {
    return report(e, err, errlen);
  }
}

// Simulates the fusion-buffer side of a fused allgather over `global_size` ranks on one
// device: every rank packs its entries (tensors[rank * n + ec], sizes[ec * global_size + rank]
// elements) into the shared buffer at its displacement -- which stands in for the collective --
// and then rank 0's outputs are unpacked.  outputs[ec] must hold the sum over ranks.
int hvd_adapter_allgather(void* handle, const void* const* tensors, void* const* outputs, const int64_t* sizes,
                          int n, int global_size, int dtype, char* err, size_t errlen) {
  Harness* h = static_cast<Harness*>(handle);
  try {
    GPUAllgather op(&h->context, &h->state);
    const int es = (int)DataType_Size((DataType)dtype);
    std::vector<int> recvcounts((size_t)global_size, 0), displ((size_t)global_size, 0);
    std::vector<std::vector<int64_t>> csz((size_t)n, std::vector<int64_t>((size_t)global_size)),
        cof((size_t)n, std::vector<int64_t>((size_t)global_size));
    std::vector<int64_t*> csz_p, cof_p;
    for (int ec = 0; ec < n; ++ec) {
      for (int rc = 0; rc < global_size; ++rc) {
        csz[(size_t)ec][(size_t)rc] = sizes[ec * global_size + rc];
        recvcounts[(size_t)rc] += (int)sizes[ec * global_size + rc];
      }
      csz_p.push_back(csz[(size_t)ec].data());
      cof_p.push_back(cof[(size_t)ec].data());
    }
    int* dp = displ.data();
    GPUAllgather::SetDisplacements(recvcounts.data(), dp, global_size);
    int64_t** cofpp = cof_p.data();
    GPUAllgather::SetEntryComponentOffsets((size_t)n, csz_p.data(), recvcounts.data(), cofpp, global_size);
    if (h->context.streams.empty()) h->context.streams.resize(1);
    gpuStream_t& s = h->context.streams[(size_t)h->state.current_nccl_stream][0];
    if (!s) h->context.StreamCreate(&s);
    void* buffer_data = nullptr;
    std::vector<TensorTableEntry> entries((size_t)n);
    for (int rank = 0; rank < global_size; ++rank) {
      for (int ec = 0; ec < n; ++ec) {
        entries[(size_t)ec].tensor_data = tensors[rank * n + ec];
        entries[(size_t)ec].output_data = outputs[ec];
        entries[(size_t)ec].num_elements = sizes[ec * global_size + rank];
        entries[(size_t)ec].dtype = (DataType)dtype;
      }
      op.MemcpyInFusionBuffer(entries, displ.data(), rank, es, buffer_data);
    }
    op.MemcpyOutFusionBuffer(cof_p.data(), csz_p.data(), buffer_data, es, global_size, entries);
    h->context.StreamSynchronize(s);
    return 0;
  } catch (const std::exception& e) {
    return report(e, err, errlen);
  }
}

int hvd_adapter_fuse(const int64_t* tensor_bytes, int n, int64_t threshold, int batch_d2d_memcopies, int* group_of) {
  std::vector<int64_t> tb(tensor_bytes, tensor_bytes + n);
  auto groups = FuseResponses(tb, threshold, batch_d2d_memcopies != 0);
  for (size_t g = 0; g < groups.size(); ++g)
    for (int i : groups[g]) group_of[i] = (int)g;
  return (int)groups.size();
}

// keys[i]: an opaque class of responses that may fuse with each other.
int hvd_adapter_fuse_keyed(const int64_t* tensor_bytes, const int* keys, int n, int64_t threshold,
                           int batch_d2d_memcopies, int* group_of) {
  std::vector<int64_t> tb(tensor_bytes, tensor_bytes + n);
  std::vector<int> k(keys, keys + n);
  auto groups = FuseResponses(tb, k, threshold, batch_d2d_memcopies != 0);
  for (size_t g = 0; g < groups.size(); ++g)
    for (int i : groups[g]) group_of[i] = (int)g;
  return (int)groups.size();
}

}  // extern "C"
