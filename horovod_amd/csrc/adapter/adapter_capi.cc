// adapter_capi.cc -- a small C surface over the adapter classes so that the
// Python tests can drive them (exceptions are turned into a message buffer).
#include <cstring>
#include <stdexcept>

#include "hvd_hip_adapter.h"

using namespace horovod::common;

namespace {
struct Harness {
  GPUContext context;
  GlobalState state;
  GPUAllreduce* allreduce = nullptr;
  AdasumGPU* adasum = nullptr;
};

int report(const std::exception& e, char* err, size_t errlen) {
  if (err && errlen) {
    std::strncpy(err, e.what(), errlen - 1);
    err[errlen - 1] = 0;
  }
  return -1;
}
}  // namespace

extern "C" {

void* hvd_adapter_create(int num_streams, int batch_d2d_memcopies, int enable_async_completion, int elastic,
                         void* const* fusion_buffers) {
  Harness* h = new Harness();
  h->state.num_nccl_streams = num_streams;
  h->state.batch_d2d_memcopies = batch_d2d_memcopies != 0;
  h->state.enable_async_completion = enable_async_completion != 0;
  h->state.elastic_enabled = elastic != 0;
  for (int i = 0; i < num_streams; ++i) h->state.fusion_buffer.push_back(fusion_buffers[i]);
  h->allreduce = new GPUAllreduce(&h->context, &h->state);
  h->adasum = new AdasumGPU(&h->context);
  return h;
}

void hvd_adapter_destroy(void* handle) {
  Harness* h = static_cast<Harness*>(handle);
  if (!h) return;
  delete h->allreduce;
  delete h->adasum;
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

// buffer_dtype: the dtype of the fusion buffer and of the peers' buffers (-1: that of the tensors).
int hvd_adapter_allreduce_wire(void* handle, const void* const* tensors, void* const* outputs,
                               const int64_t* counts, int n, int dtype, int buffer_dtype, double prescale,
                               double postscale, const void* const* peers, int npeers, char* err, size_t errlen) {
  Harness* h = static_cast<Harness*>(handle);
  try {
    std::vector<TensorTableEntry> entries((size_t)n);
    for (int i = 0; i < n; ++i) {
      entries[(size_t)i].tensor_name = "t" + std::to_string(i);
      entries[(size_t)i].tensor_data = tensors[i];
      entries[(size_t)i].output_data = outputs[i];
      entries[(size_t)i].num_elements = counts[i];
      entries[(size_t)i].dtype = (DataType)dtype;
      entries[(size_t)i].buffer_dtype = buffer_dtype;
      entries[(size_t)i].device = 0;
    }
    std::vector<const void*> p(peers, peers + npeers);
    h->allreduce->Execute(entries, prescale, postscale, p);
    return 0;
  } catch (const std::exception& e) {
    return report(e, err, errlen);
  }
}

// Switches the timeline hooks on or off.
void hvd_adapter_set_timeline(void* handle, int on) {
  static_cast<Harness*>(handle)->state.timeline_initialized = on != 0;
}

// Copies the activity names waited for so far, separated by ',', and clears them.
int hvd_adapter_timeline(void* handle, char* out, size_t outlen) {
  Harness* h = static_cast<Harness*>(handle);
  std::string s;
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
