// fake_hvdhip.cc -- a host-only stand-in for libhvdhip.so, for testing the C++ adapter's HOST logic
// (finalizer threads, stream slots, event pooling, callbacks) on a machine without a GPU and under
// ThreadSanitizer.  It is test infrastructure: nothing in the product links or loads it.
//
// A "stream" is a worker thread that runs queued closures in order; a "kernel" is a closure that
// does the arithmetic on host memory (float32 only: one IEEE multiply per scaled element, one add
// per peer) after an optional delay that makes the pretend device slow; an "event" completes when
// the marker queued by its record has run.  Only what the adapter's allreduce path calls is
// modelled; the Adasum and allgather entry points exist so that the adapter links, and refuse.
#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstring>
#include <deque>
#include <functional>
#include <map>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#include "hvdhip.h"

namespace {

struct FakeEvent {
  std::mutex mu;
  std::condition_variable cv;
  uint64_t recorded = 0;   // generation of the latest record
  uint64_t completed = 0;  // latest generation whose marker has run
};

struct FakeStream {
  std::mutex mu;
  std::condition_variable cv;
  std::deque<std::function<void()>> queue;
  bool busy = false;
  bool stop = false;
  std::thread worker;
  FakeStream() : worker([this] { run(); }) {}
  ~FakeStream() {
    {
      std::lock_guard<std::mutex> g(mu);
      stop = true;
    }
    cv.notify_all();
    worker.join();
  }
  void push(std::function<void()> f) {
    {
      std::lock_guard<std::mutex> g(mu);
      queue.push_back(std::move(f));
    }
    cv.notify_all();
  }
  void run() {
    std::unique_lock<std::mutex> lock(mu);
    for (;;) {
      cv.wait(lock, [this] { return stop || !queue.empty(); });
      if (queue.empty()) return;
      std::function<void()> f = std::move(queue.front());
      queue.pop_front();
      busy = true;
      lock.unlock();
      f();
      f = nullptr;
      lock.lock();
      busy = false;
      cv.notify_all();
    }
  }
  void drain() {
    std::unique_lock<std::mutex> lock(mu);
    cv.wait(lock, [this] { return queue.empty() && !busy; });
  }
};

thread_local std::string t_error;
thread_local int t_device = -1;  // -1: this thread has not selected a device
std::atomic<int> g_kernel_delay_us{0};
std::atomic<int> g_fail_event_syncs{0};
std::atomic<int> g_launches{0};
std::mutex g_devices_mu;
std::map<std::thread::id, int> g_set_device_calls;  // per thread

int fail(int code, const char* what) {
  t_error = what;
  return code;
}

void kernel_delay() {
  int us = g_kernel_delay_us.load();
  if (us > 0) std::this_thread::sleep_for(std::chrono::microseconds(us));
}

FakeStream* S(void* s) { return static_cast<FakeStream*>(s); }
FakeEvent* E(void* e) { return static_cast<FakeEvent*>(e); }

std::mutex g_streams_mu;
std::vector<FakeStream*> g_streams;  // every live stream: the pretend device

// hipDeviceSynchronize: everything queued on any stream has run.
void device_synchronize() {
  std::vector<FakeStream*> all;
  {
    std::lock_guard<std::mutex> g(g_streams_mu);
    all = g_streams;
  }
  for (FakeStream* s : all) s->drain();
}

std::mutex g_pool_mu;
std::map<void*, std::vector<FakeEvent*>> g_pool;  // by stream
std::atomic<int> g_events_out{0};                 // acquired and not yet released

}  // namespace

struct hvdhip_fusion_plan {
  std::vector<const float*> tensors;
  std::vector<float*> outputs;
  std::vector<int64_t> counts;
  std::vector<int64_t> offsets;
  int64_t buffer_len = 0;
};
struct hvdhip_adasum_plan {};

extern "C" {

// ---- controls of the pretend device (not part of hvdhip.h)
void fake_set_kernel_delay_us(int us) { g_kernel_delay_us = us; }
void fake_fail_next_event_syncs(int n) { g_fail_event_syncs = n; }
int fake_launches() { return g_launches.load(); }
int fake_events_outstanding() { return g_events_out.load(); }
int fake_set_device_calls_on_other_threads(void) {
  std::lock_guard<std::mutex> g(g_devices_mu);
  int n = 0;
  for (auto& kv : g_set_device_calls)
    if (kv.first != std::this_thread::get_id()) n += kv.second;
  return n;
}

const char* hvdhip_error_string(int code) { return code == 0 ? "success" : code > 0 ? "pretend device error" : "invalid"; }
const char* hvdhip_last_error(void) { return t_error.c_str(); }
int hvdhip_set_fp16_scale_mode(int) { return 0; }
int hvdhip_get_fp16_scale_mode(void) { return 0; }
int64_t hvdhip_dtype_size(int dtype) {
  static const int sizes[] = {1, 1, 2, 2, 4, 8, 2, 4, 8, 1};
  return dtype >= 0 && dtype <= 9 ? sizes[dtype] : -1;
}
int hvdhip_get_device(int* device) {
  *device = t_device < 0 ? 0 : t_device;
  return 0;
}
int hvdhip_set_device(int device) {
  t_device = device;
  std::lock_guard<std::mutex> g(g_devices_mu);
  ++g_set_device_calls[std::this_thread::get_id()];
  return 0;
}

int hvdhip_stream_create(void** stream) {
  FakeStream* s = new FakeStream();
  std::lock_guard<std::mutex> g(g_streams_mu);
  g_streams.push_back(s);
  *stream = s;
  return 0;
}
int hvdhip_stream_destroy(void* stream) {
  S(stream)->drain();
  {
    std::lock_guard<std::mutex> g(g_streams_mu);
    for (size_t i = 0; i < g_streams.size(); ++i)
      if (g_streams[i] == S(stream)) g_streams.erase(g_streams.begin() + (long)i);
  }
  {
    std::lock_guard<std::mutex> g(g_pool_mu);
    for (FakeEvent* e : g_pool[stream]) delete e;
    g_pool.erase(stream);
  }
  delete S(stream);
  return 0;
}
int hvdhip_stream_forget(void* stream) {
  S(stream)->drain();
  return 0;
}
int hvdhip_stream_synchronize(void* stream) {
  S(stream)->drain();
  return 0;
}
int hvdhip_stream_wait_event(void* stream, void* event) {
  if (!stream) return 0;  // the pretend null stream holds no work
  FakeEvent* e = E(event);
  uint64_t target;
  {
    std::lock_guard<std::mutex> g(e->mu);
    target = e->recorded;
  }
  S(stream)->push([e, target] {
    std::unique_lock<std::mutex> lock(e->mu);
    e->cv.wait(lock, [&] { return e->completed >= target; });
  });
  return 0;
}

int hvdhip_event_acquire(void* stream, void** event) {
  // the calling thread must have a device: the real pool is keyed by (device, stream)
  if (t_device < 0) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "event acquired on a thread that never called SetDevice");
  std::lock_guard<std::mutex> g(g_pool_mu);
  auto& idle = g_pool[stream];
  if (idle.empty()) {
    *event = new FakeEvent();
  } else {
    *event = idle.back();
    idle.pop_back();
  }
  ++g_events_out;
  return 0;
}
int hvdhip_event_release(void* stream, void* event) {
  if (t_device < 0) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "event released on a thread that never called SetDevice");
  std::lock_guard<std::mutex> g(g_pool_mu);
  g_pool[stream].push_back(E(event));
  --g_events_out;
  return 0;
}
int hvdhip_event_pool_size(void* stream, int* count) {
  std::lock_guard<std::mutex> g(g_pool_mu);
  *count = (int)g_pool[stream].size();
  return 0;
}
int hvdhip_event_record(void* event, void* stream) {
  FakeEvent* e = E(event);
  uint64_t gen;
  {
    std::lock_guard<std::mutex> g(e->mu);
    gen = ++e->recorded;
  }
  S(stream)->push([e, gen] {
    {
      std::lock_guard<std::mutex> g(e->mu);
      if (e->completed < gen) e->completed = gen;
    }
    e->cv.notify_all();
  });
  return 0;
}
int hvdhip_event_query(void* event, int* done) {
  FakeEvent* e = E(event);
  std::lock_guard<std::mutex> g(e->mu);
  *done = e->completed >= e->recorded;
  return 0;
}
int hvdhip_event_synchronize(void* event) {
  FakeEvent* e = E(event);
  {
    std::unique_lock<std::mutex> lock(e->mu);
    const uint64_t target = e->recorded;
    e->cv.wait(lock, [&] { return e->completed >= target; });
  }
  int left = g_fail_event_syncs.load();
  while (left > 0 && !g_fail_event_syncs.compare_exchange_weak(left, left - 1)) {
  }
  if (left > 0) return fail(719, "pretend device fault");
  return 0;
}

int hvdhip_memcpy_async(void* dst, const void* src, size_t count, int, void* stream) {
  ++g_launches;
  S(stream)->push([=] {
    kernel_delay();
    std::memmove(dst, src, count);
  });
  return 0;
}

int hvdhip_timer_create(void**) { return HVDHIP_ERR_INVALID_ARGUMENT; }
int hvdhip_timer_start(void*, void*) { return HVDHIP_ERR_INVALID_ARGUMENT; }
int hvdhip_timer_stop(void*, void*) { return HVDHIP_ERR_INVALID_ARGUMENT; }
int hvdhip_timer_elapsed_ms(void*, float*) { return HVDHIP_ERR_INVALID_ARGUMENT; }
int hvdhip_timer_destroy(void*) { return 0; }

int hvdhip_batched_d2d_memcpy(void* const* out, const void* const* in, const size_t* sizes, int n, void* stream) {
  std::vector<void*> o(out, out + n);
  std::vector<const void*> i(in, in + n);
  std::vector<size_t> s(sizes, sizes + n);
  ++g_launches;
  S(stream)->push([o, i, s] {
    kernel_delay();
    for (size_t k = 0; k < s.size(); ++k) std::memmove(o[k], i[k], s[k]);
  });
  return 0;
}
int hvdhip_batched_scaled_d2d_memcpy(void* const*, const void* const*, const size_t*, int, double, int, void*) {
  return fail(HVDHIP_ERR_UNSUPPORTED_DTYPE, "not modelled");
}
int hvdhip_copy_cache_stats(uint64_t*, uint64_t*, uint64_t*, uint64_t*) { return 0; }
int hvdhip_copy_cache_set_limits(uint64_t, uint64_t) { return 0; }

int hvdhip_scale_buffer(const void* in, void* out, int64_t n, double scale, int dtype, void* stream) {
  if (dtype != HVDHIP_FLOAT32) return fail(HVDHIP_ERR_UNSUPPORTED_DTYPE, "the pretend device scales float32 only");
  ++g_launches;
  const float f = (float)scale;
  S(stream)->push([=] {
    kernel_delay();
    const float* x = static_cast<const float*>(in);
    float* y = static_cast<float*>(out);
    for (int64_t i = 0; i < n; ++i) y[i] = f * x[i];
  });
  return 0;
}

int hvdhip_fusion_plan_create(const void* const* tensors, void* const* outputs, const int64_t* num_elements, int n,
                              int tensor_dtype, int buffer_dtype, hvdhip_fusion_plan** plan) {
  if (tensor_dtype != HVDHIP_FLOAT32 || buffer_dtype != HVDHIP_FLOAT32)
    return fail(HVDHIP_ERR_UNSUPPORTED_DTYPE, "the pretend device packs float32 only");
  hvdhip_fusion_plan* p = new hvdhip_fusion_plan();
  int64_t off = 0;
  for (int i = 0; i < n; ++i) {
    p->tensors.push_back(static_cast<const float*>(tensors[i]));
    p->outputs.push_back(static_cast<float*>(outputs[i]));
    p->counts.push_back(num_elements[i]);
    p->offsets.push_back(off);
    off += 16 * ((num_elements[i] * 4 + 15) / 16);
  }
  p->buffer_len = off;
  *plan = p;
  return 0;
}
int hvdhip_fusion_plan_destroy(hvdhip_fusion_plan* plan) {
  device_synchronize();  // queued kernels may still read the plan, as the real library's tables
  delete plan;
  return 0;
}
int64_t hvdhip_fusion_plan_buffer_len(const hvdhip_fusion_plan* plan) { return plan->buffer_len; }
int hvdhip_fusion_plan_offsets(const hvdhip_fusion_plan* plan, int64_t* offsets) {
  for (size_t i = 0; i < plan->offsets.size(); ++i) offsets[i] = plan->offsets[i];
  return 0;
}
int64_t hvdhip_fusion_plan_num_chunks(const hvdhip_fusion_plan* plan) { return (int64_t)plan->counts.size(); }

int hvdhip_fusion_pack(hvdhip_fusion_plan* plan, void* fusion_buffer, double scale, unsigned, void* stream) {
  ++g_launches;
  const float f = (float)scale;
  S(stream)->push([=] {
    kernel_delay();
    char* base = static_cast<char*>(fusion_buffer);
    std::memset(base, 0, (size_t)plan->buffer_len);
    for (size_t i = 0; i < plan->counts.size(); ++i) {
      float* dst = reinterpret_cast<float*>(base + plan->offsets[i]);
      for (int64_t j = 0; j < plan->counts[i]; ++j) dst[j] = scale == 1.0 ? plan->tensors[i][j] : f * plan->tensors[i][j];
    }
  });
  return 0;
}
int hvdhip_fusion_unpack(hvdhip_fusion_plan* plan, const void* fusion_buffer, double scale, void* stream) {
  ++g_launches;
  const float f = (float)scale;
  S(stream)->push([=] {
    kernel_delay();
    const char* base = static_cast<const char*>(fusion_buffer);
    for (size_t i = 0; i < plan->counts.size(); ++i) {
      const float* src = reinterpret_cast<const float*>(base + plan->offsets[i]);
      for (int64_t j = 0; j < plan->counts[i]; ++j) plan->outputs[i][j] = scale == 1.0 ? src[j] : f * src[j];
    }
  });
  return 0;
}
int hvdhip_fusion_unpack_record(hvdhip_fusion_plan* plan, const void* fusion_buffer, double scale, void* stream,
                                void* event) {
  int rc = hvdhip_fusion_unpack(plan, fusion_buffer, scale, stream);
  return rc ? rc : hvdhip_event_record(event, stream);
}

int hvdhip_reduce_sum_k(void* resident, const void* const* incoming, int k, int64_t n, int dtype, void* stream) {
  if (dtype != HVDHIP_FLOAT32) return fail(HVDHIP_ERR_UNSUPPORTED_DTYPE, "the pretend device sums float32 only");
  std::vector<const float*> peers;
  for (int i = 0; i < k; ++i) peers.push_back(static_cast<const float*>(incoming[i]));
  ++g_launches;
  S(stream)->push([=] {
    kernel_delay();
    float* r = static_cast<float*>(resident);
    for (int64_t i = 0; i < n; ++i)
      for (const float* p : peers) r[i] = r[i] + p[i];
  });
  return 0;
}
int hvdhip_reduce_sum(void* resident, const void* incoming, int64_t n, int dtype, void* stream) {
  const void* one[1] = {incoming};
  return hvdhip_reduce_sum_k(resident, one, 1, n, dtype, stream);
}

int hvdhip_adasum_plan_create(const int*, int, int, hvdhip_adasum_plan**) { return fail(HVDHIP_ERR_UNSUPPORTED_DTYPE, "not modelled"); }
int hvdhip_adasum_plan_destroy(hvdhip_adasum_plan*) { return 0; }
int hvdhip_adasum_dot_norms(hvdhip_adasum_plan*, const void*, const void*, void*) { return HVDHIP_ERR_UNSUPPORTED_DTYPE; }
int hvdhip_adasum_scaled_add(hvdhip_adasum_plan*, void*, const void*, void*) { return HVDHIP_ERR_UNSUPPORTED_DTYPE; }
int hvdhip_adasum_combine(hvdhip_adasum_plan*, void*, const void*, void*) { return HVDHIP_ERR_UNSUPPORTED_DTYPE; }
int hvdhip_adasum_read(hvdhip_adasum_plan*, double*, double*, void*) { return HVDHIP_ERR_UNSUPPORTED_DTYPE; }
int hvdhip_adasum_set_coeffs(hvdhip_adasum_plan*, const double*, void*) { return HVDHIP_ERR_UNSUPPORTED_DTYPE; }
int hvdhip_adasum_dot_and_norm_sqrds(const void*, const void*, int, int, double*, double*, double*, void*) {
  return HVDHIP_ERR_UNSUPPORTED_DTYPE;
}
int hvdhip_adasum_dispatch_scaled_add(int, int, double, void*, double, const void*, void*) { return HVDHIP_ERR_UNSUPPORTED_DTYPE; }
int hvdhip_adasum_combine_static(void*, const void*, int, int, double*, void*) { return HVDHIP_ERR_UNSUPPORTED_DTYPE; }

}  // extern "C"
