// context.cc -- errors, device, streams, pooled events, timers and the
// table upload shared by all plans.  Host code only.
//
// The stream and event handling follows the member set of the reference's
// GPUContext::impl (ops/cuda_operations.cc:28-210): one pool of
// timing-disabled events per (device, stream), filled with 128 events on
// first use, guarded by a mutex because finalizer threads release events
// while the background thread acquires them.
#include <atomic>
#include <cstdarg>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <utility>

#include "internal.h"

namespace hvdhip {

namespace {
thread_local std::string g_last_error;

struct EventPools {
  std::mutex mu;
  std::map<std::pair<int, hipStream_t>, std::vector<hipEvent_t>> idle;
  std::map<std::pair<int, hipStream_t>, bool> filled;
};
EventPools& pools() {
  static EventPools* p = new EventPools();  // never destroyed: outlives static teardown
  return *p;
}
constexpr int kPrepopulate = 128;  // N_CUDA_EVENTS_PREPOPULATE, ops/cuda_operations.cc:218

// Flags of the pooled events: no timing, like the reference's (ops/cuda_operations.cc:58).  A record
// of such an event costs 2.9 us on the stream between two kernels, 1.8 us of which is the
// system-scope fence that makes the work before it visible to the host and to other devices.
// Horovod's consumers of a completed response are kernels and copies on the same device, which
// the fence does nothing for; HVDHIP_EVENT_SYSTEM_FENCE=0 leaves it out (1.1 us per record).
// The default keeps it, as every HIP event has it unless asked otherwise.
unsigned pooled_event_flags() {
  static const unsigned flags = [] {
    const char* e = std::getenv("HVDHIP_EVENT_SYSTEM_FENCE");
    const bool fence = !(e && e[0] == '0');
    return (unsigned)hipEventDisableTiming | (fence ? 0u : (unsigned)hipEventDisableSystemFence);
  }();
  return flags;
}

struct Timer {
  hipEvent_t start;
  hipEvent_t stop;
};
}  // namespace

int fail(int code, const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_last_error = buf;
  return code;
}

int ok() {
  g_last_error.clear();
  return 0;
}

uint32_t chunk_bytes(Family f) {
#ifdef HVDHIP_TUNING
  // Tuning builds only (libhvdhip_tuning.so): HVDHIP_CHUNK_BYTES, a multiple of 4096, replaces every
  // family's chunk size, so that tests reach the kernels' multi-vector loops.
  static uint32_t forced = [] {
    const char* e = getenv("HVDHIP_CHUNK_BYTES");
    if (e) {
      long x = strtol(e, nullptr, 10);
      if (x >= 4096 && x <= (1 << 24) && x % 4096 == 0) return (uint32_t)x;
    }
    return 0u;
  }();
  if (forced) return forced;
  // HVDHIP_UNPACK_CHUNK_BYTES: the unpack tables alone.
  static uint32_t forced_unpack = [] {
    const char* e = getenv("HVDHIP_UNPACK_CHUNK_BYTES");
    if (e) {
      long x = strtol(e, nullptr, 10);
      if (x >= 4096 && x <= (1 << 24) && x % 4096 == 0) return (uint32_t)x;
    }
    return 0u;
  }();
  if (forced_unpack && f == Family::kUnpack) return forced_unpack;
#endif
  switch (f) {
  case Family::kXfer: return kXferChunkBytes;
  case Family::kXferNarrowing: return kXferNarrowingChunkBytes;
  case Family::kUnpack: return kUnpackChunkBytes;
  case Family::kReduce: return kReduceChunkBytes;
  default: return kAdasumChunkBytes;
  }
}

int upload_chunks(const std::vector<Chunk>& chunks, DevTables* out) {
  if (chunks.size() > kMaxWorkgroups)
    return fail(HVDHIP_ERR_TOO_LARGE, "plan needs %zu workgroups; the limit is %llu", chunks.size(),
                (unsigned long long)kMaxWorkgroups);
  const size_t total = chunks.empty() ? 256 : chunks.size() * sizeof(Chunk);
  void* dev = nullptr;
  hipError_t e = hipMalloc(&dev, total);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    return fail(e == hipErrorOutOfMemory ? HVDHIP_ERR_OUT_OF_MEMORY : (int)e,
                "hipMalloc of %zu table bytes failed: %s", total, hipGetErrorString(e));
  }
  if (!chunks.empty()) {
    e = hipMemcpy(dev, chunks.data(), total, hipMemcpyHostToDevice);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      (void)hipFree(dev);
      return fail((int)e, "hipMemcpy of plan tables failed: %s", hipGetErrorString(e));
    }
  }
  out->alloc = dev;
  out->chunks = static_cast<Chunk*>(dev);
  out->nchunks = (uint32_t)chunks.size();
  out->nlaunch = out->nchunks;
  return 0;
}

uint64_t count_chunks(const std::vector<Seg>& segs, uint32_t chunk_units) {
  uint64_t nchunks = 0;
  for (const Seg& s : segs) nchunks += (s.n + chunk_units - 1) / chunk_units;
  return nchunks > kMaxWorkgroups ? ~0ull : nchunks;
}

uint32_t xcd_run(uint64_t nchunks, uint32_t chunk_bytes, bool long_runs) {
  if (chunk_bytes == 0) return 0;
  const uint32_t bytes =
      !long_runs && nchunks * (uint64_t)chunk_bytes <= kXcdLongRunFrom ? kXcdRunBytes : kXcdLongRunBytes;
  return bytes > chunk_bytes ? bytes / chunk_bytes : 1;
}

int store_policy(Stores family) {
  constexpr unsigned kDefaultThrough = 1u << (unsigned)Stores::kPack | 1u << (unsigned)Stores::kPackNarrowing |
                                       1u << (unsigned)Stores::kReduceFew | 1u << (unsigned)Stores::kReduceMany;
#ifdef HVDHIP_TUNING
  // Tuning builds only: HVDHIP_WRITE_THROUGH=<mask> (bit = enumerator value) replaces the table.
  static const unsigned through = [] {
    const char* e = std::getenv("HVDHIP_WRITE_THROUGH");
    return e ? (unsigned)std::strtoul(e, nullptr, 0) : kDefaultThrough;
  }();
#else
  constexpr unsigned through = kDefaultThrough;
#endif
  return (through >> (unsigned)family) & 1u;
}

XcdOrder xcd_order(uint64_t nblocks, uint32_t tile_bytes) {
  const uint32_t run = xcd_run(nblocks, tile_bytes);
  XcdOrder o = {0, 0};
  if (run == 0 || (run & (run - 1)) != 0) return o;  // natural order
  while ((1u << o.shift) < run) ++o.shift;
  const uint64_t group = (uint64_t)kXcds << o.shift;
  o.ordered = (uint32_t)(nblocks / group * group);
  return o;
}

void fill_chunks(const std::vector<Seg>& segs, uint32_t chunk_units, uint32_t tensor_es,
                 uint32_t buffer_es, Chunk* out, uint64_t nchunks) {
  const uint32_t run = xcd_run(nchunks, chunk_units * (tensor_es > buffer_es ? tensor_es : buffer_es));
  const uint64_t slots = table_slots(nchunks);
  for (uint64_t i = nchunks / kLineGroup * kLineGroup; i < slots; ++i) out[i] = Chunk{0, 0, 0, 0, 0};  // the padded last group
  uint64_t index = 0;
  for (const Seg& s : segs) {
    const uint64_t nbytes = s.n * buffer_es;
    for (uint64_t start = 0; start < s.n; start += chunk_units) {
      const uint64_t left = s.n - start;
      Chunk c;
      c.tensor = s.tensor + start * tensor_es;
      c.output = s.output + start * tensor_es;
      c.off = s.off + start * buffer_es;
      c.n = (uint32_t)(left < chunk_units ? left : chunk_units);
      c.pad = left <= chunk_units ? (uint32_t)((16 - (nbytes & 15)) & 15) : 0;
      out[line_slot((uint32_t)xcd_slot(index++, nchunks, run))] = c;
    }
  }
}

int build_tables(const std::vector<Seg>& segs, uint32_t chunk_units, uint32_t tensor_es,
                 uint32_t buffer_es, DevTables* out) {
  if (chunk_units == 0) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "chunk_units is zero");
  const uint64_t nchunks = count_chunks(segs, chunk_units);
  if (nchunks == ~0ull) return fail(HVDHIP_ERR_TOO_LARGE, "plan needs more than 2^23 workgroups");
  std::vector<Chunk> chunks((size_t)table_slots(nchunks));
  fill_chunks(segs, chunk_units, tensor_es, buffer_es, chunks.data(), nchunks);
  int rc = upload_chunks(chunks, out);
  if (rc == 0) out->nchunks = (uint32_t)nchunks;
  return rc;
}

int free_tables(DevTables* t) {
  if (t->alloc) {
    HVDHIP_CHECK(hipFree(t->alloc));
    t->alloc = nullptr;
  }
  return 0;
}

std::atomic<int> g_fp16_scale_mode{HVDHIP_FP16_SCALE_FP32_FACTOR};

float fp16_scale_factor(double scale) {
  const float f = (float)scale;
  if (g_fp16_scale_mode.load(std::memory_order_relaxed) == HVDHIP_FP16_SCALE_HALF_FACTOR)
    return (float)(_Float16)f;  // __float2half((float)scale_factor), ops/cuda/cuda_kernels.cu:167
  return f;
}

}  // namespace hvdhip

using namespace hvdhip;

extern "C" {

const char* hvdhip_error_string(int code) {
  if (code == 0) return "success";
  if (code > 0) return hipGetErrorString((hipError_t)code);
  switch (code) {
  case HVDHIP_ERR_INVALID_ARGUMENT: return "invalid argument";
  case HVDHIP_ERR_UNSUPPORTED_DTYPE: return "data type not supported by this operation";
  case HVDHIP_ERR_OUT_OF_MEMORY: return "out of device memory";
  case HVDHIP_ERR_TOO_LARGE: return "size exceeds what one launch can cover";
  default: return "unknown hvdhip error";
  }
}

const char* hvdhip_last_error(void) { return g_last_error.c_str(); }

int hvdhip_set_fp16_scale_mode(int mode) {
  if (mode != HVDHIP_FP16_SCALE_FP32_FACTOR && mode != HVDHIP_FP16_SCALE_HALF_FACTOR)
    return fail(HVDHIP_ERR_INVALID_ARGUMENT, "unknown fp16 scale mode %d", mode);
  g_fp16_scale_mode.store(mode, std::memory_order_relaxed);
  return ok();
}

int hvdhip_get_fp16_scale_mode(void) { return g_fp16_scale_mode.load(std::memory_order_relaxed); }

int64_t hvdhip_dtype_size(int dtype) { return dtype_size(dtype); }

int hvdhip_get_device(int* device) {
  if (!device) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "device is NULL");
  HVDHIP_CHECK(hipGetDevice(device));
  return ok();
}

int hvdhip_set_device(int device) {
  HVDHIP_CHECK(hipSetDevice(device));
  return ok();
}

int hvdhip_stream_create(void** stream) {
  if (!stream) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "stream is NULL");
  hipStream_t s;
  HVDHIP_CHECK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  *stream = s;
  return ok();
}

namespace {
// Waits for the stream and drops everything the library keeps per stream: idle pooled events,
// the streams' marks on cached copy tables, single-layer Adasum plans.
int forget_stream(hipStream_t s) {
  int dev = 0;
  HVDHIP_CHECK(hipGetDevice(&dev));
  // Work still queued completes first, so that nothing the library remembers about the stream
  // (tables a launch on it reads) outlives it.
  HVDHIP_CHECK(hipStreamSynchronize(s));
  {
    EventPools& p = pools();
    std::lock_guard<std::mutex> g(p.mu);
    auto key = std::make_pair(dev, s);
    auto it = p.idle.find(key);
    if (it != p.idle.end()) {
      for (hipEvent_t ev : it->second) (void)hipEventDestroy(ev);
      p.idle.erase(it);
    }
    p.filled.erase(key);
  }
  copy_cache_forget_stream(s);
  adasum_forget_stream(s);
  return 0;
}
}  // namespace

int hvdhip_stream_destroy(void* stream) {
  hipStream_t s = static_cast<hipStream_t>(stream);
  int rc = forget_stream(s);
  if (rc) return rc;
  HVDHIP_CHECK(hipStreamDestroy(s));
  return ok();
}

int hvdhip_stream_forget(void* stream) {
  int rc = forget_stream(static_cast<hipStream_t>(stream));
  return rc ? rc : ok();
}

int hvdhip_stream_synchronize(void* stream) {
  HVDHIP_CHECK(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
  return ok();
}

int hvdhip_stream_wait_event(void* stream, void* event) {
  if (!event) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "event is NULL");
  HVDHIP_CHECK(hipStreamWaitEvent(static_cast<hipStream_t>(stream), static_cast<hipEvent_t>(event), 0));
  return ok();
}

int hvdhip_event_acquire(void* stream, void** event) {
  if (!event) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "event is NULL");
  int dev = 0;
  HVDHIP_CHECK(hipGetDevice(&dev));
  hipStream_t s = static_cast<hipStream_t>(stream);
  EventPools& p = pools();
  {
    std::lock_guard<std::mutex> g(p.mu);
    auto key = std::make_pair(dev, s);
    auto& q = p.idle[key];
    if (!p.filled[key]) {
      p.filled[key] = true;  // one attempt per stream, also when it stops early on an error
      for (int i = 0; i < kPrepopulate; ++i) {
        hipEvent_t ev;
        HVDHIP_CHECK(hipEventCreateWithFlags(&ev, pooled_event_flags()));
        q.push_back(ev);
      }
    }
    if (!q.empty()) {
      *event = q.back();
      q.pop_back();
      return ok();
    }
  }
  hipEvent_t ev;
  HVDHIP_CHECK(hipEventCreateWithFlags(&ev, pooled_event_flags()));
  *event = ev;
  return ok();
}

int hvdhip_event_record(void* event, void* stream) {
  if (!event) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "event is NULL");
  HVDHIP_CHECK(hipEventRecord(static_cast<hipEvent_t>(event), static_cast<hipStream_t>(stream)));
  return ok();
}

int hvdhip_event_query(void* event, int* done) {
  if (!event || !done) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "event or done is NULL");
  hipError_t e = hipEventQuery(static_cast<hipEvent_t>(event));
  if (e == hipSuccess) {
    *done = 1;
    return ok();
  }
  if (e == hipErrorNotReady) {
    *done = 0;
    return ok();
  }
  return fail((int)e, "hipEventQuery failed: %s", hipGetErrorString(e));
}

int hvdhip_event_synchronize(void* event) {
  if (!event) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "event is NULL");
  HVDHIP_CHECK(hipEventSynchronize(static_cast<hipEvent_t>(event)));
  return ok();
}

int hvdhip_event_release(void* stream, void* event) {
  if (!event) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "event is NULL");
  int dev = 0;
  HVDHIP_CHECK(hipGetDevice(&dev));
  EventPools& p = pools();
  std::lock_guard<std::mutex> g(p.mu);
  p.idle[std::make_pair(dev, static_cast<hipStream_t>(stream))].push_back(static_cast<hipEvent_t>(event));
  return ok();
}

int hvdhip_event_pool_size(void* stream, int* count) {
  if (!count) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "count is NULL");
  int dev = 0;
  HVDHIP_CHECK(hipGetDevice(&dev));
  EventPools& p = pools();
  std::lock_guard<std::mutex> g(p.mu);
  auto it = p.idle.find(std::make_pair(dev, static_cast<hipStream_t>(stream)));
  *count = it == p.idle.end() ? 0 : (int)it->second.size();
  return ok();
}

int hvdhip_memcpy_async(void* dst, const void* src, size_t count, int kind, void* stream) {
  hipMemcpyKind k;
  switch (kind) {
  case HVDHIP_MEMCPY_H2D: k = hipMemcpyHostToDevice; break;
  case HVDHIP_MEMCPY_D2H: k = hipMemcpyDeviceToHost; break;
  case HVDHIP_MEMCPY_D2D: k = hipMemcpyDeviceToDevice; break;
  default: return fail(HVDHIP_ERR_INVALID_ARGUMENT, "unknown memcpy kind %d", kind);
  }
  if (count == 0) return ok();
  HVDHIP_CHECK(hipMemcpyAsync(dst, src, count, k, static_cast<hipStream_t>(stream)));
  return ok();
}

int hvdhip_timer_create(void** timer) {
  if (!timer) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "timer is NULL");
  Timer* t = new Timer();
  hipError_t e = hipEventCreate(&t->start);
  if (e == hipSuccess) {
    e = hipEventCreate(&t->stop);
    if (e != hipSuccess) (void)hipEventDestroy(t->start);
  }
  if (e != hipSuccess) {
    delete t;
    return fail((int)e, "hipEventCreate failed: %s", hipGetErrorString(e));
  }
  *timer = t;
  return ok();
}

int hvdhip_timer_start(void* timer, void* stream) {
  if (!timer) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "timer is NULL");
  HVDHIP_CHECK(hipEventRecord(static_cast<Timer*>(timer)->start, static_cast<hipStream_t>(stream)));
  return ok();
}

int hvdhip_timer_stop(void* timer, void* stream) {
  if (!timer) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "timer is NULL");
  HVDHIP_CHECK(hipEventRecord(static_cast<Timer*>(timer)->stop, static_cast<hipStream_t>(stream)));
  return ok();
}

int hvdhip_timer_elapsed_ms(void* timer, float* ms) {
  if (!timer || !ms) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "timer or ms is NULL");
  Timer* t = static_cast<Timer*>(timer);
  HVDHIP_CHECK(hipEventSynchronize(t->stop));
  HVDHIP_CHECK(hipEventElapsedTime(ms, t->start, t->stop));
  return ok();
}

int hvdhip_timer_destroy(void* timer) {
  if (!timer) return ok();
  Timer* t = static_cast<Timer*>(timer);
  (void)hipEventDestroy(t->start);
  (void)hipEventDestroy(t->stop);
  delete t;
  return ok();
}

}  // extern "C"
