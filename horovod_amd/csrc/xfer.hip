// xfer.hip -- batched fusion-buffer packing and unpacking, with the pre/post
// scale and the fp32<->fp16 compression cast fused in, plus the whole-buffer
// scale.  gfx950 only.
//
// One launch moves a whole fused response.  The host describes it with one
// device-resident table of self-contained 32-byte chunk entries (source,
// destination, fusion-buffer offset, element count), one per workgroup.  A
// workgroup of four wave64 wavefronts loads its entry with a single scalar
// load and streams its chunk with one 16-byte access per lane each way
// (4 KiB per workgroup: the occupancy of many small workgroups keeps about
// 8 MiB in flight, which is what HBM latency times bandwidth asks for).
// Loads are non-temporal; stores either bypass the Infinity Cache or write
// through it for the kernel that reads the destination next.  Workgroups are
// dispatched round-robin over the XCDs and the table is ordered so that each
// XCD walks runs of consecutive chunks: a single big tensor is spread over
// all XCDs and HBM stacks while a tiny one costs a single short
// workgroup.  This is bandwidth-bound byte/element work with no reuse: no
// LDS and no matrix cores are involved.
//
// All vector accesses are declared with element alignment only.  gfx950
// serves multi-dword global accesses at any alignment, so no alignment
// ladder or head peeling is needed; 16-byte aligned data (the normal case:
// fusion offsets are padded to 16 bytes) takes exactly the same instructions.
//
// Arithmetic follows the reference's CPU path (ScaleBufferCPUImpl,
// ops/collective_operations.h:91-127), not its CUDA kernels: fp16 is scaled
// in fp32 with an fp32 factor and rounded to nearest even once; integers are
// scaled in double and truncated toward zero.
#include <algorithm>
#include <cstring>
#include <deque>
#include <iterator>
#include <list>
#include <map>
#include <mutex>
#include <unordered_map>

#include "internal.h"
#include "vecmem.h"

namespace hvdhip {
namespace {

// ----------------------------------------------------------------------
// Device side
// ----------------------------------------------------------------------

// Each Op gives the source and destination element types, the number of
// elements per lane access (16 bytes on the wider side), the by-value launch
// parameter and the per-element function.

// Plain copy of elements as unsigned integers of the same width: bit-exact
// for every dtype.
template <typename U>
struct Copy {
  typedef U S;
  typedef U D;
  static constexpr int VEC = 16 / (int)sizeof(U);
  struct P {};
  static __device__ __forceinline__ D f(S x, P) { return x; }
};

// out = (T)(factor * in): factor type TS is double for u8/i8/i32/i64/f64 and
// float for f32 (ops/collective_operations.cc:119-140).
template <typename T, typename TS>
struct Scale {
  typedef T S;
  typedef T D;
  static constexpr int VEC = 16 / (int)sizeof(T);
  struct P {
    TS s;
  };
  static __device__ __forceinline__ D f(S x, P p) { return (T)(p.s * x); }
};

// fp16 scaled through fp32 with an fp32 factor, one rounding to nearest even
// (ops/collective_operations.h:99-127).  When the host hands over a factor that a
// half holds exactly, the fp32 product of two halves is exact and the result is the
// correctly rounded half product, i.e. __hmul (ops/cuda/cuda_kernels.cu:96-136).
struct ScaleHalf {
  typedef half_t S;
  typedef half_t D;
  static constexpr int VEC = 8;
  struct P {
    float s;
  };
  static __device__ __forceinline__ D f(S x, P p) { return (half_t)opaque(p.s * (float)x); }
};

// fp32 -> fp16 with the prescale applied in fp32 first: a single rounding.
// A lane takes 32 bytes of fp32 (two 16-byte loads) and stores 16 bytes of fp16: with 8-byte
// stores (four elements per lane) the same pack is 2 % slower.
struct PackF32F16 {
  typedef float S;
  typedef half_t D;
  static constexpr int VEC = 8;
  struct P {
    float s;
  };
  static __device__ __forceinline__ D f(S x, P p) { return (half_t)opaque(p.s * x); }
};

// fp32 -> fp16 first (horovod/torch/compression.py:49-55), then the fp16
// scale: two roundings, the order of the reference pipeline.
struct PackF32F16CastFirst {
  typedef float S;
  typedef half_t D;
  static constexpr int VEC = 8;
  struct P {
    float s;
  };
  static __device__ __forceinline__ D f(S x, P p) {
    half_t h = (half_t)x;
    return (half_t)opaque(p.s * (float)h);
  }
};

// Postscale on the fp16 value (rounded back to fp16), then the exact widening
// of Compression.fp16.decompress (horovod/torch/compression.py:58-64).
// Four elements per lane: 8 bytes in, one 16-byte store out.  (Eight per lane would store two
// 16-byte pieces at a 32-byte stride, and such half-covered store instructions cost 40 %.)
struct UnpackF16F32 {
  typedef half_t S;
  typedef float D;
  static constexpr int VEC = 4;
  struct P {
    float s;
  };
  static __device__ __forceinline__ D f(S x, P p) {
    half_t h = (half_t)opaque(p.s * (float)x);
    return (float)h;
  }
};

constexpr int kUnroll = 4;  // 16-byte loads in flight per lane, for chunks of more than one vector per lane

// Streams n elements from src to dst through Op::f with the whole workgroup.
template <class Op, int ST>
__device__ __forceinline__ void stream_range(gptr<const typename Op::S> src,
                                             gptr<typename Op::D> dst, uint32_t n,
                                             typename Op::P p) {
  typedef typename Op::S S;
  typedef typename Op::D D;
  constexpr int VEC = Op::VEC;
  // src and dst may be the same buffer (in-place scale): every lane loads all
  // of an iteration's vectors before it stores any, and touches no address
  // another lane touches.
  const uint32_t nv = n / VEC;
  const Window out = store_window<ST>(dst, n * (uint32_t)sizeof(D));
  constexpr bool kBytes = sizeof(S) == 1;  // byte elements are read through a window (vecmem.h)
  ReadWindow in;
  if constexpr (kBytes) in = load_window(src, n);
  auto load = [&](uint32_t vec) {
    if constexpr (kBytes) {
      return ldw<S, VEC>(in, vec * 16u);
    } else {
      return ldv<S, VEC>(src + (size_t)vec * VEC);
    }
  };
  uint32_t v = threadIdx.x;
  for (; v + (kUnroll - 1) * kWG < nv; v += kUnroll * kWG) {
    Arr<S, VEC> x[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) x[u] = load(v + u * kWG);
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      Arr<D, VEC> y;
#pragma unroll
      for (int j = 0; j < VEC; ++j) y.v[j] = Op::f(x[u].v[j], p);
      stw<ST, D, VEC>(out, (v + u * kWG) * (uint32_t)(VEC * sizeof(D)), y);
    }
  }
  for (; v < nv; v += kWG) {
    const Arr<S, VEC> x = load(v);
    Arr<D, VEC> y;
#pragma unroll
    for (int j = 0; j < VEC; ++j) y.v[j] = Op::f(x.v[j], p);
    stw<ST, D, VEC>(out, v * (uint32_t)(VEC * sizeof(D)), y);
  }
  const uint32_t t = nv * VEC + threadIdx.x;  // fewer than VEC elements remain
  if (t < n) dst[t] = Op::f(src[t], p);
}

enum Mode { kPack = 0, kUnpack = 1, kDirect = 2 };

// One workgroup per chunk-table entry (entry line_slot(b) for workgroup b; the entries that pad
// the table to a multiple of 32 are empty and their workgroups leave at once).
//   kPack:   src = chunk.tensor,      dst = base + chunk.off (pad bytes zeroed)
//   kUnpack: src = base + chunk.off,  dst = chunk.output
//   kDirect: src = chunk.tensor,      dst = chunk.output
template <class Op, int MODE, int ST>
__global__ __launch_bounds__(kWG) void xfer_k(const Chunk* __restrict__ chunks, uint64_t base,
                                              typename Op::P p) {
  typedef typename Op::S S;
  typedef typename Op::D D;
  const Chunk c = chunks[line_slot(blockIdx.x)];
  const uint64_t src_addr = (MODE == kUnpack) ? base + c.off : c.tensor;
  const uint64_t dst_addr = (MODE == kPack) ? base + c.off : c.output;
  stream_range<Op, ST>(as_global<const S>(src_addr), as_global<D>(dst_addr), c.n, p);
  if (MODE == kPack && threadIdx.x < c.pad)
    as_global<uint8_t>(dst_addr)[(uint64_t)c.n * sizeof(D) + threadIdx.x] = 0;
}

// Contiguous buffer: workgroup b handles tile t = xcd_tile(b), elements [t*tile, (t+1)*tile).
template <class Op, int ST>
__global__ __launch_bounds__(kWG) void contig_k(const typename Op::S* src, typename Op::D* dst, uint64_t n,
                                                uint32_t tile, uint32_t shift, uint32_t ordered,
                                                typename Op::P p) {
  const uint64_t start = (uint64_t)xcd_tile(blockIdx.x, XcdOrder{shift, ordered}) * tile;
  const uint64_t left = n - start;
  const uint32_t m = left < tile ? (uint32_t)left : tile;
  stream_range<Op, ST>(as_global(src + start), as_global(dst + start), m, p);
}

// ----------------------------------------------------------------------
// Host side
// ----------------------------------------------------------------------

// gathers: a direct transfer whose destinations lie back to back, i.e. a pack into a fusion buffer
// through the array-taking entry points; it stores like a pack.
//
// completion: an event that is to read as recorded behind this transfer.  It is bound to the
// kernel's own completion signal (the launch's stop event) instead of going onto the stream as a
// marker of its own behind the kernel, which costs the stream about 2 us more.
template <class Op, int MODE>
int launch_xfer(const DevTables& t, uint64_t base, typename Op::P p, hipStream_t stream, bool gathers = false,
                hipEvent_t completion = nullptr) {
  if (t.nchunks == 0) {
    if (completion) HVDHIP_CHECK(hipEventRecord(completion, stream));
    return 0;
  }
  constexpr bool converting = sizeof(typename Op::S) != sizeof(typename Op::D);
  const Stores family = MODE == kDirect ? (gathers ? Stores::kPack : Stores::kDirect)
                        : MODE == kPack ? (converting ? Stores::kPackNarrowing : Stores::kPack)
                                        : (converting ? Stores::kUnpackWidening : Stores::kUnpack);
  const hipError_t status = with_store_policy(family, [&](auto st) {
    return launch_with(completion, xfer_k<Op, MODE, decltype(st)::value>, t.nlaunch, stream, t.chunks, base, p);
  });
  HVDHIP_CHECK_LAUNCH("xfer_k", status);
  return 0;
}

// Dispatches the same-dtype transfer over MODE; the tables count elements of
// dtype.  scale == 1.0 is a plain copy, valid for every dtype.
template <int MODE>
int launch_same_dtype(const DevTables& t, uint64_t base, double scale, int dtype,
                      hipStream_t stream, bool gathers = false, hipEvent_t completion = nullptr) {
  if (scale == 1.0) {
    switch (dtype_size(dtype)) {
    case 1: return launch_xfer<Copy<uint8_t>, MODE>(t, base, {}, stream, gathers, completion);
    case 2: return launch_xfer<Copy<uint16_t>, MODE>(t, base, {}, stream, gathers, completion);
    case 4: return launch_xfer<Copy<uint32_t>, MODE>(t, base, {}, stream, gathers, completion);
    case 8: return launch_xfer<Copy<uint64_t>, MODE>(t, base, {}, stream, gathers, completion);
    default: return fail(HVDHIP_ERR_UNSUPPORTED_DTYPE, "unknown dtype %d", dtype);
    }
  }
  switch (dtype) {
  case HVDHIP_UINT8: return launch_xfer<Scale<uint8_t, double>, MODE>(t, base, {scale}, stream, gathers, completion);
  case HVDHIP_INT8: return launch_xfer<Scale<int8_t, double>, MODE>(t, base, {scale}, stream, gathers, completion);
  case HVDHIP_INT32: return launch_xfer<Scale<int32_t, double>, MODE>(t, base, {scale}, stream, gathers, completion);
  case HVDHIP_INT64: return launch_xfer<Scale<int64_t, double>, MODE>(t, base, {scale}, stream, gathers, completion);
  case HVDHIP_FLOAT16: return launch_xfer<ScaleHalf, MODE>(t, base, {fp16_scale_factor(scale)}, stream, gathers, completion);
  case HVDHIP_FLOAT32: return launch_xfer<Scale<float, float>, MODE>(t, base, {(float)scale}, stream, gathers, completion);
  case HVDHIP_FLOAT64: return launch_xfer<Scale<double, double>, MODE>(t, base, {scale}, stream, gathers, completion);
  default:
    return fail(HVDHIP_ERR_UNSUPPORTED_DTYPE, "dtype %d cannot be scaled by a factor other than 1", dtype);
  }
}

bool scalable(int dtype) {
  switch (dtype) {
  case HVDHIP_UINT8: case HVDHIP_INT8: case HVDHIP_INT32: case HVDHIP_INT64:
  case HVDHIP_FLOAT16: case HVDHIP_FLOAT32: case HVDHIP_FLOAT64: return true;
  default: return false;
  }
}

template <class Op>
int launch_contig(const void* in, void* out, int64_t n, typename Op::P p, hipStream_t stream) {
  typedef typename Op::S S;
  typedef typename Op::D D;
  const uint32_t tile = chunk_bytes(Family::kXfer) / (uint32_t)std::max(sizeof(S), sizeof(D));
  const S* src = static_cast<const S*>(in);
  D* dst = static_cast<D*>(out);
  uint64_t left = (uint64_t)n;
  while (left > 0) {  // one launch unless the buffer needs more than kMaxWorkgroups workgroups
    const uint64_t slice = std::min<uint64_t>(left, kMaxWorkgroups * tile);
    const uint32_t blocks = (uint32_t)((slice + tile - 1) / tile);
    const XcdOrder order = xcd_order(blocks, chunk_bytes(Family::kXfer));
    const hipError_t status = with_store_policy(Stores::kContig, [&](auto st) {
      return launch(contig_k<Op, decltype(st)::value>, blocks, stream, src, dst, slice, tile, order.shift,
                    order.ordered, p);
    });
    HVDHIP_CHECK_LAUNCH("contig_k", status);
    src += slice;
    dst += slice;
    left -= slice;
  }
  return 0;
}

// ---- cache of tables for the array-taking entry points ----------------
//
// The reference passes its copy descriptors by value with every launch, so a
// caller of these entry points expects no set-up cost.  The cache keeps one
// device-resident table per distinct (out, in, sizes) set, found through a hash
// of the arrays; a hit costs the hash and one comparison.  It grows with the
// number of sets a job cycles through (a GPT-2 XL step has 49 fusion cycles
// times two directions) and is bounded by the device memory its tables take,
// not by a count of entries.
//
// A miss never waits for the device: the table is written into a pinned staging
// buffer that belongs to the entry, copied to the entry's device buffer with an
// asynchronous copy on the caller's stream, and the kernel follows on the same
// stream.  Launches leave nothing behind on the stream; an entry only remembers
// which streams have read its table.  When an entry is evicted, an event is
// recorded at the current tail of each of those streams and the entry's buffers
// are retired with those events; a later miss reuses retired buffers whose
// events have completed and allocates new ones otherwise.

struct TableBuf {
  void* dev = nullptr;
  void* pinned = nullptr;
  size_t cap = 0;
};

struct CachedCopy {
  uint64_t hash = 0;
  std::vector<uint64_t> key;  // unit size, n, then out/in/size triples
  DevTables tables;           // tables.alloc is not owned: it aliases buf.dev
  TableBuf buf;
  hipEvent_t uploaded = nullptr;    // recorded once, behind the table's upload on the stream that built it
  bool upload_complete = false;     // `uploaded` has been seen complete: other streams need not wait for it
  hipStream_t build_stream = nullptr;
  std::vector<hipStream_t> streams;  // every stream that holds, or held, a launch reading the table
  // The destinations lie back to back (each starts within 16 bytes after the one before ends) and
  // there are several: the caller packs into a fusion buffer, which the next kernel on the stream
  // reads, so the copy stores like a pack (through the Infinity Cache).
  bool gathers = false;
};

// Buffers of an evicted entry; free for reuse once every event has completed.
struct Retired {
  TableBuf buf;
  std::vector<hipEvent_t> events;
};

// One cache per device: its entries, their buffers and the spare buffers all live on that
// device, and it is only ever touched with that device current.
struct CopyCache {
  std::mutex mu;
  std::list<CachedCopy> lru;  // front = most recent
  std::unordered_multimap<uint64_t, std::list<CachedCopy>::iterator> index;  // by CachedCopy::hash
  std::vector<TableBuf> spare;
  std::deque<Retired> retired;       // oldest first
  std::vector<hipEvent_t> idle_events;
  size_t bytes = 0;                  // device bytes of the live entries' tables
  size_t max_entries = 4096;
  size_t max_bytes = (size_t)256 << 20;
  uint64_t hits = 0, misses = 0, evictions = 0;
};
struct CacheRegistry {
  std::mutex mu;
  std::map<int, CopyCache*> by_device;
};
CacheRegistry& registry() {
  static CacheRegistry* r = new CacheRegistry();  // never destroyed: outlives static teardown
  return *r;
}
int copy_cache(CopyCache** out) {
  int device = 0;
  HVDHIP_CHECK(hipGetDevice(&device));
  CacheRegistry& r = registry();
  std::lock_guard<std::mutex> g(r.mu);
  CopyCache*& c = r.by_device[device];
  if (!c) c = new CopyCache();
  *out = c;
  return 0;
}
constexpr size_t kSpareBufs = 16;
constexpr size_t kMaxRetired = 64;

void release_buf(TableBuf* b) {
  if (b->dev) (void)hipFree(b->dev);
  if (b->pinned) (void)hipHostFree(b->pinned);
  *b = TableBuf();
}

// Internal ordering only (table uploads and table reads): no timing, no system-scope fence.
int order_event(CopyCache& c, hipEvent_t* out) {
  if (!c.idle_events.empty()) {
    *out = c.idle_events.back();
    c.idle_events.pop_back();
    return 0;
  }
  HVDHIP_CHECK(hipEventCreateWithFlags(out, hipEventDisableTiming | hipEventDisableSystemFence));
  return 0;
}

void keep_buf(CopyCache& c, TableBuf* b) {
  if (c.spare.size() < kSpareBufs) {
    c.spare.push_back(*b);
    *b = TableBuf();
  } else {
    release_buf(b);
  }
}

// Moves retired buffers whose events have completed to the spares.  wait_oldest: block for the
// oldest one's events first (only when too many are retired, which means the device is far behind).
void reap_retired(CopyCache& c, bool wait_oldest) {
  while (!c.retired.empty()) {
    Retired& r = c.retired.front();
    bool complete = true;
    for (hipEvent_t e : r.events) {
      hipError_t q = wait_oldest ? hipEventSynchronize(e) : hipEventQuery(e);
      if (q != hipSuccess) {
        (void)hipGetLastError();  // hipErrorNotReady is not an error here
        complete = false;
        break;
      }
    }
    if (!complete) return;
    for (hipEvent_t e : r.events) c.idle_events.push_back(e);
    keep_buf(c, &r.buf);
    c.retired.pop_front();
    wait_oldest = false;
  }
}

// A device + pinned buffer pair of at least `bytes`: the smallest spare that fits, else new.
int acquire_buf(CopyCache& c, size_t bytes, TableBuf* out) {
  reap_retired(c, c.retired.size() > kMaxRetired);
  size_t best = c.spare.size();
  for (size_t i = 0; i < c.spare.size(); ++i)
    if (c.spare[i].cap >= bytes && (best == c.spare.size() || c.spare[i].cap < c.spare[best].cap)) best = i;
  if (best != c.spare.size()) {
    *out = c.spare[best];
    c.spare.erase(c.spare.begin() + (long)best);
    return 0;
  }
  size_t cap = 4096;
  while (cap < bytes) cap *= 2;
  TableBuf b;
  hipError_t e = hipMalloc(&b.dev, cap);
  if (e == hipSuccess) e = hipHostMalloc(&b.pinned, cap, hipHostMallocDefault);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    release_buf(&b);
    return fail(e == hipErrorOutOfMemory ? HVDHIP_ERR_OUT_OF_MEMORY : (int)e,
                "allocating %zu bytes for a copy table failed: %s", cap, hipGetErrorString(e));
  }
  b.cap = cap;
  *out = b;
  return 0;
}

// Takes the least recently used entry out of the cache.  Nothing is waited for: an event goes
// behind whatever each stream that used the table holds now, and the buffers are retired with
// those events.  Streams that were given up through hvdhip_stream_destroy or hvdhip_stream_forget
// have been taken off every entry first.  What is left is a caller's own stream that was destroyed
// without either call; the contract asks for it to have been idle then.  If the runtime rejects the
// handle, the rest of the device is waited for; if another stream has since been created at the
// same address, the event lands behind that stream's work, which is later than needed and
// harmless, because the old stream's reads had completed before it went away.
int evict_one(CopyCache& c) {
  auto victim = std::prev(c.lru.end());
  Retired r;
  r.buf = victim->buf;
  bool lost_stream = false;
  for (hipStream_t s : victim->streams) {
    hipEvent_t e = nullptr;
    int rc = order_event(c, &e);
    if (rc) {  // the victim stays; the events taken so far go back (recording them again later is fine)
      for (hipEvent_t taken : r.events) c.idle_events.push_back(taken);
      return rc;
    }
    if (hipEventRecord(e, s) == hipSuccess) {
      r.events.push_back(e);
    } else {
      (void)hipGetLastError();
      c.idle_events.push_back(e);
      lost_stream = true;
    }
  }
  if (lost_stream) HVDHIP_CHECK(hipDeviceSynchronize());
  if (victim->uploaded) r.events.push_back(victim->uploaded);  // the pinned half is read by the upload
  c.retired.push_back(std::move(r));
  c.bytes -= victim->buf.cap;
  auto range = c.index.equal_range(victim->hash);
  for (auto it = range.first; it != range.second; ++it) {
    if (it->second == victim) {
      c.index.erase(it);
      break;
    }
  }
  c.lru.erase(victim);
  ++c.evictions;
  return 0;
}

uint64_t hash_arrays(void* const* out, const void* const* in, const size_t* sizes, int n, uint32_t unit) {
  uint64_t h = 0x9e3779b97f4a7c15ull ^ ((uint64_t)unit << 32) ^ (uint64_t)n;
  auto mix = [&h](uint64_t x) {
    h ^= x;
    h *= 0xff51afd7ed558ccdull;
    h ^= h >> 32;
  };
  for (int i = 0; i < n; ++i) {
    mix((uint64_t)(uintptr_t)out[i]);
    mix((uint64_t)(uintptr_t)in[i]);
    mix((uint64_t)sizes[i]);
  }
  return h;
}

bool same_arrays(const std::vector<uint64_t>& key, void* const* out, const void* const* in,
                 const size_t* sizes, int n, uint32_t unit) {
  if (key.size() != 2 + 3 * (size_t)n || key[0] != unit || key[1] != (uint64_t)n) return false;
  const uint64_t* k = key.data() + 2;
  for (int i = 0; i < n; ++i, k += 3)
    if (k[0] != (uint64_t)(uintptr_t)out[i] || k[1] != (uint64_t)(uintptr_t)in[i] || k[2] != (uint64_t)sizes[i])
      return false;
  return true;
}

// Finds or builds the table for (out, in, sizes) with elements of unit bytes; a newly
// built table is uploaded asynchronously on `stream`.  The caller holds the cache mutex,
// launches on `stream`, then calls mark_used() before releasing the mutex.
int cached_tables(CopyCache& c, void* const* out, const void* const* in, const size_t* sizes, int n,
                  uint32_t unit, hipStream_t stream, CachedCopy** result) {
  const uint64_t hash = hash_arrays(out, in, sizes, n, unit);
  auto range = c.index.equal_range(hash);
  for (auto it = range.first; it != range.second; ++it) {
    if (!same_arrays(it->second->key, out, in, sizes, n, unit)) continue;
    c.lru.splice(c.lru.begin(), c.lru, it->second);  // iterators into a list survive a splice
    CachedCopy* hit = &c.lru.front();
    // The table was uploaded asynchronously on the stream that built it; another stream
    // must not read it earlier.
    if (!hit->upload_complete) {
      if (hipEventQuery(hit->uploaded) == hipSuccess) {
        hit->upload_complete = true;
      } else {
        (void)hipGetLastError();  // hipErrorNotReady is not an error here
        if (stream != hit->build_stream) HVDHIP_CHECK(hipStreamWaitEvent(stream, hit->uploaded, 0));
      }
    }
    ++c.hits;
    *result = hit;
    return 0;
  }
  std::vector<Seg> segs((size_t)n);
  for (int i = 0; i < n; ++i)
    segs[(size_t)i] = Seg{(uint64_t)(uintptr_t)in[i], (uint64_t)(uintptr_t)out[i], 0, sizes[i] / unit};
  const uint32_t chunk_units = chunk_bytes(Family::kXfer) / unit;
  const uint64_t nchunks = count_chunks(segs, chunk_units);
  if (nchunks == ~0ull) return fail(HVDHIP_ERR_TOO_LARGE, "the copies need more than 2^23 workgroups");
  const size_t bytes = (size_t)table_slots(nchunks) * sizeof(Chunk);
  while (!c.lru.empty() && (c.lru.size() >= c.max_entries || c.bytes + bytes > c.max_bytes)) {
    int rc = evict_one(c);
    if (rc) return rc;
  }
  CachedCopy entry;
  int rc = acquire_buf(c, bytes ? bytes : 32, &entry.buf);
  if (rc) return rc;
  rc = order_event(c, &entry.uploaded);
  hipError_t e = hipSuccess;
  if (rc == 0 && nchunks) {
    fill_chunks(segs, chunk_units, unit, unit, static_cast<Chunk*>(entry.buf.pinned), nchunks);
    e = hipMemcpyAsync(entry.buf.dev, entry.buf.pinned, bytes, hipMemcpyHostToDevice, stream);
  }
  if (rc == 0 && e == hipSuccess) e = hipEventRecord(entry.uploaded, stream);
  if (rc || e != hipSuccess) {
    (void)hipGetLastError();
    if (entry.uploaded) c.idle_events.push_back(entry.uploaded);
    // the copy may have been queued: do not hand the buffers on before the stream is idle
    (void)hipStreamSynchronize(stream);
    keep_buf(c, &entry.buf);
    return rc ? rc : fail((int)e, "staging a copy table failed: %s", hipGetErrorString(e));
  }
  entry.hash = hash;
  entry.key.reserve(2 + 3 * (size_t)n);
  entry.key.push_back((uint64_t)unit);
  entry.key.push_back((uint64_t)n);
  for (int i = 0; i < n; ++i) {
    entry.key.push_back((uint64_t)(uintptr_t)out[i]);
    entry.key.push_back((uint64_t)(uintptr_t)in[i]);
    entry.key.push_back((uint64_t)sizes[i]);
  }
  entry.tables.alloc = nullptr;
  entry.tables.chunks = static_cast<Chunk*>(entry.buf.dev);
  entry.tables.nchunks = (uint32_t)nchunks;
  entry.tables.nlaunch = (uint32_t)table_slots(nchunks);
  entry.build_stream = stream;
  entry.gathers = n > 1;
  for (int i = 0; i + 1 < n && entry.gathers; ++i) {
    const uint64_t end = (uint64_t)(uintptr_t)out[i] + sizes[i], next = (uint64_t)(uintptr_t)out[i + 1];
    entry.gathers = next >= end && next - end < 16;
  }
  c.bytes += entry.buf.cap;
  c.lru.push_front(std::move(entry));
  c.index.emplace(hash, c.lru.begin());
  ++c.misses;
  *result = &c.lru.front();
  return 0;
}

// Notes that `stream` now holds work reading the entry's table.
void mark_used(CachedCopy* entry, hipStream_t stream) {
  for (hipStream_t s : entry->streams)
    if (s == stream) return;
  entry->streams.push_back(stream);
}

int check_arrays(void* const* out, const void* const* in, const size_t* sizes, int n) {
  if (n < 0) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "num_copies is negative");
  if (n > 0 && (!out || !in || !sizes)) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "out, in or sizes is NULL");
  for (int i = 0; i < n; ++i)
    if (sizes[i] && (!out[i] || !in[i]))
      return fail(HVDHIP_ERR_INVALID_ARGUMENT, "copy %d has a NULL pointer with non-zero size", i);
  return 0;
}

}  // namespace

// The stream is idle and about to be destroyed: no table is read on it any more.
void copy_cache_forget_stream(hipStream_t stream) {
  std::vector<CopyCache*> caches;
  {
    CacheRegistry& r = registry();
    std::lock_guard<std::mutex> g(r.mu);
    for (auto& kv : r.by_device) caches.push_back(kv.second);
  }
  for (CopyCache* c : caches) {
    std::lock_guard<std::mutex> g(c->mu);
    for (CachedCopy& e : c->lru) {
      e.streams.erase(std::remove(e.streams.begin(), e.streams.end(), stream), e.streams.end());
      if (e.build_stream == stream) {
        e.build_stream = nullptr;
        e.upload_complete = true;  // the stream was synchronised before this call
      }
    }
  }
}

}  // namespace hvdhip

using namespace hvdhip;

struct hvdhip_fusion_plan {
  int n = 0;
  int device = 0;  // the device that holds the tables
  int tensor_dtype = 0;
  int buffer_dtype = 0;
  int64_t buffer_len = 0;
  std::vector<int64_t> offsets;
  DevTables tables;         // pack, and unpack when both are cut into chunks of the same size
  DevTables unpack_tables;  // unpack, when it prefers another chunk size than pack (the converting plans)
  bool own_unpack_tables = false;
  bool converting = false;
};

extern "C" {

int hvdhip_batched_d2d_memcpy(void* const* out, const void* const* in, const size_t* sizes,
                              int num_copies, void* stream) {
  int rc = check_arrays(out, in, sizes, num_copies);
  if (rc) return rc;
  if (num_copies == 0) return ok();
  hipStream_t s = static_cast<hipStream_t>(stream);
  CachedCopy* entry = nullptr;
  CopyCache* cache = nullptr;
  rc = copy_cache(&cache);
  if (rc) return rc;
  std::lock_guard<std::mutex> g(cache->mu);
  rc = cached_tables(*cache, out, in, sizes, num_copies, 1, s, &entry);
  if (rc) return rc;
  mark_used(entry, s);
  rc = launch_xfer<Copy<uint8_t>, kDirect>(entry->tables, 0, {}, s, entry->gathers);
  return rc ? rc : ok();
}

int hvdhip_batched_scaled_d2d_memcpy(void* const* out, const void* const* in,
                                     const size_t* sizes, int num_copies, double scale_factor,
                                     int dtype, void* stream) {
  int rc = check_arrays(out, in, sizes, num_copies);
  if (rc) return rc;
  if (!scalable(dtype))
    return fail(HVDHIP_ERR_UNSUPPORTED_DTYPE, "dtype %d is not supported by the scaled batched copy", dtype);
  if (num_copies == 0) return ok();
  const uint32_t es = (uint32_t)dtype_size(dtype);
  for (int i = 0; i < num_copies; ++i) {
    if (sizes[i] % es)
      return fail(HVDHIP_ERR_INVALID_ARGUMENT, "size of copy %d is not a multiple of the element size", i);
    if (((uintptr_t)out[i] | (uintptr_t)in[i]) % es)
      return fail(HVDHIP_ERR_INVALID_ARGUMENT, "copy %d is not aligned to its element size", i);
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  CachedCopy* entry = nullptr;
  CopyCache* cache = nullptr;
  rc = copy_cache(&cache);
  if (rc) return rc;
  std::lock_guard<std::mutex> g(cache->mu);
  rc = cached_tables(*cache, out, in, sizes, num_copies, es, s, &entry);
  if (rc) return rc;
  mark_used(entry, s);
  rc = launch_same_dtype<kDirect>(entry->tables, 0, scale_factor, dtype, s, entry->gathers);
  return rc ? rc : ok();
}

int hvdhip_copy_cache_stats(uint64_t* hits, uint64_t* misses, uint64_t* evictions, uint64_t* entries) {
  CopyCache* cache = nullptr;
  int rc = copy_cache(&cache);
  if (rc) return rc;
  std::lock_guard<std::mutex> g(cache->mu);
  if (hits) *hits = cache->hits;
  if (misses) *misses = cache->misses;
  if (evictions) *evictions = cache->evictions;
  if (entries) *entries = (uint64_t)cache->lru.size();
  return ok();
}

int hvdhip_copy_cache_set_limits(uint64_t max_entries, uint64_t max_bytes) {
  if (max_entries == 0) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "max_entries is zero");
  CopyCache* cache = nullptr;
  int rc = copy_cache(&cache);
  if (rc) return rc;
  std::lock_guard<std::mutex> g(cache->mu);
  cache->max_entries = (size_t)max_entries;
  cache->max_bytes = (size_t)max_bytes;
  while (!cache->lru.empty() && (cache->lru.size() > cache->max_entries || cache->bytes > cache->max_bytes)) {
    rc = evict_one(*cache);
    if (rc) return rc;
  }
  return ok();
}

int hvdhip_scale_buffer(const void* fused_input_data, void* buffer_data, int64_t num_elements,
                        double scale_factor, int dtype, void* stream) {
  if (!scalable(dtype))
    return fail(HVDHIP_ERR_UNSUPPORTED_DTYPE, "dtype %d is not supported by ScaleBuffer", dtype);
  if (num_elements < 0) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "num_elements is negative");
  if (num_elements == 0) return ok();
  if (!fused_input_data || !buffer_data) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "buffer is NULL");
  if (((uintptr_t)fused_input_data | (uintptr_t)buffer_data) % (uintptr_t)dtype_size(dtype))
    return fail(HVDHIP_ERR_INVALID_ARGUMENT, "buffer is not aligned to its element size");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const void* in = fused_input_data;
  void* out = buffer_data;
  const int64_t n = num_elements;
  int rc;
  switch (dtype) {
  case HVDHIP_UINT8: rc = launch_contig<Scale<uint8_t, double>>(in, out, n, {scale_factor}, s); break;
  case HVDHIP_INT8: rc = launch_contig<Scale<int8_t, double>>(in, out, n, {scale_factor}, s); break;
  case HVDHIP_INT32: rc = launch_contig<Scale<int32_t, double>>(in, out, n, {scale_factor}, s); break;
  case HVDHIP_INT64: rc = launch_contig<Scale<int64_t, double>>(in, out, n, {scale_factor}, s); break;
  case HVDHIP_FLOAT16: rc = launch_contig<ScaleHalf>(in, out, n, {fp16_scale_factor(scale_factor)}, s); break;
  case HVDHIP_FLOAT32: rc = launch_contig<Scale<float, float>>(in, out, n, {(float)scale_factor}, s); break;
  default: rc = launch_contig<Scale<double, double>>(in, out, n, {scale_factor}, s); break;
  }
  return rc ? rc : ok();
}

int hvdhip_fusion_plan_create(const void* const* tensors, void* const* outputs,
                              const int64_t* num_elements, int n, int tensor_dtype,
                              int buffer_dtype, hvdhip_fusion_plan** plan) {
  if (!plan) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "plan is NULL");
  *plan = nullptr;
  if (n < 0 || (n > 0 && (!tensors || !outputs || !num_elements)))
    return fail(HVDHIP_ERR_INVALID_ARGUMENT, "bad entry arrays");
  const int64_t ts = dtype_size(tensor_dtype);
  const int64_t bs = dtype_size(buffer_dtype);
  if (ts < 0 || bs < 0) return fail(HVDHIP_ERR_UNSUPPORTED_DTYPE, "unknown dtype");
  if (buffer_dtype != tensor_dtype &&
      !(tensor_dtype == HVDHIP_FLOAT32 && buffer_dtype == HVDHIP_FLOAT16))
    return fail(HVDHIP_ERR_UNSUPPORTED_DTYPE,
                "buffer dtype %d with tensor dtype %d: only FLOAT32 tensors in a FLOAT16 buffer convert",
                buffer_dtype, tensor_dtype);
  std::vector<Seg> segs((size_t)n);
  std::vector<int64_t> offsets((size_t)n);
  int64_t off = 0;
  for (int i = 0; i < n; ++i) {
    if (num_elements[i] < 0) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "entry %d has a negative size", i);
    if (num_elements[i] > 0) {
      if (!tensors[i] || !outputs[i]) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "entry %d has a NULL pointer", i);
      if (((uintptr_t)tensors[i] | (uintptr_t)outputs[i]) % (uintptr_t)ts)
        return fail(HVDHIP_ERR_INVALID_ARGUMENT, "entry %d is not aligned to its element size", i);
    }
    offsets[i] = off;
    segs[i] = Seg{(uint64_t)(uintptr_t)tensors[i], (uint64_t)(uintptr_t)outputs[i], (uint64_t)off,
                  (uint64_t)num_elements[i]};
    off += 16 * ((num_elements[i] * bs + 15) / 16);  // ops/gpu_operations.cc:141
  }
  hvdhip_fusion_plan* p = new hvdhip_fusion_plan();
  p->n = n;
  p->tensor_dtype = tensor_dtype;
  p->buffer_dtype = buffer_dtype;
  p->buffer_len = off;
  p->offsets.swap(offsets);
  p->converting = buffer_dtype != tensor_dtype;
  (void)hipGetDevice(&p->device);
  // Chunks are sized on the wider (tensor) side.  The narrowing pack stores only 8 bytes per
  // lane and access and streams best with 8 KiB of fp32 per workgroup; the widening unpack and
  // every same-width transfer with 4 KiB.
  const uint32_t wide = (uint32_t)std::max(ts, bs);
  const uint32_t pack_bytes = p->converting ? chunk_bytes(Family::kXferNarrowing) : chunk_bytes(Family::kXfer);
  const uint32_t unpack_bytes = chunk_bytes(Family::kUnpack);
  int rc = build_tables(segs, pack_bytes / wide, (uint32_t)ts, (uint32_t)bs, &p->tables);
  p->own_unpack_tables = unpack_bytes != pack_bytes;
  if (rc == 0 && p->own_unpack_tables) {
    rc = build_tables(segs, unpack_bytes / wide, (uint32_t)ts, (uint32_t)bs, &p->unpack_tables);
    if (rc) free_tables(&p->tables);
  }
  if (rc) {
    delete p;
    return rc;
  }
  *plan = p;
  return ok();
}

int hvdhip_fusion_plan_destroy(hvdhip_fusion_plan* plan) {
  if (!plan) return ok();
  DeviceGuard on_plan_device(plan->device);
  // Queued kernels may still read the tables.
  HVDHIP_CHECK(hipDeviceSynchronize());
  int rc = free_tables(&plan->tables);
  int rc2 = free_tables(&plan->unpack_tables);
  delete plan;
  if (rc == 0) rc = rc2;
  return rc ? rc : ok();
}

int64_t hvdhip_fusion_plan_buffer_len(const hvdhip_fusion_plan* plan) {
  return plan ? plan->buffer_len : -1;
}

int hvdhip_fusion_plan_offsets(const hvdhip_fusion_plan* plan, int64_t* offsets) {
  if (!plan || (plan->n > 0 && !offsets)) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "plan or offsets is NULL");
  for (int i = 0; i < plan->n; ++i) offsets[i] = plan->offsets[(size_t)i];
  return ok();
}

int64_t hvdhip_fusion_plan_num_chunks(const hvdhip_fusion_plan* plan) {
  return plan ? (int64_t)plan->tables.nchunks : -1;
}

int hvdhip_fusion_pack(hvdhip_fusion_plan* plan, void* fusion_buffer, double scale_factor,
                       unsigned flags, void* stream) {
  if (!plan) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "plan is NULL");
  if (plan->buffer_len > 0 && !fusion_buffer) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "fusion_buffer is NULL");
  if ((uintptr_t)fusion_buffer % 16) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "fusion_buffer must be 16-byte aligned");
  if (flags & ~HVDHIP_PACK_CAST_THEN_SCALE) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "unknown flags 0x%x", flags);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const uint64_t base = (uint64_t)(uintptr_t)fusion_buffer;
  int rc;
  if (plan->buffer_dtype != plan->tensor_dtype) {
    if (flags & HVDHIP_PACK_CAST_THEN_SCALE)
      rc = launch_xfer<PackF32F16CastFirst, kPack>(plan->tables, base, {fp16_scale_factor(scale_factor)}, s);
    else
      rc = launch_xfer<PackF32F16, kPack>(plan->tables, base, {(float)scale_factor}, s);
  } else {
    if (flags) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "HVDHIP_PACK_CAST_THEN_SCALE needs a converting plan");
    if (scale_factor != 1.0 && !scalable(plan->tensor_dtype))
      return fail(HVDHIP_ERR_UNSUPPORTED_DTYPE, "dtype %d cannot be scaled", plan->tensor_dtype);
    rc = launch_same_dtype<kPack>(plan->tables, base, scale_factor, plan->tensor_dtype, s);
  }
  return rc ? rc : ok();
}

namespace {
int unpack(hvdhip_fusion_plan* plan, const void* fusion_buffer, double scale_factor, void* stream,
           hipEvent_t completion) {
  if (!plan) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "plan is NULL");
  if (plan->buffer_len > 0 && !fusion_buffer) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "fusion_buffer is NULL");
  if ((uintptr_t)fusion_buffer % 16) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "fusion_buffer must be 16-byte aligned");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const uint64_t base = (uint64_t)(uintptr_t)fusion_buffer;
  int rc;
  if (plan->buffer_dtype != plan->tensor_dtype) {
    rc = launch_xfer<UnpackF16F32, kUnpack>(plan->own_unpack_tables ? plan->unpack_tables : plan->tables, base,
                                            {fp16_scale_factor(scale_factor)}, s, false, completion);
  } else {
    if (scale_factor != 1.0 && !scalable(plan->tensor_dtype))
      return fail(HVDHIP_ERR_UNSUPPORTED_DTYPE, "dtype %d cannot be scaled", plan->tensor_dtype);
    rc = launch_same_dtype<kUnpack>(plan->own_unpack_tables ? plan->unpack_tables : plan->tables, base, scale_factor,
                                    plan->tensor_dtype, s, false, completion);
  }
  return rc ? rc : ok();
}
}  // namespace

int hvdhip_fusion_unpack(hvdhip_fusion_plan* plan, const void* fusion_buffer,
                         double scale_factor, void* stream) {
  return unpack(plan, fusion_buffer, scale_factor, stream, nullptr);
}

int hvdhip_fusion_unpack_record(hvdhip_fusion_plan* plan, const void* fusion_buffer,
                                double scale_factor, void* stream, void* event) {
  if (!event) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "event is NULL");
  return unpack(plan, fusion_buffer, scale_factor, stream, static_cast<hipEvent_t>(event));
}

}  // extern "C"
