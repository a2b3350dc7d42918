// reduce.hip -- the local reduce-sum: resident[i] += incoming[i], one GPU's
// share of a reduce-scatter.  gfx950 only.
//
// The arithmetic is the element-wise sum that the collective applies in the
// reference (ncclSum ops/nccl_operations.cc:190-193, gloo::sum<T>
// ops/gloo_operations.cc:66-74, MPI_SUM / float16_sum common/half.cc:44-76):
// one IEEE add for f32/f64, fp16 through an fp32 add rounded to nearest even,
// wrapping adds for integers.  The k-way form rounds to the element type
// after every peer, in peer order, so it equals k successive two-way sums
// while reading the resident chunk once and writing it once.
//
// Pure streaming: 16-byte accesses per lane, all loads of an iteration in
// flight before the first add; no LDS, no matrix cores.
#include "internal.h"
#include "vecmem.h"

namespace hvdhip {
namespace {

template <typename T>
struct Add {
  static __device__ __forceinline__ T f(T r, T x) { return (T)(r + x); }
};
// float16_sum, common/half.cc:68-75: widen both, add in fp32, round to half.
template <>
struct Add<half_t> {
  static __device__ __forceinline__ half_t f(half_t r, half_t x) {
    return (half_t)opaque((float)r + (float)x);
  }
};

// acc += x for one 16-byte vector.
template <typename T, int VEC>
__device__ __forceinline__ void accumulate(Arr<T, VEC>& acc, const Arr<T, VEC>& x) {
#pragma unroll
  for (int j = 0; j < VEC; ++j) acc.v[j] = Add<T>::f(acc.v[j], x.v[j]);
}
// Sixteen wrapping byte sums as four word operations each: the low seven bits of every byte
// add without a carry into the neighbour, the top bit is the exclusive or of the three
// inputs (both top bits and the carry out of bit 6).
template <>
__device__ __forceinline__ void accumulate<uint8_t, 16>(Arr<uint8_t, 16>& acc, const Arr<uint8_t, 16>& x) {
  uint32_t a[4], b[4];
  __builtin_memcpy(a, acc.v, 16);
  __builtin_memcpy(b, x.v, 16);
#pragma unroll
  for (int w = 0; w < 4; ++w)
    a[w] = ((a[w] & 0x7f7f7f7fu) + (b[w] & 0x7f7f7f7fu)) ^ ((a[w] ^ b[w]) & 0x80808080u);
  __builtin_memcpy(acc.v, a, 16);
}

constexpr int kMaxK = 8;  // peers per launch; more are folded in by further launches

template <int K>
struct Peers {
  const void* p[K];
};

constexpr int kUnroll = 2;

// Workgroup b accumulates K peers into tile t = xcd_tile(b), elements [t*tile, (t+1)*tile).
template <typename T, int K, bool WT>
__global__ __launch_bounds__(kWG) void reduce_k(T* resident, Peers<K> peers, uint64_t n,
                                                uint32_t tile, uint32_t run) {
  constexpr int VEC = 16 / (int)sizeof(T);
  typedef Arr<T, VEC> V;
  const uint64_t start = (uint64_t)xcd_tile(blockIdx.x, gridDim.x, run) * tile;
  const uint64_t left = n - start;
  const uint32_t m = left < tile ? (uint32_t)left : tile;
  gptr<T> r = as_global(resident + start);
  gptr<const T> in[K];
#pragma unroll
  for (int k = 0; k < K; ++k) in[k] = as_global(static_cast<const T*>(peers.p[k]) + start);
  const uint32_t nv = m / VEC;
  const Window out = store_window<WT>(r, m * (uint32_t)sizeof(T));
  constexpr bool kBytes = sizeof(T) == 1;  // byte elements are read through windows (vecmem.h)
  ReadWindow rin, pin[K];
  if constexpr (kBytes) {
    rin = load_window(gptr<const T>(r), m);
#pragma unroll
    for (int k = 0; k < K; ++k) pin[k] = load_window(in[k], m);
  }
  auto load_resident = [&](uint32_t vec) {
    if constexpr (kBytes) {
      return ldw<T, VEC>(rin, vec * 16u);
    } else {
      return ldv<T, VEC>(r + (size_t)vec * VEC);
    }
  };
  auto load_peer = [&](int k, uint32_t vec) {
    if constexpr (kBytes) {
      return ldw<T, VEC>(pin[k], vec * 16u);
    } else {
      return ldv<T, VEC>(in[k] + (size_t)vec * VEC);
    }
  };
  uint32_t v = threadIdx.x;
  for (; v + (kUnroll - 1) * kWG < nv; v += kUnroll * kWG) {
    V acc[kUnroll];
    V x[kUnroll][K];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      acc[u] = load_resident(v + u * kWG);
#pragma unroll
      for (int k = 0; k < K; ++k) x[u][k] = load_peer(k, v + u * kWG);
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
#pragma unroll
      for (int k = 0; k < K; ++k) accumulate<T, VEC>(acc[u], x[u][k]);
      stw<WT, T, VEC>(out, (v + u * kWG) * 16u, acc[u]);
    }
  }
  for (; v < nv; v += kWG) {
    V acc = load_resident(v);
#pragma unroll
    for (int k = 0; k < K; ++k) {
      accumulate<T, VEC>(acc, load_peer(k, v));
    }
    stw<WT, T, VEC>(out, v * 16u, acc);
  }
  const uint32_t t = nv * VEC + threadIdx.x;
  if (t < m) {
    T acc = r[t];
#pragma unroll
    for (int k = 0; k < K; ++k) acc = Add<T>::f(acc, in[k][t]);
    r[t] = acc;
  }
}

template <typename T, int K>
int launch_k(void* resident, const void* const* incoming, int64_t n, hipStream_t stream) {
  const uint32_t tile = chunk_bytes(Family::kReduce) / (uint32_t)sizeof(T);
  uint64_t done = 0, left = (uint64_t)n;
  while (left > 0) {  // one launch unless the chunk needs more than kMaxWorkgroups workgroups
    const uint64_t slice = left < kMaxWorkgroups * tile ? left : kMaxWorkgroups * tile;
    const uint32_t blocks = (uint32_t)((slice + tile - 1) / tile);
    Peers<K> peers;
    for (int k = 0; k < K; ++k) peers.p[k] = static_cast<const T*>(incoming[k]) + done;
    if (write_through(K <= 2 ? Stores::kReduceFew : Stores::kReduceMany))
      launch(reduce_k<T, K, true>, blocks, stream, static_cast<T*>(resident) + done,
                         peers, slice, tile, xcd_shift(blocks, tile * (uint32_t)sizeof(T)));
    else
      launch(reduce_k<T, K, false>, blocks, stream, static_cast<T*>(resident) + done,
                         peers, slice, tile, xcd_shift(blocks, tile * (uint32_t)sizeof(T)));
    HVDHIP_CHECK_LAUNCH("reduce_k");
    done += slice;
    left -= slice;
  }
  return 0;
}

template <typename T>
int launch_t(void* resident, const void* const* incoming, int k, int64_t n, hipStream_t stream) {
  while (k > 0) {
    int rc;
    int step = k < kMaxK ? k : kMaxK;
    switch (step) {
    case 1: rc = launch_k<T, 1>(resident, incoming, n, stream); break;
    case 2: rc = launch_k<T, 2>(resident, incoming, n, stream); break;
    case 3: rc = launch_k<T, 3>(resident, incoming, n, stream); break;
    case 4: rc = launch_k<T, 4>(resident, incoming, n, stream); break;
    case 5: rc = launch_k<T, 5>(resident, incoming, n, stream); break;
    case 6: rc = launch_k<T, 6>(resident, incoming, n, stream); break;
    case 7: rc = launch_k<T, 7>(resident, incoming, n, stream); break;
    default: rc = launch_k<T, 8>(resident, incoming, n, stream); break;
    }
    if (rc) return rc;
    incoming += step;
    k -= step;
  }
  return 0;
}

}  // namespace
}  // namespace hvdhip

using namespace hvdhip;

extern "C" {

int hvdhip_reduce_sum_k(void* resident, const void* const* incoming, int k, int64_t num_elements,
                        int dtype, void* stream) {
  if (k < 1 || k > 16) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "k = %d is outside 1..16", k);
  if (num_elements < 0) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "num_elements is negative");
  const int64_t es = dtype_size(dtype);
  if (es < 0 || dtype == HVDHIP_BOOL)
    return fail(HVDHIP_ERR_UNSUPPORTED_DTYPE, "dtype %d cannot be summed", dtype);
  if (num_elements == 0) return ok();
  if (!resident || !incoming) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "resident or incoming is NULL");
  uintptr_t bits = (uintptr_t)resident;
  for (int i = 0; i < k; ++i) {
    if (!incoming[i]) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "incoming[%d] is NULL", i);
    bits |= (uintptr_t)incoming[i];
  }
  if (bits % (uintptr_t)es) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "chunk is not aligned to its element size");
  hipStream_t s = static_cast<hipStream_t>(stream);
  int rc;
  switch (dtype) {
  // Wrapping integer sums are the same bits for signed and unsigned.
  case HVDHIP_UINT8: case HVDHIP_INT8: rc = launch_t<uint8_t>(resident, incoming, k, num_elements, s); break;
  case HVDHIP_UINT16: case HVDHIP_INT16: rc = launch_t<uint16_t>(resident, incoming, k, num_elements, s); break;
  case HVDHIP_INT32: rc = launch_t<uint32_t>(resident, incoming, k, num_elements, s); break;
  case HVDHIP_INT64: rc = launch_t<uint64_t>(resident, incoming, k, num_elements, s); break;
  case HVDHIP_FLOAT16: rc = launch_t<half_t>(resident, incoming, k, num_elements, s); break;
  case HVDHIP_FLOAT32: rc = launch_t<float>(resident, incoming, k, num_elements, s); break;
  default: rc = launch_t<double>(resident, incoming, k, num_elements, s); break;
  }
  return rc ? rc : ok();
}

int hvdhip_reduce_sum(void* resident, const void* incoming, int64_t num_elements, int dtype,
                      void* stream) {
  const void* one[1] = {incoming};
  if (!incoming && num_elements > 0) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "incoming is NULL");
  return hvdhip_reduce_sum_k(resident, one, 1, num_elements, dtype, stream);
}

}  // extern "C"
