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
// Pure streaming: 16-byte accesses per lane, all loads of a tile in flight
// before the first add; no LDS, no matrix cores.
#include "internal.h"
#include "vecmem.h"

namespace hvdhip {
namespace {

template <typename T>
struct Add {
  static __device__ __forceinline__ T f(T r, T x) { return (T)(r + x); }
};
// float16_sum, common/half.cc:68-75: widen both, add in fp32, round to half.  The fp32 sum of two
// halves carries 24 bits, at least 2 * 11 + 2, so rounding it to half equals rounding the exact sum
// once: the correctly rounded half-precision add gives the same bits (subnormals included; the
// kernels run with fp16 denormals on and round to nearest even), and it adds two elements per
// instruction where the fp32 route takes four instructions per element.
template <>
struct Add<half_t> {
  static __device__ __forceinline__ half_t f(half_t r, half_t x) { return (half_t)(r + x); }
};

// acc += x for one 16-byte vector.
template <typename T, int VEC>
__device__ __forceinline__ void accumulate(Arr<T, VEC>& acc, const Arr<T, VEC>& x) {
#pragma unroll
  for (int j = 0; j < VEC; ++j) acc.v[j] = Add<T>::f(acc.v[j], x.v[j]);
}
// Eight half sums as four packed adds.
template <>
__device__ __forceinline__ void accumulate<half_t, 8>(Arr<half_t, 8>& acc, const Arr<half_t, 8>& x) {
  typedef half_t h2 __attribute__((ext_vector_type(2)));
  h2 a[4], b[4];
  __builtin_memcpy(a, acc.v, 16);
  __builtin_memcpy(b, x.v, 16);
#pragma unroll
  for (int w = 0; w < 4; ++w) a[w] = a[w] + b[w];
  __builtin_memcpy(acc.v, a, 16);
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

// Workgroup b accumulates K peers into tile t = xcd_tile(b), elements [t*tile, (t+1)*tile).
//
// A chunk of a few MiB (one GPU's share of a reduce-scatter) is a grid that the device holds all at
// once, so whatever a workgroup does before its first load is paid in full by the launch.  The
// arguments are therefore plain scalars in an order that lets the command processor hand the first
// fourteen dwords over in registers (resident, n, tile, the tile order, the first three peers; a struct
// of pointers would not be preloaded), the rest arrives with one scalar load, and no branch stands
// between a workgroup's start and its loads: with the prologue of three dependent scalar loads and
// two branches that this replaces, the 7-peer sum of an 8 MiB chunk took 14.5 instead of 12.6 us.
template <typename T, int K, int ST>
__global__ __launch_bounds__(kWG) void reduce_k(T* resident, uint64_t n, uint32_t tile, uint32_t shift,
                                                uint32_t ordered, uint32_t, const T* p0, const T* p1,
                                                const T* p2, const T* p3, const T* p4, const T* p5,
                                                const T* p6, const T* p7) {
  constexpr int VEC = 16 / (int)sizeof(T);
  typedef Arr<T, VEC> V;
  const T* const ps[kMaxK] = {p0, p1, p2, p3, p4, p5, p6, p7};
  const uint64_t start = (uint64_t)xcd_tile(blockIdx.x, XcdOrder{shift, ordered}) * tile;
  const uint64_t left = n - start;
  const uint32_t m = left < tile ? (uint32_t)left : tile;
  gptr<T> r = as_global(resident + start);
  gptr<const T> in[K];
#pragma unroll
  for (int k = 0; k < K; ++k) in[k] = as_global(ps[k] + start);
  const uint32_t nv = m / VEC;
  const Window out = store_window<ST>(r, m * (uint32_t)sizeof(T));
  constexpr bool kBytes = sizeof(T) == 1;  // byte elements are read through windows (vecmem.h)
  ReadWindow rin, pin[K];
  if constexpr (kBytes) {
    rin = load_window(gptr<const T>(r), m);
#pragma unroll
    for (int k = 0; k < K; ++k) pin[k] = load_window(in[k], m);
  }
  // One 16-byte vector per lane and stream for a tile of the standard size: K + 1 loads in flight
  // per lane, then the sums in peer order, then one store.
  for (uint32_t v = threadIdx.x; v < nv; v += kWG) {
    V acc, x[K];
    if constexpr (kBytes) {
      acc = ldw<T, VEC>(rin, v * 16u);
#pragma unroll
      for (int k = 0; k < K; ++k) x[k] = ldw<T, VEC>(pin[k], v * 16u);
    } else {
      acc = ldv<T, VEC>(r + (size_t)v * VEC);
#pragma unroll
      for (int k = 0; k < K; ++k) x[k] = ldv<T, VEC>(in[k] + (size_t)v * VEC);
    }
#pragma unroll
    for (int k = 0; k < K; ++k) accumulate<T, VEC>(acc, x[k]);
    stw<ST, T, VEC>(out, v * 16u, acc);
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
    const T* p[kMaxK];
    for (int k = 0; k < kMaxK; ++k) p[k] = k < K ? static_cast<const T*>(incoming[k]) + done : nullptr;
    const XcdOrder order = xcd_order(blocks, tile * (uint32_t)sizeof(T));
    const hipError_t status = with_store_policy(K <= 2 ? Stores::kReduceFew : Stores::kReduceMany, [&](auto st) {
      return launch(reduce_k<T, K, decltype(st)::value>, blocks, stream, static_cast<T*>(resident) + done, slice,
                    tile, order.shift, order.ordered, 0u, p[0], p[1], p[2], p[3], p[4], p[5], p[6], p[7]);
    });
    HVDHIP_CHECK_LAUNCH("reduce_k", status);
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
