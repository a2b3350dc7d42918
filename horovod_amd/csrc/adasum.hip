// adasum.hip -- Adasum's pairwise combine on one device: per-layer dot
// product and squared norms accumulated in double, the coefficient formula,
// and the fused scaled add.  gfx950 only.
//
// Follows Adasum<Comm>::FusedPairwiseReduceWithComm, ops/adasum/adasum.h:344-410,
// with ComputeDotAndNormSqrds (:413-426) and ScaledAdd (:429-435); in the
// reference all of it runs on the host.
//
// Pass 1 (dot_partials_k): one workgroup per chunk of a layer.  Each lane
// streams 16-byte pieces of a and b, widens to double and keeps two
// independent fma chains per sum; lanes combine with wave64 DPP adds, the four
// wavefronts through LDS, and the workgroup writes one {dot, |a|^2, |b|^2}
// triple.  Pass 1b (finalize_k): one workgroup per layer adds that layer's
// triples in a fixed order and evaluates the coefficients.  No floating-point
// atomics anywhere, so results are identical from run to run.
// Pass 2 (scaled_add_k): one workgroup per chunk, a = ca*a + cb*b in double,
// rounded once.  In the combine, when no layer has more than 512 triples, pass 2
// does pass 1b's work itself (every workgroup re-adds its layer's triples in that
// same fixed order under the shadow of its data loads) and pass 1b is not launched.
//
// Products of two fp32 (or fp16) values are exact in double, so only the
// order of the double additions differs from the reference's sequential
// loop.  Bandwidth-bound: 3 double fmas per 8 bytes read in pass 1.
#include <cfloat>
#include <cmath>
#include <list>
#include <mutex>

#include "internal.h"
#include "vecmem.h"

namespace hvdhip {
namespace {

// Chunk table entry as used here: tensor = index of the chunk's first element
// in the vectors, output = layer number in the low and the layer's first partial
// triple in the high 32 bits, off = the chunk's number in layer order (the slot of
// its partial triple; the table itself is in XCD order), n = elements in the chunk,
// pad = number of partial triples of the layer.  With its layer's entry folded in,
// a workgroup needs no second dependent load to find its layer's partial sums.
//
// Layer table entry: first partial triple of the layer and how many it has.
struct Layer {
  uint32_t first;
  uint32_t count;
};

struct Triple {
  double d, a, b;
};

// x + (x of the lane that the DPP control CTRL names), for the rows in ROW_MASK; lanes without a
// source (or outside the mask) add zero.  Two 32-bit DPP moves and one add: data-parallel
// primitives move data between lanes inside the vector ALU, where a shuffle goes through the LDS
// crossbar and costs a memory-pipeline round trip per step.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ double dpp_add(double x) {
  const int lo = __double2loint(x), hi = __double2hiint(x);
  const int lo2 = __builtin_amdgcn_update_dpp(0, lo, CTRL, ROW_MASK, 0xf, false);
  const int hi2 = __builtin_amdgcn_update_dpp(0, hi, CTRL, ROW_MASK, 0xf, false);
  return x + __hiloint2double(hi2, lo2);
}

// Sum over the 64 lanes of a wavefront in a fixed order; the total arrives in lane 63.  Within
// each row of 16 lanes a shifted-add scan (by 1, 2, 4, 8), then lane 15 of rows 0 and 2 into rows
// 1 and 3, then lane 31 into rows 2 and 3.
__device__ __forceinline__ double wave_sum(double x) {
  x = dpp_add<0x111, 0xf>(x);  // row_shr:1
  x = dpp_add<0x112, 0xf>(x);  // row_shr:2
  x = dpp_add<0x114, 0xf>(x);  // row_shr:4
  x = dpp_add<0x118, 0xf>(x);  // row_shr:8
  x = dpp_add<0x142, 0xa>(x);  // row_bcast:15 into rows 1 and 3
  x = dpp_add<0x143, 0xc>(x);  // row_bcast:31 into rows 2 and 3
  return x;
}

__device__ __forceinline__ Triple wg_reduce(Triple t) {
  // wave64 sums, then the four wavefronts in order through LDS
  t.d = wave_sum(t.d);
  t.a = wave_sum(t.a);
  t.b = wave_sum(t.b);
  __shared__ double red[3][kWG / 64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 63) {
    red[0][wave] = t.d;
    red[1][wave] = t.a;
    red[2][wave] = t.b;
  }
  __syncthreads();
  Triple r = {0., 0., 0.};
  if (threadIdx.x == 0) {
#pragma unroll
    for (int w = 0; w < kWG / 64; ++w) {
      r.d += red[0][w];
      r.a += red[1][w];
      r.b += red[2][w];
    }
  }
  return r;  // valid in thread 0
}

constexpr int kUnroll = 4;

// KEEP: which vectors the loads leave in the Infinity Cache for the scaled add that follows
// (1 a, 2 a and b; chosen by the host by what fits there).
template <typename T, int KEEP>
__global__ __launch_bounds__(kWG) void dot_partials_k(const Chunk* __restrict__ chunks,
                                                      const T* __restrict__ a,
                                                      const T* __restrict__ b,
                                                      double* __restrict__ partials) {
  constexpr int VEC = 16 / (int)sizeof(T);
  typedef Arr<T, VEC> V;
  const Chunk c = chunks[blockIdx.x];
  const uint32_t n = c.n;
  gptr<const T> pa = as_global(a + c.tensor);
  gptr<const T> pb = as_global(b + c.tensor);
  const uint32_t nv = n / VEC;
  double d0 = 0., d1 = 0., a0 = 0., a1 = 0., b0 = 0., b1 = 0.;
  uint32_t v = threadIdx.x;
  for (; v + (kUnroll - 1) * kWG < nv; v += kUnroll * kWG) {
    V x[kUnroll], y[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      x[u] = ldv<T, VEC, false>(pa + (size_t)(v + u * kWG) * VEC);
      y[u] = ldv<T, VEC, KEEP != 2>(pb + (size_t)(v + u * kWG) * VEC);
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
#pragma unroll
      for (int j = 0; j < VEC; j += 2) {
        const double p = (double)x[u].v[j], q = (double)y[u].v[j];
        d0 = fma(p, q, d0);
        a0 = fma(p, p, a0);
        b0 = fma(q, q, b0);
        if (j + 1 < VEC) {
          const double r = (double)x[u].v[j + 1], s = (double)y[u].v[j + 1];
          d1 = fma(r, s, d1);
          a1 = fma(r, r, a1);
          b1 = fma(s, s, b1);
        }
      }
    }
  }
  for (; v < nv; v += kWG) {
    const V x = ldv<T, VEC, false>(pa + (size_t)v * VEC), y = ldv<T, VEC, KEEP != 2>(pb + (size_t)v * VEC);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const double p = (double)x.v[j], q = (double)y.v[j];
      d0 = fma(p, q, d0);
      a0 = fma(p, p, a0);
      b0 = fma(q, q, b0);
    }
  }
  const uint32_t t = nv * VEC + threadIdx.x;
  if (t < n) {
    const double p = (double)pa[t], q = (double)pb[t];
    d1 = fma(p, q, d1);
    a1 = fma(p, p, a1);
    b1 = fma(q, q, b1);
  }
  Triple r = wg_reduce(Triple{d0 + d1, a0 + a1, b0 + b1});
  if (threadIdx.x == 0) {
    partials[3 * c.off + 0] = r.d;  // c.off: the chunk's number in layer order, whatever workgroup has it
    partials[3 * c.off + 1] = r.a;
    partials[3 * c.off + 2] = r.b;
  }
}

// Coefficients of adasum.h:397-404 from a layer's sums.
__device__ __forceinline__ void layer_coeffs(const Triple& r, double guard, double* ca, double* cb) {
  *ca = 1.;
  *cb = 1.;
  if (r.a >= guard) *ca = 1.0 - r.d / r.a * 0.5;
  if (r.b >= guard) *cb = 1.0 - r.d / r.b * 0.5;
}

// One workgroup per layer: sums the layer's partial triples in a fixed order,
// stores {dot, |a|^2, |b|^2} and the coefficients of adasum.h:397-404.
__global__ __launch_bounds__(kWG) void finalize_k(const Layer* __restrict__ layers,
                                                  const double* __restrict__ partials,
                                                  double* __restrict__ normdots,
                                                  double* __restrict__ coeffs, double guard) {
  const Layer L = layers[blockIdx.x];
  const uint64_t first = L.first, count = L.count;
  Triple t = {0., 0., 0.};
  // A lane adds triples lane, lane + kWG, lane + 2 kWG ... in that order; eight are fetched at a
  // time so that a layer of thousands of chunks (one workgroup reads them all) does not pay one
  // memory round trip per step.
  constexpr int kAhead = 8;
  uint64_t i = threadIdx.x;
  for (; i + (kAhead - 1) * kWG < count; i += kAhead * kWG) {
    double v[kAhead][3];
#pragma unroll
    for (int u = 0; u < kAhead; ++u) {
#pragma unroll
      for (int j = 0; j < 3; ++j) v[u][j] = partials[3 * (first + i + (uint64_t)u * kWG) + j];
    }
#pragma unroll
    for (int u = 0; u < kAhead; ++u) {
      t.d += v[u][0];
      t.a += v[u][1];
      t.b += v[u][2];
    }
  }
  for (; i < count; i += kWG) {
    t.d += partials[3 * (first + i) + 0];
    t.a += partials[3 * (first + i) + 1];
    t.b += partials[3 * (first + i) + 2];
  }
  Triple r = wg_reduce(t);
  if (threadIdx.x == 0) {
    normdots[3 * (uint64_t)blockIdx.x + 0] = r.d;
    normdots[3 * (uint64_t)blockIdx.x + 1] = r.a;
    normdots[3 * (uint64_t)blockIdx.x + 2] = r.b;
    double ca, cb;
    layer_coeffs(r, guard, &ca, &cb);
    coeffs[2 * (uint64_t)blockIdx.x + 0] = ca;
    coeffs[2 * (uint64_t)blockIdx.x + 1] = cb;
  }
}

// ScaledAdd<T>, adasum.h:429-435: acoeff * a[i] + bcoeff * b[i] with the operands widened to
// double: two rounded products, their rounded sum, then the conversion to T.  Contraction is
// switched off for this expression (device code contracts by default, and the rounded-operation
// intrinsics are plain operators to the compiler), so no product is fused into the sum.
template <typename T>
struct Axpby {
  static __device__ __forceinline__ T f(double ca, T a, double cb, T b) {
#pragma clang fp contract(off)
    const double pa = ca * (double)a, pb = cb * (double)b;
    return (T)(pa + pb);
  }
};
// ScaledAddfp16, adasum.h:482-500: float coefficients, t = ca*a rounded to fp32, r = fma(cb, b, t)
// rounded to fp32, then to half.  Both fp32 results are kept apart from what follows them: a fused
// mixed-precision product would take a +0 addend and lose the sign of a -0 product, and a fused
// fma-and-narrow rounds the exact sum once where fmadd_ps followed by cvtps_ph rounds twice
// (it differs from the reference in the last bit of some elements).  The widening of b folds
// into the fma, and pairs of results narrow with one packed conversion.
template <>
struct Axpby<half_t> {
  static __device__ __forceinline__ half_t f(double ca, half_t a, double cb, half_t b) {
    const float t = opaque(__fmul_rn((float)ca, (float)a));
    return (half_t)opaque(__fmaf_rn((float)cb, (float)b, t));
  }
};

// FUSED = false: the coefficients come from `coeffs` (or, when that is null, from the
// by-value pair).
// FUSED = true (the combine, when no layer has more than 2*kWG partial triples): every
// workgroup sums its layer's triples itself, in exactly the order finalize_k uses, while its
// data loads are in flight, which saves the finalize launch between the two passes.  All
// workgroups of a layer execute the same additions in the same order, so they agree to the
// bit; the layer's first workgroup also stores the sums and coefficients for readers.
template <typename T, bool FUSED, int ST>
__global__ __launch_bounds__(kWG) void scaled_add_k(const Chunk* __restrict__ chunks, T* a,
                                                    const T* __restrict__ b,
                                                    const double* __restrict__ coeffs,
                                                    double ca_arg, double cb_arg,
                                                    const Layer* __restrict__ layers,
                                                    const double* __restrict__ partials,
                                                    double* __restrict__ normdots,
                                                    double* __restrict__ coeffs_out, double guard,
                                                    uint32_t nlayers) {
  constexpr int VEC = 16 / (int)sizeof(T);
  typedef Arr<T, VEC> V;
  const Chunk c = chunks[blockIdx.x];
  const uint32_t n = c.n;
  gptr<T> pa = as_global(a + c.tensor);
  gptr<const T> pb = as_global(b + c.tensor);
  const uint32_t nv = n / VEC;
  const Window out = store_window<ST>(pa, n * (uint32_t)sizeof(T));
  uint32_t v = threadIdx.x;
  double ca, cb;
  const uint32_t layer = (uint32_t)c.output;
  if (FUSED) {
    const Layer L = {(uint32_t)(c.output >> 32), c.pad};
    // this lane's share of the layer's triples first, the data loads right behind them: loads
    // return in order, so the sums below wait for the triples only.  The triple loads are
    // unconditional (a lane beyond the layer's count re-reads the last triple and drops it), so
    // that nothing waits for them before the data loads are out.
    const uint32_t last = L.count - 1;  // a chunk's layer has at least this chunk's triple
    const uint64_t i0 = 3 * ((uint64_t)L.first + (threadIdx.x < last ? threadIdx.x : last));
    const uint64_t i1 = 3 * ((uint64_t)L.first + (threadIdx.x + kWG < last ? threadIdx.x + kWG : last));
    const Triple r0 = {partials[i0], partials[i0 + 1], partials[i0 + 2]};
    const Triple r1 = {partials[i1], partials[i1 + 1], partials[i1 + 2]};
    const bool full = v + (kUnroll - 1) * kWG < nv;
    V x[kUnroll], y[kUnroll];
    if (full) {
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        x[u] = ldv<T, VEC>(pa + (size_t)(v + u * kWG) * VEC);
        y[u] = ldv<T, VEC>(pb + (size_t)(v + u * kWG) * VEC);
      }
    }
    const bool in0 = threadIdx.x < L.count, in1 = threadIdx.x + kWG < L.count;
    const Triple t0 = {in0 ? r0.d : 0., in0 ? r0.a : 0., in0 ? r0.b : 0.};
    const Triple t1 = {in1 ? r1.d : 0., in1 ? r1.a : 0., in1 ? r1.b : 0.};
    Triple t = {0., 0., 0.};
    t.d += t0.d; t.a += t0.a; t.b += t0.b;  // the order of finalize_k: i = lane, lane + kWG
    t.d += t1.d; t.a += t1.a; t.b += t1.b;
    const Triple r = wg_reduce(t);
    __shared__ double cc[2];
    if (threadIdx.x == 0) {
      layer_coeffs(r, guard, &ca, &cb);
      cc[0] = ca;
      cc[1] = cb;
      if (c.off == L.first) {
        normdots[3 * (uint64_t)layer + 0] = r.d;
        normdots[3 * (uint64_t)layer + 1] = r.a;
        normdots[3 * (uint64_t)layer + 2] = r.b;
        coeffs_out[2 * (uint64_t)layer + 0] = ca;
        coeffs_out[2 * (uint64_t)layer + 1] = cb;
      }
    }
    if (blockIdx.x == 0) {
      // layers without elements have no workgroup of their own: sums 0, coefficients 1
      for (uint32_t l = threadIdx.x; l < nlayers; l += kWG) {
        if (layers[l].count == 0) {
          normdots[3 * (uint64_t)l + 0] = 0.;
          normdots[3 * (uint64_t)l + 1] = 0.;
          normdots[3 * (uint64_t)l + 2] = 0.;
          coeffs_out[2 * (uint64_t)l + 0] = 1.;
          coeffs_out[2 * (uint64_t)l + 1] = 1.;
        }
      }
    }
    __syncthreads();
    ca = cc[0];
    cb = cc[1];
    if (full) {
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) x[u].v[j] = Axpby<T>::f(ca, x[u].v[j], cb, y[u].v[j]);
        stw<ST, T, VEC>(out, (v + u * kWG) * 16u, x[u]);
      }
      v += kUnroll * kWG;
    }
  } else {
    // coeffs == nullptr: every layer uses the by-value pair (ca_arg, cb_arg).
    ca = coeffs ? coeffs[2 * (uint64_t)layer] : ca_arg;
    cb = coeffs ? coeffs[2 * (uint64_t)layer + 1] : cb_arg;
  }
  for (; v + (kUnroll - 1) * kWG < nv; v += kUnroll * kWG) {
    V x[kUnroll], y[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      x[u] = ldv<T, VEC>(pa + (size_t)(v + u * kWG) * VEC);
      y[u] = ldv<T, VEC>(pb + (size_t)(v + u * kWG) * VEC);
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) x[u].v[j] = Axpby<T>::f(ca, x[u].v[j], cb, y[u].v[j]);
      stw<ST, T, VEC>(out, (v + u * kWG) * 16u, x[u]);
    }
  }
  for (; v < nv; v += kWG) {
    V x = ldv<T, VEC>(pa + (size_t)v * VEC);
    const V y = ldv<T, VEC>(pb + (size_t)v * VEC);
#pragma unroll
    for (int j = 0; j < VEC; ++j) x.v[j] = Axpby<T>::f(ca, x.v[j], cb, y.v[j]);
    stw<ST, T, VEC>(out, v * 16u, x);
  }
  const uint32_t t = nv * VEC + threadIdx.x;
  if (t < n) pa[t] = Axpby<T>::f(ca, pa[t], cb, pb[t]);
}

// Writes the chunk and layer tables of a single layer of `count` elements, as
// hvdhip_adasum_plan_create lays them out for one layer: chunk c starts at element
// c * chunk_units and sits at table position xcd_slot(c).
__global__ __launch_bounds__(kWG) void one_layer_tables_k(Chunk* __restrict__ chunks,
                                                          Layer* __restrict__ layer, uint32_t nchunks,
                                                          uint64_t count, uint32_t chunk_units,
                                                          uint32_t run) {
  const uint32_t c = blockIdx.x * kWG + threadIdx.x;
  if (c == 0) *layer = Layer{0, nchunks};
  if (c >= nchunks) return;
  const uint64_t start = (uint64_t)c * chunk_units;
  const uint64_t left = count - start;
  chunks[xcd_slot(c, nchunks, run)] =
      Chunk{start, 0, (uint64_t)c, (uint32_t)(left < chunk_units ? left : chunk_units), nchunks};
}

// Scratch of hvdhip_adasum_combine_static: the tables and partial sums that a plan would hold in
// memory it allocates.  One copy per device, for the life of the process.
constexpr uint32_t kStaticMaxChunks = 16384;  // 256 MiB per vector at 16 KiB per chunk
constexpr size_t kStaticChunksOff = 0;
constexpr size_t kStaticPartialsOff = kStaticChunksOff + (size_t)kStaticMaxChunks * sizeof(Chunk);
constexpr size_t kStaticResultsOff = kStaticPartialsOff + (size_t)kStaticMaxChunks * 3 * sizeof(double);
constexpr size_t kStaticLayerOff = kStaticResultsOff + 8 * sizeof(double);  // {dot, |a|^2, |b|^2, ca, cb}, padded
constexpr size_t kStaticScratchBytes = (kStaticLayerOff + sizeof(Layer) + 255) / 256 * 256;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

}  // namespace
}  // namespace hvdhip

using namespace hvdhip;

struct hvdhip_adasum_plan {
  int nlayers = 0;
  int dtype = 0;
  int device = 0;  // the device that holds the tables and results
  int64_t total = 0;
  uint32_t max_layer_chunks = 0;
  DevTables tables;
  Layer* layers = nullptr;    // device, nlayers entries
  double* results = nullptr;  // one allocation: partials | normdots | coeffs | layer table
  double* partials = nullptr;
  double* normdots = nullptr;
  double* coeffs = nullptr;
};

namespace {

// The scaled add reads both vectors a second time, and the first pass decides with its loads what
// the 256 MB Infinity Cache holds by then: loads without the non-temporal hint leave their lines
// there.  Measured on the combine of fp32 vectors in 64 layers (neither / a alone / both kept):
//   2 x  32 MiB: 29.0 / 25.9 / 24.7 us      2 x 128 MiB: 103.8 /  96.7 / 100.7 us
//   2 x  64 MiB: 54.0 / 49.6 / 49.7 us      2 x 192 MiB: 152.2 / 145.6 / 150.1 us
//   2 x  96 MiB: 79.2 / 73.6 / 75.5 us      2 x 384 MiB: 304.2 / 291.5 / 305.1 us
// Keeping both pays while the pair fits the cache with room to spare; keeping one of the two pays
// at every size beyond, even where one vector by itself exceeds the cache (keeping b instead of a
// measures the same), and a pair that fills the cache to the brim (2 x 128 MiB) thrashes when both
// are kept.
constexpr uint64_t kKeepBothBytes = (uint64_t)160 << 20;  // largest pair (both vectors) kept whole
inline int keep_mode(uint64_t vector_bytes) { return 2 * vector_bytes <= kKeepBothBytes ? 2 : 1; }

template <int KEEP>
hipError_t launch_dot_partials(hvdhip_adasum_plan* p, const void* a, const void* b, hipStream_t s) {
  const DevTables& t = p->tables;
  switch (p->dtype) {
  case HVDHIP_FLOAT16:
    return launch(dot_partials_k<half_t, KEEP>, t.nchunks, s, t.chunks, static_cast<const half_t*>(a),
                  static_cast<const half_t*>(b), p->partials);
  case HVDHIP_FLOAT32:
    return launch(dot_partials_k<float, KEEP>, t.nchunks, s, t.chunks, static_cast<const float*>(a),
                  static_cast<const float*>(b), p->partials);
  default:
    return launch(dot_partials_k<double, KEEP>, t.nchunks, s, t.chunks, static_cast<const double*>(a),
                  static_cast<const double*>(b), p->partials);
  }
}

// finalize = false leaves the partial triples for a fused scaled add to sum.
int plan_dot_norms(hvdhip_adasum_plan* p, const void* a, const void* b, hipStream_t s,
                   bool finalize = true) {
  if (p->nlayers == 0) return 0;
  const DevTables& t = p->tables;
  if (t.nchunks > 0) {
    const bool both = keep_mode((uint64_t)p->total * (uint64_t)dtype_size(p->dtype)) == 2;
    HVDHIP_CHECK_LAUNCH("dot_partials_k", both ? launch_dot_partials<2>(p, a, b, s) : launch_dot_partials<1>(p, a, b, s));
  }
  if (!finalize) return 0;
  HVDHIP_CHECK_LAUNCH("finalize_k", launch(finalize_k, (uint32_t)p->nlayers, s, p->layers, p->partials, p->normdots,
                                           p->coeffs, std::sqrt(DBL_MIN)));
  return 0;
}

template <typename T, bool FUSED>
hipError_t launch_scaled_add(hvdhip_adasum_plan* p, void* a, const void* b, const double* coeffs,
                             double ca, double cb, hipStream_t s) {
  const DevTables& t = p->tables;
  return with_store_policy(Stores::kAdasum, [&](auto st) {
    return launch(scaled_add_k<T, FUSED, decltype(st)::value>, t.nchunks, s, t.chunks, static_cast<T*>(a),
                  static_cast<const T*>(b), coeffs, ca, cb, p->layers, p->partials, p->normdots, p->coeffs,
                  std::sqrt(DBL_MIN), (uint32_t)p->nlayers);
  });
}

template <bool FUSED>
int scaled_add_by_dtype(hvdhip_adasum_plan* p, void* a, const void* b, const double* coeffs,
                        double ca, double cb, hipStream_t s) {
  if (p->tables.nchunks == 0) return 0;
  hipError_t status;
  switch (p->dtype) {
  case HVDHIP_FLOAT16: status = launch_scaled_add<half_t, FUSED>(p, a, b, coeffs, ca, cb, s); break;
  case HVDHIP_FLOAT32: status = launch_scaled_add<float, FUSED>(p, a, b, coeffs, ca, cb, s); break;
  default: status = launch_scaled_add<double, FUSED>(p, a, b, coeffs, ca, cb, s); break;
  }
  HVDHIP_CHECK_LAUNCH("scaled_add_k", status);
  return 0;
}

// coeffs == nullptr selects the by-value pair (ca, cb) for every layer.
int plan_scaled_add(hvdhip_adasum_plan* p, void* a, const void* b, const double* coeffs,
                    double ca, double cb, hipStream_t s) {
  return scaled_add_by_dtype<false>(p, a, b, coeffs, ca, cb, s);
}

// The combine leaves the layer sums to the scaled add when every layer's partial triples fit the
// two loads per lane that kernel spends on them and there is a workgroup to do it (worth 0.6 % at
// 64 layers of 2^25 elements, 3.5 % at 1,000 layers, 9 % at 2^22 elements).
bool fused_coeffs(const hvdhip_adasum_plan* p) {
  return p->tables.nchunks > 0 && p->max_layer_chunks <= 2 * (uint32_t)kWG;
}

int check_vectors(const hvdhip_adasum_plan* p, const void* a, const void* b) {
  if (!p) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "plan is NULL");
  if (p->total > 0) {
    if (!a || !b) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "a or b is NULL");
    if (((uintptr_t)a | (uintptr_t)b) % (uintptr_t)dtype_size(p->dtype))
      return fail(HVDHIP_ERR_INVALID_ARGUMENT, "a or b is not aligned to its element size");
  }
  return 0;
}

// Single-layer plans for the Dispatch* entry points, keyed by (count, dtype, device, stream): a
// plan carries the partial sums of the launch that is using it, and callers on different streams
// must not share those.  The cache's mutex is held for lookup and insertion only; an entry is
// pinned by a use count while its caller launches on it and (for the blocking entry point)
// waits for the result, and pinned entries are neither handed to a second caller nor evicted.
struct OneLayerEntry {
  hvdhip_adasum_plan* plan = nullptr;
  hipStream_t stream = nullptr;
  int users = 0;
};
struct OneLayerCache {
  std::mutex mu;
  std::list<OneLayerEntry> lru;
};
OneLayerCache& one_layer_cache() {
  static OneLayerCache* c = new OneLayerCache();
  return *c;
}
constexpr size_t kOneLayerCapacity = 256;

// Pins a plan for (count, dtype) on the current device and `stream`; release with unpin().
int pin_one_layer_plan(int count, int dtype, hipStream_t stream, OneLayerEntry** out) {
  OneLayerCache& c = one_layer_cache();
  int device = 0;
  HVDHIP_CHECK(hipGetDevice(&device));
  {
    std::lock_guard<std::mutex> g(c.mu);
    for (auto it = c.lru.begin(); it != c.lru.end(); ++it) {
      if (it->users == 0 && it->stream == stream && it->plan->total == count && it->plan->dtype == dtype &&
          it->plan->device == device) {
        c.lru.splice(c.lru.begin(), c.lru, it);
        ++c.lru.front().users;
        *out = &c.lru.front();
        return 0;
      }
    }
  }
  // building a plan allocates and synchronises: outside the mutex
  hvdhip_adasum_plan* p = nullptr;
  int rc = hvdhip_adasum_plan_create(&count, 1, dtype, &p);
  if (rc) return rc;
  hvdhip_adasum_plan* victim = nullptr;
  {
    std::lock_guard<std::mutex> g(c.mu);
    if (c.lru.size() >= kOneLayerCapacity) {
      for (auto it = c.lru.end(); it != c.lru.begin();) {
        --it;
        if (it->users == 0) {
          victim = it->plan;
          c.lru.erase(it);
          break;
        }
      }
    }
    OneLayerEntry e;
    e.plan = p;
    e.stream = stream;
    e.users = 1;
    c.lru.push_front(e);
    *out = &c.lru.front();  // list nodes do not move
  }
  if (victim) hvdhip_adasum_plan_destroy(victim);  // waits for the device: outside the mutex
  return 0;
}

void unpin(OneLayerEntry* e) {
  std::lock_guard<std::mutex> g(one_layer_cache().mu);
  --e->users;
}

}  // namespace

// The stream is idle and about to be destroyed: the plans made for it would never be found again
// (a later stream at the same address on another device aside) and hold device memory.
void hvdhip::adasum_forget_stream(hipStream_t stream) {
  OneLayerCache& c = one_layer_cache();
  std::vector<hvdhip_adasum_plan*> dead;
  {
    std::lock_guard<std::mutex> g(c.mu);
    for (auto it = c.lru.begin(); it != c.lru.end();) {
      if (it->stream == stream && it->users == 0) {
        dead.push_back(it->plan);
        it = c.lru.erase(it);
      } else {
        ++it;
      }
    }
  }
  for (hvdhip_adasum_plan* p : dead) (void)hvdhip_adasum_plan_destroy(p);  // waits for the device: outside the mutex
}

extern "C" {

int hvdhip_adasum_plan_create(const int* tensor_counts, int nlayers, int dtype,
                              hvdhip_adasum_plan** plan) {
  if (!plan) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "plan is NULL");
  *plan = nullptr;
  if (nlayers < 0 || (nlayers > 0 && !tensor_counts)) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "bad tensor_counts");
  if (dtype != HVDHIP_FLOAT16 && dtype != HVDHIP_FLOAT32 && dtype != HVDHIP_FLOAT64)
    return fail(HVDHIP_ERR_UNSUPPORTED_DTYPE, "Adasum supports FLOAT16, FLOAT32 and FLOAT64, not dtype %d", dtype);
  const uint32_t chunk_units = chunk_bytes(Family::kAdasum) / (uint32_t)dtype_size(dtype);
  std::vector<Layer> layers((size_t)nlayers);
  std::vector<Chunk> chunks;
  uint64_t off = 0;
  uint32_t max_layer_chunks = 0;
  for (int i = 0; i < nlayers; ++i) {
    if (tensor_counts[i] < 0) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "tensor_counts[%d] is negative", i);
    const uint64_t n = (uint64_t)tensor_counts[i];
    layers[(size_t)i].first = (uint32_t)chunks.size();
    // Chunks are cut at multiples of the chunk size counted from the start of the vectors, not of
    // the layer: a layer begins wherever the one before it ends, and a chunk that starts in the
    // middle of a 16-byte piece (let alone of a cache line) makes every load of its workgroup
    // straddle two.  So a layer's first chunk runs up to the next such boundary, and all its
    // other chunks start on one.
    uint64_t start = 0;
    while (start < n) {
      const uint64_t to_boundary = chunk_units - (off + start) % chunk_units;
      const uint64_t left = n - start;
      const uint64_t len = left < to_boundary ? left : to_boundary;
      chunks.push_back(Chunk{off + start, (uint64_t)i, (uint64_t)chunks.size(), (uint32_t)len, 0});
      start += len;
    }
    layers[(size_t)i].count = (uint32_t)chunks.size() - layers[(size_t)i].first;
    for (size_t c = layers[(size_t)i].first; c < chunks.size(); ++c) {  // the layer's entry, folded into its chunks
      chunks[c].output |= (uint64_t)layers[(size_t)i].first << 32;
      chunks[c].pad = layers[(size_t)i].count;
    }
    if (layers[(size_t)i].count > max_layer_chunks) max_layer_chunks = layers[(size_t)i].count;
    if (chunks.size() > kMaxWorkgroups) return fail(HVDHIP_ERR_TOO_LARGE, "the vectors need more than 2^23 workgroups");
    off += n;
  }
  hvdhip_adasum_plan* p = new hvdhip_adasum_plan();
  p->nlayers = nlayers;
  p->dtype = dtype;
  p->total = (int64_t)off;
  p->max_layer_chunks = max_layer_chunks;
  (void)hipGetDevice(&p->device);
  {
    std::vector<Chunk> ordered(chunks.size());
    const uint32_t run = xcd_run(chunks.size(), chunk_bytes(Family::kAdasum), true);
    for (size_t c = 0; c < chunks.size(); ++c) ordered[xcd_slot(c, chunks.size(), run)] = chunks[c];
    chunks.swap(ordered);
  }
  int rc = upload_chunks(chunks, &p->tables);
  if (rc) {
    delete p;
    return rc;
  }
  const size_t ndoubles = 3 * (size_t)p->tables.nchunks + 5 * (size_t)nlayers + 8;
  const size_t layer_bytes = (size_t)nlayers * sizeof(Layer);
  hipError_t e = hipMalloc(reinterpret_cast<void**>(&p->results), ndoubles * sizeof(double) + layer_bytes);
  if (e == hipSuccess) e = hipMemset(p->results, 0, ndoubles * sizeof(double));
  if (e == hipSuccess && nlayers > 0)
    e = hipMemcpy(p->results + ndoubles, layers.data(), layer_bytes, hipMemcpyHostToDevice);
  // the fill above may return before the device has done it; the plan is used on other streams
  if (e == hipSuccess) e = hipStreamSynchronize(nullptr);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    if (p->results) (void)hipFree(p->results);
    free_tables(&p->tables);
    delete p;
    return fail(e == hipErrorOutOfMemory ? HVDHIP_ERR_OUT_OF_MEMORY : (int)e,
                "allocating Adasum results failed: %s", hipGetErrorString(e));
  }
  p->layers = reinterpret_cast<Layer*>(p->results + ndoubles);
  p->partials = p->results;
  p->normdots = p->partials + 3 * (size_t)p->tables.nchunks;
  p->coeffs = p->normdots + 3 * (size_t)nlayers;
  *plan = p;
  return ok();
}

int hvdhip_adasum_plan_destroy(hvdhip_adasum_plan* plan) {
  if (!plan) return ok();
  DeviceGuard on_plan_device(plan->device);
  HVDHIP_CHECK(hipDeviceSynchronize());  // queued kernels may still read the tables
  int rc = free_tables(&plan->tables);
  if (plan->results) (void)hipFree(plan->results);
  delete plan;
  return rc ? rc : ok();
}

int hvdhip_adasum_dot_norms(hvdhip_adasum_plan* plan, const void* a, const void* b, void* stream) {
  int rc = check_vectors(plan, a, b);
  if (rc) return rc;
  rc = plan_dot_norms(plan, a, b, static_cast<hipStream_t>(stream));
  return rc ? rc : ok();
}

int hvdhip_adasum_scaled_add(hvdhip_adasum_plan* plan, void* a, const void* b, void* stream) {
  int rc = check_vectors(plan, a, b);
  if (rc) return rc;
  rc = plan_scaled_add(plan, a, b, plan->coeffs, 0., 0., static_cast<hipStream_t>(stream));
  return rc ? rc : ok();
}

int hvdhip_adasum_combine(hvdhip_adasum_plan* plan, void* a, const void* b, void* stream) {
  int rc = check_vectors(plan, a, b);
  if (rc) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool fused = fused_coeffs(plan);
  rc = plan_dot_norms(plan, a, b, s, !fused);
  if (rc) return rc;
  rc = fused ? scaled_add_by_dtype<true>(plan, a, b, nullptr, 0., 0., s)
             : plan_scaled_add(plan, a, b, plan->coeffs, 0., 0., s);
  return rc ? rc : ok();
}

int hvdhip_adasum_read(hvdhip_adasum_plan* plan, double* normdots, double* coeffs, void* stream) {
  if (!plan) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "plan is NULL");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (plan->nlayers > 0) {
    if (normdots)
      HVDHIP_CHECK(hipMemcpyAsync(normdots, plan->normdots, 3 * (size_t)plan->nlayers * sizeof(double),
                                  hipMemcpyDeviceToHost, s));
    if (coeffs)
      HVDHIP_CHECK(hipMemcpyAsync(coeffs, plan->coeffs, 2 * (size_t)plan->nlayers * sizeof(double),
                                  hipMemcpyDeviceToHost, s));
  }
  HVDHIP_CHECK(hipStreamSynchronize(s));
  return ok();
}

int hvdhip_adasum_set_coeffs(hvdhip_adasum_plan* plan, const double* coeffs, void* stream) {
  if (!plan || (plan->nlayers > 0 && !coeffs)) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "plan or coeffs is NULL");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (plan->nlayers > 0) {
    HVDHIP_CHECK(hipMemcpyAsync(plan->coeffs, coeffs, 2 * (size_t)plan->nlayers * sizeof(double),
                                hipMemcpyHostToDevice, s));
    // The source is caller memory that may change as soon as this returns.
    HVDHIP_CHECK(hipStreamSynchronize(s));
  }
  return ok();
}

int hvdhip_adasum_dot_and_norm_sqrds(const void* a, const void* b, int dtype, int count,
                                     double* dot, double* anormsq, double* bnormsq,
                                     void* stream) {
  if (!dot || !anormsq || !bnormsq) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "result pointer is NULL");
  if (count < 0) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "count is negative");
  OneLayerEntry* e = nullptr;
  int rc = pin_one_layer_plan(count, dtype, static_cast<hipStream_t>(stream), &e);
  if (rc) return rc;
  double out[3] = {0., 0., 0.};
  rc = check_vectors(e->plan, a, b);
  if (rc == 0) rc = plan_dot_norms(e->plan, a, b, static_cast<hipStream_t>(stream));
  if (rc == 0) rc = hvdhip_adasum_read(e->plan, out, nullptr, stream);  // blocks; the mutex is not held
  unpin(e);
  if (rc) return rc;
  *dot = out[0];
  *anormsq = out[1];
  *bnormsq = out[2];
  return ok();
}

int hvdhip_adasum_dispatch_scaled_add(int dtype, int count, double acoeff, void* a,
                                      double bcoeff, const void* b, void* stream) {
  if (count < 0) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "count is negative");
  OneLayerEntry* e = nullptr;
  int rc = pin_one_layer_plan(count, dtype, static_cast<hipStream_t>(stream), &e);
  if (rc) return rc;
  rc = check_vectors(e->plan, a, b);
  if (rc == 0) rc = plan_scaled_add(e->plan, a, b, nullptr, acoeff, bcoeff, static_cast<hipStream_t>(stream));
  unpin(e);
  return rc ? rc : ok();
}

// ---- the combine that allocates nothing -------------------------------------

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
unsigned char* g_scratch_ptr[kMaxDevices];  // the device address of `scratch`, per device
// All calls on a device share its one array, so each call is ordered behind the one before it:
// an event is recorded behind a call's last kernel, and a call on another stream makes its stream
// wait for that event first.  The event is made once per device, with the address look-up.
hipEvent_t g_scratch_last_use[kMaxDevices];
hipStream_t g_scratch_last_stream[kMaxDevices];
bool g_scratch_used[kMaxDevices];

// The address of the current device's copy of `scratch`.  In host code the array's name is only
// a handle for the symbol; every use below goes through this pointer.
int static_scratch(unsigned char** out, int* device_out) {
  int device = 0;
  HVDHIP_CHECK(hipGetDevice(&device));
  *device_out = device;
  if (device < 0 || device >= kMaxDevices)
    return fail(HVDHIP_ERR_INVALID_ARGUMENT, "device %d is beyond the %d devices this entry point serves", device,
                kMaxDevices);
  std::lock_guard<std::mutex> g(g_scratch_mu);
  if (!g_scratch_ptr[device]) {
    void* p = nullptr;
    HVDHIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "hipGetSymbolAddress returned no address for the scratch array");
    HVDHIP_CHECK(hipEventCreateWithFlags(&g_scratch_last_use[device], hipEventDisableTiming | hipEventDisableSystemFence));
    g_scratch_ptr[device] = static_cast<unsigned char*>(p);
  }
  *out = g_scratch_ptr[device];
  return 0;
}
}  // namespace

int hvdhip_adasum_combine_static(void* a, const void* b, int dtype, int count, double* results,
                                 void* stream) {
  if (count < 0) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "count is negative");
  if (dtype != HVDHIP_FLOAT16 && dtype != HVDHIP_FLOAT32 && dtype != HVDHIP_FLOAT64)
    return fail(HVDHIP_ERR_UNSUPPORTED_DTYPE, "Adasum supports FLOAT16, FLOAT32 and FLOAT64, not dtype %d", dtype);
  if ((uintptr_t)results % sizeof(double)) return fail(HVDHIP_ERR_INVALID_ARGUMENT, "results is not aligned for doubles");
  const uint32_t chunk_units = chunk_bytes(Family::kAdasum) / (uint32_t)dtype_size(dtype);
  const uint64_t nchunks = ((uint64_t)count + chunk_units - 1) / chunk_units;
  if (nchunks > kStaticMaxChunks)
    return fail(HVDHIP_ERR_TOO_LARGE,
                "count %d needs %llu chunks of %u elements; hvdhip_adasum_combine_static holds %u (use a plan)",
                count, (unsigned long long)nchunks, chunk_units, kStaticMaxChunks);
  unsigned char* base = nullptr;
  int device = 0;
  int rc = static_scratch(&base, &device);
  if (rc) return rc;
  // A plan-shaped view of the scratch: nothing here is owned, nothing is freed.
  hvdhip_adasum_plan view;
  view.nlayers = 1;
  view.dtype = dtype;
  view.total = count;
  view.max_layer_chunks = (uint32_t)nchunks;
  view.tables.chunks = reinterpret_cast<Chunk*>(base + kStaticChunksOff);
  view.tables.nchunks = (uint32_t)nchunks;
  view.partials = reinterpret_cast<double*>(base + kStaticPartialsOff);
  view.normdots = results ? results : reinterpret_cast<double*>(base + kStaticResultsOff);
  view.coeffs = view.normdots + 3;
  view.layers = reinterpret_cast<Layer*>(base + kStaticLayerOff);
  rc = check_vectors(&view, a, b);
  if (rc) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  // One call at a time per device, on the host (the launches of two calls must not interleave) and
  // on the device (behind the last call's kernels).  A stream that is being captured takes neither
  // the wait nor the record: events recorded outside a capture cannot be waited for inside one, so
  // whoever launches the graph orders it against other calls.
  std::lock_guard<std::mutex> one_call(g_scratch_mu);
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  HVDHIP_CHECK(hipStreamIsCapturing(s, &capture));
  const bool eager = capture == hipStreamCaptureStatusNone;
  if (eager && g_scratch_used[device] && g_scratch_last_stream[device] != s)
    HVDHIP_CHECK(hipStreamWaitEvent(s, g_scratch_last_use[device], 0));
  // The array keeps what the last call left: the tables are rewritten for this count, and every
  // partial sum that is read is written first by this call's first pass.
  const uint32_t run = xcd_run(nchunks, chunk_bytes(Family::kAdasum), true);
  HVDHIP_CHECK_LAUNCH("one_layer_tables_k",
                      launch(one_layer_tables_k, (uint32_t)(nchunks / kWG + 1), s, view.tables.chunks, view.layers,
                             (uint32_t)nchunks, (uint64_t)count, chunk_units, run));
  const bool fused = fused_coeffs(&view);
  rc = plan_dot_norms(&view, a, b, s, !fused);
  if (rc) return rc;
  rc = fused ? scaled_add_by_dtype<true>(&view, a, b, nullptr, 0., 0., s)
             : plan_scaled_add(&view, a, b, view.coeffs, 0., 0., s);
  if (rc) return rc;
  if (eager) {
    HVDHIP_CHECK(hipEventRecord(g_scratch_last_use[device], s));
    g_scratch_last_stream[device] = s;
    g_scratch_used[device] = true;
  }
  return ok();
}

}  // extern "C"
