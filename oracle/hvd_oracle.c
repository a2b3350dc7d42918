/*
 * hvd_oracle.c -- CPU restatement of Horovod's gradient hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library links, loads or
 * calls this file.  It exists so the GPU kernels can be compared with what
 * the reference's own CPU path computes on the same seeded inputs, and so
 * the benchmark can time that CPU path on the GPU host.  Only the tests, the
 * smoke check and the benchmark's cpu_baseline leg may use it, and only as
 * the checker.
 *
 * Every function cites the reference lines (relative to the horovod source
 * tree) whose arithmetic it restates.  Build flags follow the reference's:
 * -O3 -mf16c -mavx -mfma (CMakeLists.txt:85-93).
 *
 * How each function is pinned (a function with no pin would say
 * "parity unpinned" here; none does):
 *   orc_half2float / orc_float2half  exhaustive / strided sweeps against the
 *       reference's own common/half.h compiled into oracle/_ref, against F16C
 *       hardware conversion and against numpy float16.
 *   orc_float16_sum                  against common/half.cc's float16_sum
 *       compiled into oracle/_ref, and against numpy (fp32 add, RNE to half).
 *   orc_pack / orc_unpack (+padded)  brute-force byte maps on tiny inputs,
 *       round trip identity, byte-pattern tensors (no cross-tensor bleed).
 *   orc_scale_buffer                 IEEE closed forms in numpy: one fp32 or
 *       fp64 product; trunc-toward-zero for integers; fp16 through fp32.
 *   orc_scale_half_cuda              numpy float16 product (exact product of two
 *       halves, one rounding) with the factor rounded to float16 first, on every
 *       half bit pattern; the expectation test/parallel/test_torch.py:339-445
 *       computes for device half tensors (factor.type(half) * tensor.type(half)).
 *   orc_sum                          numpy elementwise add per dtype.
 *   orc_adasum_dot_norms             math.fsum / numpy float64 dot.
 *   orc_adasum_coeffs, _scaled_add,  the numpy restatement held by the
 *   orc_adasum_pairwise              reference's own test
 *       (test/parallel/test_adasum_tensorflow.py:29-44) and the algebraic
 *       invariants of test/parallel/test_adasum_pytorch.py:46-211.
 *   orc_fuse_responses               hand-computed cases + brute force.
 *   orc_allgather_*                  closed form: every output equals the
 *       concatenation over ranks of that entry's per-rank tensor.
 */
#include <float.h>
#include <immintrin.h>
#include <math.h>
#include <stdint.h>
#include <string.h>

/* horovod::common::DataType values, common/message.h:30-41 */
enum {
  ORC_UINT8 = 0, ORC_INT8 = 1, ORC_UINT16 = 2, ORC_INT16 = 3, ORC_INT32 = 4,
  ORC_INT64 = 5, ORC_FLOAT16 = 6, ORC_FLOAT32 = 7, ORC_FLOAT64 = 8, ORC_BOOL = 9
};

/* DataType_Size, common/message.cc:66-92 */
int64_t orc_dtype_size(int dtype) {
  switch (dtype) {
  case ORC_UINT8: case ORC_INT8: case ORC_BOOL: return 1;
  case ORC_UINT16: case ORC_INT16: case ORC_FLOAT16: return 2;
  case ORC_INT32: case ORC_FLOAT32: return 4;
  case ORC_INT64: case ORC_FLOAT64: return 8;
  default: return -1;
  }
}

/* ------------------------------------------------------------------ */
/* fp16 <-> fp32, software, common/half.h:43-77 and :79-139           */
/* ------------------------------------------------------------------ */

static inline float bits_to_float(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t float_to_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

/* half.h:43-77.  Normals rebias by 112; subnormals are renormalised; zero
 * keeps its sign; inf keeps its sign; every NaN becomes 0x7fffffff. */
static inline float half_bits_to_float(uint16_t h) {
  uint32_t sgn = (uint32_t)(h >> 15) << 31;
  uint32_t e = (h >> 10) & 0x1fu;
  uint32_t m = h & 0x3ffu;
  if (e == 31) return bits_to_float(m ? 0x7fffffffu : (sgn | 0x7f800000u));
  if (e == 0) {
    if (m == 0) return bits_to_float(sgn);
    /* value = m * 2^-24; find the leading one of the 10-bit field */
    uint32_t fe = 113;
    while (!(m & 0x400u)) { m <<= 1; --fe; }
    return bits_to_float(sgn | (fe << 23) | ((m & 0x3ffu) << 13));
  }
  return bits_to_float(sgn | ((e + 112u) << 23) | (m << 13));
}

/* half.h:79-139.  Round to nearest even with a sticky bit; overflow gives
 * +-inf, NaN gives 0x7fff (sign dropped), fp32 magnitudes whose shift would
 * reach 32 bits give +-0. */
static inline uint16_t float_to_half_bits(float f) {
  uint32_t s = float_to_bits(f);
  uint16_t sgn = (uint16_t)((s >> 16) & 0x8000u);
  if ((s & 0x7fffffffu) == 0) return sgn;
  int e = (int)((s >> 23) & 0xffu) - 127;
  uint32_t m = s & 0x7fffffu;
  if (e > 15) return (e == 128 && m) ? (uint16_t)0x7fff : (uint16_t)(sgn | 0x7c00u);
  uint32_t u;
  int sticky = 0;
  if (e >= -14) {
    u = ((uint32_t)(e + 15) << 10) | (m >> 13);
  } else {
    int rs = -14 - e;
    if (rs < 32) {
      m |= 1u << 23;
      sticky = (m & ((1u << rs) - 1u)) != 0;
      m >>= rs;
      u = (m >> 13) & 0x3ffu;
    } else {
      m = 0;
      u = 0;
    }
  }
  int round_bit = (m >> 12) & 1;
  sticky |= (m & 0xfffu) != 0;
  if (round_bit && (sticky || (u & 1u))) ++u;
  return (uint16_t)(u | sgn);
}

void orc_half2float(const uint16_t* src, float* dst, int64_t n) {
  for (int64_t i = 0; i < n; ++i) dst[i] = half_bits_to_float(src[i]);
}

void orc_float2half(const float* src, uint16_t* dst, int64_t n) {
  for (int64_t i = 0; i < n; ++i) dst[i] = float_to_half_bits(src[i]);
}

/* Hardware F16C conversions (RNE), used by the 8-wide paths below and as an
 * independent cross-check of the software converters. */
void orc_half2float_f16c(const uint16_t* src, float* dst, int64_t n) {
  for (int64_t i = 0; i < n; ++i) dst[i] = _cvtsh_ss(src[i]);
}
void orc_float2half_f16c(const float* src, uint16_t* dst, int64_t n) {
  for (int64_t i = 0; i < n; ++i)
    dst[i] = _cvtss_sh(src[i], _MM_FROUND_TO_NEAREST_INT);
}

/* ------------------------------------------------------------------ */
/* Fusion buffer pack / unpack                                        */
/* ------------------------------------------------------------------ */

/* AllreduceOp::MemcpyInFusionBuffer + MemcpyEntryInFusionBuffer,
 * ops/collective_operations.cc:68-88,100-105: memcpy each tensor at a
 * running, unpadded byte offset; returns buffer_len. */
int64_t orc_pack(const void* const* tensors, const int64_t* nbytes, int n, void* buf) {
  int64_t off = 0;
  for (int i = 0; i < n; ++i) {
    memcpy((uint8_t*)buf + off, tensors[i], (size_t)nbytes[i]);
    off += nbytes[i];
  }
  return off;
}

/* AllreduceOp::MemcpyOutFusionBuffer + MemcpyEntryOutFusionBuffer,
 * ops/collective_operations.cc:90-98,107-112. */
void orc_unpack(const void* buf, void* const* outputs, const int64_t* nbytes, int n) {
  int64_t off = 0;
  for (int i = 0; i < n; ++i) {
    memcpy(outputs[i], (const uint8_t*)buf + off, (size_t)nbytes[i]);
    off += nbytes[i];
  }
}

/* GPU layout of GPUAllreduce::MemcpyInFusionBuffer, ops/gpu_operations.cc:127-153:
 * each offset advances by the size rounded up to BATCHED_D2D_PADDING = 16
 * (ops/cuda/cuda_kernels.h:24).  offsets[n] receives the padded buffer_len. */
int64_t orc_padded_offsets(const int64_t* nbytes, int n, int64_t* offsets) {
  int64_t off = 0;
  for (int i = 0; i < n; ++i) {
    offsets[i] = off;
    off += 16 * ((nbytes[i] + 15) / 16);
  }
  offsets[n] = off;
  return off;
}

int64_t orc_pack_padded(const void* const* tensors, const int64_t* nbytes, int n, void* buf) {
  int64_t off = 0;
  for (int i = 0; i < n; ++i) {
    memcpy((uint8_t*)buf + off, tensors[i], (size_t)nbytes[i]);
    off += 16 * ((nbytes[i] + 15) / 16);
  }
  return off;
}

/* GPUAllreduce::MemcpyOutFusionBuffer, ops/gpu_operations.cc:238-275. */
void orc_unpack_padded(const void* buf, void* const* outputs, const int64_t* nbytes, int n) {
  int64_t off = 0;
  for (int i = 0; i < n; ++i) {
    memcpy(outputs[i], (const uint8_t*)buf + off, (size_t)nbytes[i]);
    off += 16 * ((nbytes[i] + 15) / 16);
  }
}

/* ------------------------------------------------------------------ */
/* ScaleBuffer                                                        */
/* ------------------------------------------------------------------ */

/* ScaleBufferCPUImpl<unsigned short,float>, ops/collective_operations.h:99-127:
 * groups of 8 through F16C (half -> fp32, one fp32 multiply by the fp32
 * factor, RNE back to half), remainder through the software converters. */
static void scale_half(const uint16_t* in, uint16_t* out, int64_t n, float factor) {
  int64_t i = 0;
  __m256 f8 = _mm256_set1_ps(factor);
  for (; i + 8 <= n; i += 8) {
    __m256 x = _mm256_cvtph_ps(_mm_loadu_si128((const __m128i*)(in + i)));
    __m128i y = _mm256_cvtps_ph(_mm256_mul_ps(x, f8), 0);
    _mm_storeu_si128((__m128i*)(out + i), y);
  }
  for (; i < n; ++i) {
    float p = factor * half_bits_to_float(in[i]);
    out[i] = float_to_half_bits(p);
  }
}

/* Same arithmetic with the software converters only; the 8-wide/tail split
 * of the reference must not change any value, which a test checks. */
void orc_scale_half_scalar(const uint16_t* in, uint16_t* out, int64_t n, float factor) {
  for (int64_t i = 0; i < n; ++i) {
    float p = factor * half_bits_to_float(in[i]);
    out[i] = float_to_half_bits(p);
  }
}

/* The fp16 scale of the reference's CUDA kernels, ops/cuda/cuda_kernels.cu:96-136 with
 * the factor prepared at :167 (and :306-309 for the batched scaled copy): the factor is
 * rounded to half first, __float2half((float)scale_factor), then half times half with one
 * rounding.  The kernels' own branch for devices without half arithmetic (:115-118,
 * :131-134) spells the same value as
 * __float2half(__half2float(scale_factor) * __half2float(input[i])), which is what this
 * restates with the software converters: the fp32 product of two halves is exact. */
void orc_scale_half_cuda(const uint16_t* in, uint16_t* out, int64_t n, double scale) {
  const uint16_t hs = float_to_half_bits((float)scale);
  const float fs = half_bits_to_float(hs);
  for (int64_t i = 0; i < n; ++i) out[i] = float_to_half_bits(fs * half_bits_to_float(in[i]));
}

#define SCALE_LOOP(T, TS)                                                     \
  do {                                                                        \
    const T* x = (const T*)in;                                                \
    T* y = (T*)out;                                                           \
    TS s = (TS)scale;                                                         \
    for (int64_t i = 0; i < n; ++i) y[i] = (T)(s * x[i]);                     \
  } while (0)

/* AllreduceOp::ScaleBuffer, ops/collective_operations.cc:114-146, over
 * ScaleBufferCPUImpl<T,TS>, ops/collective_operations.h:91-96: the factor is
 * double for u8/i8/i32/i64/f64 (product in double, converted back to T, i.e.
 * truncation toward zero for integers) and float for f32 and f16.  Returns 0,
 * or -1 for the dtypes the reference rejects with std::logic_error. */
int orc_scale_buffer(const void* in, void* out, int64_t n, double scale, int dtype) {
  switch (dtype) {
  case ORC_UINT8: SCALE_LOOP(uint8_t, double); return 0;
  case ORC_INT8: SCALE_LOOP(int8_t, double); return 0;
  case ORC_INT32: SCALE_LOOP(int32_t, double); return 0;
  case ORC_INT64: SCALE_LOOP(int64_t, double); return 0;
  case ORC_FLOAT16: scale_half((const uint16_t*)in, (uint16_t*)out, n, (float)scale); return 0;
  case ORC_FLOAT32: SCALE_LOOP(float, float); return 0;
  case ORC_FLOAT64: SCALE_LOOP(double, double); return 0;
  default: return -1;
  }
}

/* The compression cast folded into packing: prescale in fp32
 * (ScaleBufferCPUImpl<float,float>, collective_operations.h:91-96; skipped when
 * the factor is exactly 1.0 as in ops/gloo_operations.cc:145-148), then
 * Float2HalfBits (common/half.h:79-139): a single rounding to half. */
void orc_scale_cast_f32_to_f16(const float* in, uint16_t* out, int64_t n, double scale) {
  float s = (float)scale;
  if (scale != 1.0) {
    for (int64_t i = 0; i < n; ++i) out[i] = float_to_half_bits(s * in[i]);
  } else {
    for (int64_t i = 0; i < n; ++i) out[i] = float_to_half_bits(in[i]);
  }
}

/* The reference's own pipeline order: Compression.fp16 casts first
 * (horovod/torch/compression.py:49-55), then the fp16 ScaleBuffer runs on the
 * halves (collective_operations.h:99-127): two roundings. */
void orc_cast_then_scale_f32_to_f16(const float* in, uint16_t* out, int64_t n, double scale) {
  float s = (float)scale;
  for (int64_t i = 0; i < n; ++i) {
    uint16_t h = float_to_half_bits(in[i]);
    out[i] = (scale != 1.0) ? float_to_half_bits(s * half_bits_to_float(h)) : h;
  }
}

/* Postscale on the fp16 buffer (collective_operations.h:99-127, skipped at
 * 1.0 as in ops/gloo_operations.cc:157-160) followed by the decompression
 * cast back to fp32 (horovod/torch/compression.py:58-64, exact). */
void orc_scale_cast_f16_to_f32(const uint16_t* in, float* out, int64_t n, double scale) {
  float s = (float)scale;
  for (int64_t i = 0; i < n; ++i) {
    uint16_t h = in[i];
    if (scale != 1.0) h = float_to_half_bits(s * half_bits_to_float(h));
    out[i] = half_bits_to_float(h);
  }
}

/* The two casts above the way a build with F16C runs them (eight lanes per instruction, as
 * in the 8-wide path of collective_operations.h:105-112 and in the framework's own cast),
 * for timing the CPU side; remainders go through the software converters.  Same values as
 * the software versions for every input that is not a NaN, which a test checks. */
void orc_scale_cast_f32_to_f16_f16c(const float* in, uint16_t* out, int64_t n, double scale) {
  const float s = (float)scale;
  const __m256 s8 = _mm256_set1_ps(s);
  int64_t i = 0;
  if (scale != 1.0) {
    for (; i + 8 <= n; i += 8)
      _mm_storeu_si128((__m128i*)(out + i), _mm256_cvtps_ph(_mm256_mul_ps(_mm256_loadu_ps(in + i), s8), 0));
    for (; i < n; ++i) out[i] = float_to_half_bits(s * in[i]);
  } else {
    for (; i + 8 <= n; i += 8)
      _mm_storeu_si128((__m128i*)(out + i), _mm256_cvtps_ph(_mm256_loadu_ps(in + i), 0));
    for (; i < n; ++i) out[i] = float_to_half_bits(in[i]);
  }
}
void orc_scale_cast_f16_to_f32_f16c(const uint16_t* in, float* out, int64_t n, double scale) {
  const float s = (float)scale;
  const __m256 s8 = _mm256_set1_ps(s);
  int64_t i = 0;
  for (; i + 8 <= n; i += 8) {
    __m128i h = _mm_loadu_si128((const __m128i*)(in + i));
    if (scale != 1.0) h = _mm256_cvtps_ph(_mm256_mul_ps(_mm256_cvtph_ps(h), s8), 0);
    _mm256_storeu_ps(out + i, _mm256_cvtph_ps(h));
  }
  for (; i < n; ++i) {
    uint16_t h = in[i];
    if (scale != 1.0) h = float_to_half_bits(s * half_bits_to_float(h));
    out[i] = half_bits_to_float(h);
  }
}

/* ------------------------------------------------------------------ */
/* Local reduce-sum                                                   */
/* ------------------------------------------------------------------ */

/* float16_sum, common/half.cc:44-76: inout = RNE16(fp32(in) + fp32(inout)),
 * 8-wide F16C then a software tail. */
void orc_float16_sum(const uint16_t* in, uint16_t* inout, int64_t len) {
  int64_t i = 0;
  for (; i + 8 <= len; i += 8) {
    __m256 a = _mm256_cvtph_ps(_mm_loadu_si128((const __m128i*)(in + i)));
    __m256 b = _mm256_cvtph_ps(_mm_loadu_si128((const __m128i*)(inout + i)));
    _mm_storeu_si128((__m128i*)(inout + i), _mm256_cvtps_ph(_mm256_add_ps(a, b), 0));
  }
  for (; i < len; ++i) {
    float r = half_bits_to_float(inout[i]);
    r += half_bits_to_float(in[i]);
    inout[i] = float_to_half_bits(r);
  }
}

/* Software-only version of the same sum (the reference's tail loop applied to
 * every element). */
void orc_float16_sum_scalar(const uint16_t* in, uint16_t* inout, int64_t len) {
  for (int64_t i = 0; i < len; ++i) {
    float r = half_bits_to_float(inout[i]);
    r += half_bits_to_float(in[i]);
    inout[i] = float_to_half_bits(r);
  }
}

#define SUM_LOOP(T, U)                                                        \
  do {                                                                        \
    const T* x = (const T*)in;                                                \
    T* y = (T*)inout;                                                         \
    for (int64_t i = 0; i < n; ++i) y[i] = (T)((U)y[i] + (U)x[i]);            \
  } while (0)

/* The element-wise sum that the collective applies: gloo::sum<T>
 * (call site ops/gloo_operations.cc:66-74), MPI_SUM (ops/mpi_operations.cc:63-66),
 * ncclSum (ops/nccl_operations.cc:190-193); fp16 through float16_sum.
 * Integers wrap (computed in the unsigned type).  One IEEE add per element. */
int orc_sum(const void* in, void* inout, int64_t n, int dtype) {
  switch (dtype) {
  case ORC_UINT8: SUM_LOOP(uint8_t, uint8_t); return 0;
  case ORC_INT8: SUM_LOOP(int8_t, uint8_t); return 0;
  case ORC_UINT16: SUM_LOOP(uint16_t, uint16_t); return 0;
  case ORC_INT16: SUM_LOOP(int16_t, uint16_t); return 0;
  case ORC_INT32: SUM_LOOP(int32_t, uint32_t); return 0;
  case ORC_INT64: SUM_LOOP(int64_t, uint64_t); return 0;
  case ORC_FLOAT16: orc_float16_sum((const uint16_t*)in, (uint16_t*)inout, n); return 0;
  case ORC_FLOAT32: SUM_LOOP(float, float); return 0;
  case ORC_FLOAT64: SUM_LOOP(double, double); return 0;
  default: return -1;
  }
}

/* ------------------------------------------------------------------ */
/* Adasum                                                             */
/* ------------------------------------------------------------------ */

static inline double hsum4(__m256d v) {
  /* Mm256ReductionPd, ops/adasum/adasum.h:503-510: (v0+v2) + (v1+v3) */
  __m128d lo = _mm256_castpd256_pd128(v);
  __m128d hi = _mm256_extractf128_pd(v, 1);
  lo = _mm_add_pd(lo, hi);
  __m128d up = _mm_unpackhi_pd(lo, lo);
  return _mm_cvtsd_f64(_mm_add_sd(lo, up));
}

static inline __m256 load_half8_partial(const uint16_t* p, int k) {
  /* MmLoaduPhPartial, adasum.h:526-532: missing lanes read as zero */
  uint16_t tmp[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  memcpy(tmp, p, (size_t)(k < 8 ? k : 8) * 2);
  return _mm256_cvtph_ps(_mm_loadu_si128((const __m128i*)tmp));
}

/* ComputeDotAndNormSqrdsfp16, ops/adasum/adasum.h:439-480: per 8 halves,
 * widen to fp32 then to fp64 in two groups of four, fused multiply-add into
 * three 4-lane fp64 accumulators (low group first, then high group). */
static void dot_norms_half(const uint16_t* a, const uint16_t* b, int len, double* out3) {
  __m256d d = _mm256_setzero_pd(), na = _mm256_setzero_pd(), nb = _mm256_setzero_pd();
  int i = 0;
  for (; i < len; i += 8) {
    __m256 av, bv;
    if (i + 8 <= len) {
      av = _mm256_cvtph_ps(_mm_loadu_si128((const __m128i*)(a + i)));
      bv = _mm256_cvtph_ps(_mm_loadu_si128((const __m128i*)(b + i)));
    } else {
      av = load_half8_partial(a + i, len - i);
      bv = load_half8_partial(b + i, len - i);
    }
    __m256d a0 = _mm256_cvtps_pd(_mm256_extractf128_ps(av, 0));
    __m256d a1 = _mm256_cvtps_pd(_mm256_extractf128_ps(av, 1));
    __m256d b0 = _mm256_cvtps_pd(_mm256_extractf128_ps(bv, 0));
    __m256d b1 = _mm256_cvtps_pd(_mm256_extractf128_ps(bv, 1));
    d = _mm256_fmadd_pd(a0, b0, d);
    d = _mm256_fmadd_pd(a1, b1, d);
    na = _mm256_fmadd_pd(a0, a0, na);
    na = _mm256_fmadd_pd(a1, a1, na);
    nb = _mm256_fmadd_pd(b0, b0, nb);
    nb = _mm256_fmadd_pd(b1, b1, nb);
  }
  out3[0] = hsum4(d);
  out3[1] = hsum4(na);
  out3[2] = hsum4(nb);
}

/* Adasum::ComputeDotAndNormSqrds<T>, ops/adasum/adasum.h:413-426 (fp32,
 * fp64: every product and sum in double, strictly sequential) and the fp16
 * AVX variant :439-480.  out3 = {dot, |a|^2, |b|^2}.  Dispatch as in
 * DispatchComputeDotAndNormSqrds, adasum.h:101-122. */
int orc_adasum_dot_norms(const void* a, const void* b, int count, int dtype, double* out3) {
  double dot = 0., an = 0., bn = 0.;
  if (dtype == ORC_FLOAT32) {
    const float* x = (const float*)a;
    const float* y = (const float*)b;
    for (int i = 0; i < count; ++i) {
      dot += (double)x[i] * (double)y[i];
      an += (double)x[i] * (double)x[i];
      bn += (double)y[i] * (double)y[i];
    }
  } else if (dtype == ORC_FLOAT64) {
    const double* x = (const double*)a;
    const double* y = (const double*)b;
    for (int i = 0; i < count; ++i) {
      dot += x[i] * y[i];
      an += x[i] * x[i];
      bn += y[i] * y[i];
    }
  } else if (dtype == ORC_FLOAT16) {
    dot_norms_half((const uint16_t*)a, (const uint16_t*)b, count, out3);
    return 0;
  } else {
    return -1;
  }
  out3[0] = dot; out3[1] = an; out3[2] = bn;
  return 0;
}

/* Coefficients, ops/adasum/adasum.h:397-404: 1 - dot/norm * 0.5 evaluated
 * left to right, guarded by norm >= sqrt(DBL_MIN), else 1. */
void orc_adasum_coeffs(double dot, double an, double bn, double* ca, double* cb) {
  double guard = sqrt(DBL_MIN);
  double x = 1., y = 1.;
  if (an >= guard) x = 1.0 - dot / an * 0.5;
  if (bn >= guard) y = 1.0 - dot / bn * 0.5;
  *ca = x;
  *cb = y;
}

/* ScaledAddfp16, adasum.h:482-500: coefficients narrowed to float; per
 * element fp32 t = ca*a (rounded), r = fma(cb, b, t), RNE to half. */
static void scaled_add_half(int len, double ca, uint16_t* a, double cb, const uint16_t* b) {
  __m256 cav = _mm256_set1_ps((float)ca);
  __m256 cbv = _mm256_set1_ps((float)cb);
  for (int i = 0; i < len; i += 8) {
    int k = len - i < 8 ? len - i : 8;
    __m256 av = (k == 8) ? _mm256_cvtph_ps(_mm_loadu_si128((const __m128i*)(a + i)))
                         : load_half8_partial(a + i, k);
    __m256 bv = (k == 8) ? _mm256_cvtph_ps(_mm_loadu_si128((const __m128i*)(b + i)))
                         : load_half8_partial(b + i, k);
    av = _mm256_mul_ps(cav, av);
    __m128i r = _mm256_cvtps_ph(_mm256_fmadd_ps(cbv, bv, av), 0);
    uint16_t tmp[8];
    _mm_storeu_si128((__m128i*)tmp, r);
    memcpy(a + i, tmp, (size_t)k * 2);
  }
}

/* Keeps the compiler from contracting a product into the sum that follows it
 * (-mfma with the GNU fp-contract default would): the value passes through a
 * register untouched. */
static inline double rounded(double x) {
  __asm__("" : "+x"(x));
  return x;
}

/* Adasum::ScaledAdd<T>, ops/adasum/adasum.h:429-435: a = ca*a + cb*b with the
 * operands promoted to double and the result converted to T; fp16 variant
 * :482-500.  Dispatch as in DispatchScaledAdd, adasum.h:124-140.  The double
 * expression is evaluated as the source states it: two rounded products and
 * their rounded sum.  (A reference build with -mfma may contract one product
 * into the sum, which moves a result by at most one unit in the last place.) */
int orc_adasum_scaled_add(int dtype, int count, double ca, void* a, double cb, const void* b) {
  if (dtype == ORC_FLOAT32) {
    float* x = (float*)a;
    const float* y = (const float*)b;
    for (int i = 0; i < count; ++i) x[i] = (float)(rounded(ca * x[i]) + rounded(cb * y[i]));
  } else if (dtype == ORC_FLOAT64) {
    double* x = (double*)a;
    const double* y = (const double*)b;
    for (int i = 0; i < count; ++i) x[i] = rounded(ca * x[i]) + rounded(cb * y[i]);
  } else if (dtype == ORC_FLOAT16) {
    scaled_add_half(count, ca, (uint16_t*)a, cb, (const uint16_t*)b);
  } else {
    return -1;
  }
  return 0;
}

/* FusedPairwiseReduceWithComm, ops/adasum/adasum.h:344-410, for one process
 * (the group allreduce of the 3*nlayers doubles is the identity and the
 * left/right swap of the norms cancels).  Layers are consecutive slices of
 * tensor_counts[i] elements.  normdots receives {dot, an, bn} per layer, and
 * coeffs, if not NULL, {ca, cb} per layer.  a is updated in place. */
int orc_adasum_pairwise(void* a, const void* b, int dtype, const int* tensor_counts,
                        int nlayers, double* normdots, double* coeffs) {
  int64_t es = orc_dtype_size(dtype);
  if (dtype != ORC_FLOAT16 && dtype != ORC_FLOAT32 && dtype != ORC_FLOAT64) return -1;
  int64_t off = 0;
  for (int i = 0; i < nlayers; ++i) {
    orc_adasum_dot_norms((const uint8_t*)a + off, (const uint8_t*)b + off, tensor_counts[i],
                         dtype, normdots + 3 * i);
    off += (int64_t)tensor_counts[i] * es;
  }
  off = 0;
  for (int i = 0; i < nlayers; ++i) {
    double ca, cb;
    orc_adasum_coeffs(normdots[3 * i], normdots[3 * i + 1], normdots[3 * i + 2], &ca, &cb);
    if (coeffs) { coeffs[2 * i] = ca; coeffs[2 * i + 1] = cb; }
    orc_adasum_scaled_add(dtype, tensor_counts[i], ca, (uint8_t*)a + off, cb,
                          (const uint8_t*)b + off);
    off += (int64_t)tensor_counts[i] * es;
  }
  return 0;
}

/* ------------------------------------------------------------------ */
/* Fusion planning                                                    */
/* ------------------------------------------------------------------ */

/* Controller::TensorFusionThresholdBytes, common/controller.cc:463-481: on a
 * homogeneous cluster round the threshold up to a multiple of
 * local_size * sizeof(double) * FUSION_BUFFER_ATOMIC_UNIT (64, common/common.h:146). */
int64_t orc_fusion_threshold(int64_t proposed, int local_size, int homogeneous) {
  if (!homogeneous) return proposed;
  int64_t div = (int64_t)local_size * 8 * 64;
  return ((proposed + div - 1) / div) * div;
}

/* Controller::FuseResponses, common/controller.cc:793-866, for allreduce
 * responses.  Response i carries tensor_bytes[i] bytes and an opaque
 * compatibility key[i] (standing for response type, devices, dtype, prescale
 * and postscale, :831-836).  pad16 selects the 16-byte padded sizes used when
 * batched device copies are on (:807-812,824-829).  group_of[i] receives the
 * index of the fused response that tensor i lands in; groups are numbered in
 * the order they are emitted.  Returns the number of groups.
 *
 * The queue is consumed front to back: the head opens a group; following
 * responses join while compatible and within the threshold; an incompatible
 * or non-fitting response is skipped only while the running total plus
 * everything skipped so far still fits, otherwise the group closes; skipped
 * responses return to the front of the queue in their original order. */
int orc_fuse_responses(const int64_t* tensor_bytes, const int* key, int n, int64_t threshold,
                       int pad16, int* group_of) {
  int ngroups = 0;
  for (int i = 0; i < n; ++i) group_of[i] = -1;
  /* "queue" = indices with group_of == -1, in index order */
  for (int head = 0; head < n; ++head) {
    if (group_of[head] != -1) continue;
    int g = ngroups++;
    group_of[head] = g;
    int64_t size = tensor_bytes[head];
    if (pad16) size = 16 * ((size + 15) / 16);
    int64_t skipped = 0;
    for (int j = head + 1; j < n; ++j) {
      if (group_of[j] != -1) continue;
      int64_t nsz = tensor_bytes[j];
      if (pad16) nsz = 16 * ((nsz + 15) / 16);
      if (key[j] == key[head] && size + nsz <= threshold) {
        size += nsz;
        group_of[j] = g;
      } else {
        skipped += nsz;
        if (size + skipped > threshold) break;
      }
    }
  }
  return ngroups;
}

/* ------------------------------------------------------------------ */
/* Allgather fusion buffer                                            */
/* ------------------------------------------------------------------ */

/* AllgatherOp::SetDisplacements, ops/collective_operations.cc:200-209:
 * exclusive prefix sum of the per-rank element counts. */
void orc_allgather_displacements(const int* recvcounts, int* displcmnts, int global_size) {
  int acc = 0;
  for (int rc = 0; rc < global_size; ++rc) {
    displcmnts[rc] = acc;
    acc += recvcounts[rc];
  }
}

/* AllgatherOp::SetEntryComponentOffsets, ops/collective_operations.cc:211-232.
 * sizes and offsets are row-major [entry][rank] element counts: inside rank
 * rc's slab (which starts at the sum of the earlier ranks' recvcounts) the
 * entries follow one another. */
void orc_allgather_component_offsets(const int64_t* sizes, int nentries, int global_size,
                                     const int* recvcounts, int64_t* offsets) {
  int64_t rank_displacement = 0;
  for (int rc = 0; rc < global_size; ++rc) {
    for (int ec = 0; ec < nentries; ++ec) {
      if (ec == 0)
        offsets[ec * global_size + rc] = rank_displacement;
      else
        offsets[ec * global_size + rc] =
            offsets[(ec - 1) * global_size + rc] + sizes[(ec - 1) * global_size + rc];
    }
    rank_displacement += recvcounts[rc];
  }
}

/* AllgatherOp::MemcpyInFusionBuffer, ops/collective_operations.cc:234-253:
 * this rank's entries go, unpadded, to its displacement in the buffer. */
void orc_allgather_pack(const void* const* tensors, const int64_t* nbytes, int nentries,
                        const int* displcmnts, int rank, int element_size, void* buf) {
  int64_t off = (int64_t)displcmnts[rank] * element_size;
  for (int i = 0; i < nentries; ++i) {
    memcpy((uint8_t*)buf + off, tensors[i], (size_t)nbytes[i]);
    off += nbytes[i];
  }
}

/* AllgatherOp::MemcpyOutFusionBuffer, ops/collective_operations.cc:255-275:
 * output ec is the concatenation over ranks of that entry's component. */
void orc_allgather_unpack(const int64_t* offsets, const int64_t* sizes, int nentries,
                          int global_size, const void* buf, int element_size,
                          void* const* outputs) {
  for (int ec = 0; ec < nentries; ++ec) {
    int64_t copy_offset = 0;
    for (int rc = 0; rc < global_size; ++rc) {
      int64_t eo = offsets[ec * global_size + rc] * element_size;
      int64_t es = sizes[ec * global_size + rc] * element_size;
      memcpy((uint8_t*)outputs[ec] + copy_offset, (const uint8_t*)buf + eo, (size_t)es);
      copy_offset += es;
    }
  }
}
