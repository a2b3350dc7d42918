/*
 * hvdhip.h -- C ABI of the MI355X (gfx950) implementation of Horovod's
 * single-GPU gradient hot path.
 *
 * Everything here is `extern "C"`, takes plain pointers and sizes, and is
 * asynchronous on the HIP stream it is given unless stated otherwise.  Every
 * function returns an int: 0 on success, a positive value equal to the
 * hipError_t that a HIP call returned, or one of the negative HVDHIP_ERR_*
 * codes below for an argument the library itself rejected.  No exception
 * crosses this boundary; hvdhip_error_string() and hvdhip_last_error()
 * describe a failure.  The library owns only its streams, events, plans and
 * the small device tables inside plans; tensors, outputs and fusion buffers
 * belong to the caller (in Horovod: the framework and FusionBufferManager).
 *
 * File and line references name the interface of the reference (paths
 * relative to the horovod source tree) that each entry point stands behind.
 *
 * Threading: launches are expected from one thread per stream (Horovod's
 * background thread, common/operations.cc:381); the event pool and the plan
 * cache are mutex-guarded because finalizer threads acquire, query and
 * release events concurrently (ops/gpu_operations.cc:72-99).
 */
#ifndef HVDHIP_H
#define HVDHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Element types: the values of horovod::common::DataType, common/message.h:30-41. */
enum hvdhip_dtype {
  HVDHIP_UINT8 = 0,
  HVDHIP_INT8 = 1,
  HVDHIP_UINT16 = 2,
  HVDHIP_INT16 = 3,
  HVDHIP_INT32 = 4,
  HVDHIP_INT64 = 5,
  HVDHIP_FLOAT16 = 6,
  HVDHIP_FLOAT32 = 7,
  HVDHIP_FLOAT64 = 8,
  HVDHIP_BOOL = 9
};

/* Library-side argument errors (HIP errors are returned as positive hipError_t). */
#define HVDHIP_SUCCESS 0
#define HVDHIP_ERR_INVALID_ARGUMENT (-1)
/* dtype outside the table the reference scales or sums; the reference throws
 * std::logic_error("Type ... not supported by ...") here
 * (ops/collective_operations.cc:141-144, ops/cuda/cuda_kernels.cu:182-185,317-319). */
#define HVDHIP_ERR_UNSUPPORTED_DTYPE (-2)
#define HVDHIP_ERR_OUT_OF_MEMORY (-3)
/* A plan or batched copy needs more than 2^23 workgroups (32 GiB at 4 KiB each) in one launch.
 * Contiguous entry points (scale, reduce) have no such limit: they slice. */
#define HVDHIP_ERR_TOO_LARGE (-4)

/* Flags of hvdhip_fusion_pack(). */
#define HVDHIP_PACK_DEFAULT 0u
/* fp32 -> fp16 packing only: round to half first, then scale the half (the
 * order of the reference pipeline: horovod/torch/compression.py:49-55 followed
 * by the fp16 ScaleBuffer, ops/collective_operations.h:99-127).  The default is
 * scale in fp32, then one rounding to half. */
#define HVDHIP_PACK_CAST_THEN_SCALE 1u

/* How an fp16 buffer is scaled (hvdhip_set_fp16_scale_mode()).  The reference has two
 * arithmetics for it.  Its CPU path (ScaleBufferCPUImpl<unsigned short, float>,
 * ops/collective_operations.h:99-127) widens the element to fp32, multiplies by
 * (float)scale_factor and rounds once to half.  Its CUDA kernels
 * (ops/cuda/cuda_kernels.cu:96-136,167-168,306-309) first round the factor to half,
 * __float2half((float)scale_factor), and multiply half by half with one rounding.  The
 * two agree for factors a half holds exactly (1/8, 0.5, 2 ...) and differ in the last
 * bit of some elements otherwise; test/parallel/test_torch.py:339-445 expects the
 * first for host tensors and the second for device tensors. */
#define HVDHIP_FP16_SCALE_FP32_FACTOR 0 /* default: the CPU path's arithmetic */
#define HVDHIP_FP16_SCALE_HALF_FACTOR 1 /* the CUDA kernels' arithmetic */

/* Kinds for hvdhip_memcpy_async(). */
#define HVDHIP_MEMCPY_H2D 1
#define HVDHIP_MEMCPY_D2H 2
#define HVDHIP_MEMCPY_D2D 3

/* ------------------------------------------------------------------------ */
/* Errors                                                                   */
/* ------------------------------------------------------------------------ */

/* Text for a return code.  For positive codes this is hipGetErrorString(), the
 * text the reference puts into "<op> failed: <text>" (ops/cuda_operations.cc:82-86,
 * ops/hip_operations.cc:62-66).  Never NULL. */
const char* hvdhip_error_string(int code);

/* Detail of the calling thread's most recent failure ("" if none). */
const char* hvdhip_last_error(void);

/* Selects the arithmetic of every later fp16 scale in this process (scale_buffer, the
 * scaled batched copy, pack and unpack of FLOAT16 plans, the cast-then-scale pack and the
 * postscale of the unpack of converting plans): one of HVDHIP_FP16_SCALE_*.  The factor is
 * prepared on the host when a call is made, so calls already queued are not affected.  The
 * fused scale-then-cast pack of converting plans has no counterpart in the reference and
 * always multiplies in fp32 by (float)scale_factor.  hvdhip_get_fp16_scale_mode() returns
 * the current mode. */
int hvdhip_set_fp16_scale_mode(int mode);
int hvdhip_get_fp16_scale_mode(void);

/* Size in bytes of one element, DataType_Size (common/message.cc:66-92); -1 if unknown. */
int64_t hvdhip_dtype_size(int dtype);

/* ------------------------------------------------------------------------ */
/* Device, streams, events: the member set of GPUContext::impl              */
/* (ops/cuda_operations.cc:28-210, ops/hip_operations.cc:27-153,            */
/*  forwarded by ops/gpu_context_impl.cc:1-67)                              */
/* ------------------------------------------------------------------------ */

/* GPUContext::GetDevice / SetDevice, ops/cuda_operations.cc:182-190. */
int hvdhip_get_device(int* device);
int hvdhip_set_device(int device);

/* GPUContext::StreamCreate, ops/cuda_operations.cc:170-176.  The stream is
 * non-blocking with respect to the null stream.  It is created at the default
 * priority (the reference asks for the greatest priority). */
int hvdhip_stream_create(void** stream);
int hvdhip_stream_destroy(void* stream);
/* For a stream that the caller created itself (the framework's, or hipStreamCreate) and is about
 * to destroy: waits for the stream, then drops what the library remembers about it -- the copy
 * tables that launches on it have read (hvdhip_batched_*), its pooled events and the single-layer
 * Adasum plans made for it (hvdhip_adasum_dot_and_norm_sqrds).  hvdhip_stream_destroy does the
 * same for the library's own streams.  A caller's stream that is destroyed without this call
 * must have been idle, and the library then falls back to waiting for the whole device when it
 * next retires a table that the stream had read.  No counterpart in the reference, which keeps
 * its streams for the life of the process (ops/gpu_operations.cc:30-39). */
int hvdhip_stream_forget(void* stream);
/* GPUContext::StreamSynchronize, ops/cuda_operations.cc:178-180. */
int hvdhip_stream_synchronize(void* stream);
/* The framework's ready event is waited for on the Horovod stream, without a
 * host synchronisation: ops/nccl_operations.cc:140-154. */
int hvdhip_stream_wait_event(void* stream, void* event);

/* GetGpuEvent, ops/cuda_operations.cc:28-63: takes an event from the pool
 * kept per (current device, stream); the pool is filled with 128
 * timing-disabled events on first use and grows on demand.  The event is not
 * recorded yet. */
int hvdhip_event_acquire(void* stream, void** event);
/* hipEventRecord on the given stream (GPUContext::RecordEvent, ops/cuda_operations.cc:88-100). */
int hvdhip_event_record(void* event, void* stream);
/* hipEventQuery as used by the polling wait of elastic mode
 * (ops/cuda_operations.cc:116-132): *done = 1 if complete, 0 if not ready;
 * any other HIP status is returned as the error. */
int hvdhip_event_query(void* event, int* done);
/* hipEventSynchronize (ops/cuda_operations.cc:133-140). */
int hvdhip_event_synchronize(void* event);
/* ReleaseGpuEvent, ops/cuda_operations.cc:65-80: back into the pool of
 * (current device, stream). */
int hvdhip_event_release(void* stream, void* event);
/* Number of idle events in the pool of (current device, stream); for tests. */
int hvdhip_event_pool_size(void* stream, int* count);

/* GPUContext::MemcpyAsync{D2D,H2D,D2H}, ops/cuda_operations.cc:192-202. */
int hvdhip_memcpy_async(void* dst, const void* src, size_t count, int kind, void* stream);

/* Timing events for benchmarks (not part of the reference surface): a pair of
 * timing-enabled events bracketing work on one stream. */
int hvdhip_timer_create(void** timer);
int hvdhip_timer_start(void* timer, void* stream);
int hvdhip_timer_stop(void* timer, void* stream);
/* Blocks until the stop event completed; elapsed device time in milliseconds. */
int hvdhip_timer_elapsed_ms(void* timer, float* ms);
int hvdhip_timer_destroy(void* timer);

/* ------------------------------------------------------------------------ */
/* Batched device copies: the launchers of ops/cuda/cuda_kernels.h:29-43    */
/* ------------------------------------------------------------------------ */

/* BatchedD2DMemcpyCudaImpl (ops/cuda/cuda_kernels.h:35, ops/cuda/cuda_kernels.cu:78-84):
 * num_copies independent byte copies out[i] <- in[i] of sizes[i] bytes, in one
 * launch.  out/in/sizes are HOST arrays (the reference passes them by value in
 * BatchedD2DParams); there is no 160-entry limit and no alignment
 * requirement.  Ranges must not overlap each other.  The device-side offset
 * table built from the arrays is cached inside the library and reused when
 * the same arrays are seen again (one table per distinct set of copies, as many
 * as the job cycles through); the first call with a new set stages its table with
 * an asynchronous copy on the same stream and does not wait for the device.
 * When the destinations lie back to back (each begins within 16 bytes after the
 * one before ends: a pack into a fusion buffer) the copy writes through the
 * Infinity Cache as hvdhip_fusion_pack does; otherwise it stores past it.
 * A stream that these entry points have used must be idle when it is destroyed
 * (hvdhip_stream_destroy sees to that itself). */
int hvdhip_batched_d2d_memcpy(void* const* out, const void* const* in, const size_t* sizes,
                              int num_copies, void* stream);

/* Counters of the current device's cache of copy tables, for tests: calls that found their
 * table, calls that built one, tables evicted, tables held now.  Any pointer may be NULL. */
int hvdhip_copy_cache_stats(uint64_t* hits, uint64_t* misses, uint64_t* evictions, uint64_t* entries);
/* Limits of the current device's cache of copy tables: at most max_entries tables (at least 1)
 * and max_bytes of device memory for them; the least recently used go first.  The defaults
 * (4096 tables, 256 MiB) hold every fusion cycle of a multi-billion-parameter step; this call
 * exists so that tests can make eviction happen. */
int hvdhip_copy_cache_set_limits(uint64_t max_entries, uint64_t max_bytes);

/* BatchedScaledD2DMemcpyCudaImpl (ops/cuda/cuda_kernels.h:42, cuda_kernels.cu:289-321):
 * the same copies with every element multiplied by scale_factor.  Arithmetic
 * follows the CPU ScaleBuffer (see hvdhip_scale_buffer); scale_factor == 1.0
 * copies the bytes unchanged, as the CPU path skips scaling at 1.0
 * (ops/gloo_operations.cc:145-148,157-160).  sizes[i] are bytes and must be
 * multiples of the element size; pointers must be element-aligned. */
int hvdhip_batched_scaled_d2d_memcpy(void* const* out, const void* const* in,
                                     const size_t* sizes, int num_copies, double scale_factor,
                                     int dtype, void* stream);

/* ScaleBufferCudaImpl (ops/cuda/cuda_kernels.h:39-40, cuda_kernels.cu:138-187),
 * reached from GPUAllreduce::ScaleBuffer (ops/gpu_operations.cc:334-339) through
 * GPUContext::ScaleBufferImpl (ops/gpu_context_impl.cc:64-67; the ROCm
 * implementation of the reference throws, ops/hip_operations.cc:150-153).
 * out[i] = scale_factor * in[i] over num_elements; in == out is allowed.
 * Arithmetic is that of ScaleBufferCPUImpl (ops/collective_operations.h:91-127):
 * u8/i8/i32/i64/f64 multiply in double and convert back (integers truncate
 * toward zero), f32 multiplies by (float)scale_factor, f16 converts to fp32,
 * multiplies by (float)scale_factor and rounds to nearest even (or, under
 * HVDHIP_FP16_SCALE_HALF_FACTOR, by the factor rounded to half, which is the
 * arithmetic of ScaleBufferCudaImpl itself).  Other dtypes return
 * HVDHIP_ERR_UNSUPPORTED_DTYPE. */
int hvdhip_scale_buffer(const void* fused_input_data, void* buffer_data, int64_t num_elements,
                        double scale_factor, int dtype, void* stream);

/* ------------------------------------------------------------------------ */
/* Fusion buffer plans: GPUAllreduce::{Scale,}Memcpy{In,Out}FusionBuffer     */
/* (ops/gpu_operations.cc:118-168,172-226,238-275,279-324)                  */
/* ------------------------------------------------------------------------ */

/* A plan describes one fused response: n tensors and their outputs (which may
 * alias the tensors, ops/operations.cc:1439-1446), laid out in the fusion
 * buffer at offsets that advance by the entry's size in the buffer dtype
 * rounded up to 16 bytes (ops/gpu_operations.cc:141,254).  The fused tensor
 * set repeats every training step, so the device-side offset and chunk tables
 * are built once here and stay resident.
 *
 * tensor_dtype is the dtype of tensors and outputs; buffer_dtype the dtype of
 * the fusion buffer: equal to tensor_dtype, or FLOAT16 with FLOAT32 tensors,
 * which folds the fp16 compression cast (horovod/torch/compression.py:46-64)
 * into packing and unpacking.  Creating and destroying a plan allocate and
 * free device memory and synchronise; packing and unpacking do not. */
typedef struct hvdhip_fusion_plan hvdhip_fusion_plan;

int hvdhip_fusion_plan_create(const void* const* tensors, void* const* outputs,
                              const int64_t* num_elements, int n, int tensor_dtype,
                              int buffer_dtype, hvdhip_fusion_plan** plan);
int hvdhip_fusion_plan_destroy(hvdhip_fusion_plan* plan);
/* buffer_len as returned by MemcpyInFusionBuffer (padded, ops/gpu_operations.cc:151). */
int64_t hvdhip_fusion_plan_buffer_len(const hvdhip_fusion_plan* plan);
/* Byte offset of every entry in the fusion buffer; offsets has room for n values. */
int hvdhip_fusion_plan_offsets(const hvdhip_fusion_plan* plan, int64_t* offsets);
/* Number of workgroups one pack or unpack launch uses. */
int64_t hvdhip_fusion_plan_num_chunks(const hvdhip_fusion_plan* plan);

/* ScaleMemcpyInFusionBuffer (ops/gpu_operations.cc:172-226), or
 * MemcpyInFusionBuffer (:118-168) when scale_factor == 1.0: one launch copies
 * every tensor to its offset, multiplying by scale_factor and, for a
 * converting plan, rounding fp32 to fp16 (nearest even).  Pad bytes between
 * entries are written as zero so that a reduction over the whole padded
 * buffer reads defined values.  The buffer is written through the device's
 * 256 MB Infinity Cache, where the next kernel or collective on the stream
 * finds it; pass the same buffer for a stream slot every time (the
 * reference keeps one per slot, ops/gpu_operations.cc:122-124), which is
 * also the fastest for this call. */
int hvdhip_fusion_pack(hvdhip_fusion_plan* plan, void* fusion_buffer, double scale_factor,
                       unsigned flags, void* stream);

/* ScaleMemcpyOutFusionBuffer (ops/gpu_operations.cc:279-324), or
 * MemcpyOutFusionBuffer (:238-275) when scale_factor == 1.0.  For a converting
 * plan the scale is applied to the fp16 value (fp32 multiply, rounded back to
 * fp16) and the result widened to fp32, i.e. the reference's postscale on the
 * fp16 buffer followed by Compression.fp16.decompress. */
int hvdhip_fusion_unpack(hvdhip_fusion_plan* plan, const void* fusion_buffer,
                         double scale_factor, void* stream);

/* hvdhip_fusion_unpack followed by hvdhip_event_record(event, stream), i.e. the
 * unpack of a fused response and the completion event that
 * GPUOpContext::FinalizeGPUQueue records behind it (ops/gpu_operations.cc:77-98,
 * ops/cuda_operations.cc:88-100), as one submission: the event is bound to the
 * unpack kernel's own completion signal instead of going onto the stream as a
 * marker behind the kernel.  Query, synchronise and stream-wait see the event
 * exactly as after the two separate calls.  A plan without payload records the
 * event by itself.  Not for a stream that is being captured into a graph. */
int hvdhip_fusion_unpack_record(hvdhip_fusion_plan* plan, const void* fusion_buffer,
                                double scale_factor, void* stream, void* event);

/* ------------------------------------------------------------------------ */
/* Local reduce-sum: one GPU's share of a reduce-scatter                    */
/* ------------------------------------------------------------------------ */

/* resident[i] += incoming[i] for num_elements elements: the arithmetic that
 * ncclAllReduce(ncclSum) (ops/nccl_operations.cc:190-193), gloo::sum<T>
 * (ops/gloo_operations.cc:66-74) and MPI_SUM / float16_sum
 * (ops/mpi_operations.cc:63-66, common/half.cc:44-76) apply to a chunk.  One
 * IEEE add per element for f32/f64; f16 adds in fp32 and rounds to nearest
 * even; integers wrap.  Accepts every dtype except BOOL. */
int hvdhip_reduce_sum(void* resident, const void* incoming, int64_t num_elements, int dtype,
                      void* stream);

/* Accumulates k incoming chunks (1 <= k <= 16) in the order given, rounding to
 * the element type after each one exactly as k successive hvdhip_reduce_sum
 * calls would, in a single pass over memory.  incoming is a HOST array of k
 * device pointers.
 *
 * Where the chunks lie relative to each other shows in the time of this call,
 * and nowhere else: the result does not depend on it.  The memory side
 * interleaves addresses over its channels, and a sum of k + 1 streams asks every
 * channel for k + 1 rows at once; chunks whose start addresses differ by an
 * exact multiple of 8 MiB (the layout of a staging ring cut into power-of-two
 * slots: a 1/8 share of a 64 MiB fusion buffer is 8 MiB) are the slowest
 * placement measured -- 13.2 against 12.8 us for seven fp16 peers on an 8 MiB
 * share, 3 %; up to 10 % has been seen -- while chunks laid back to back, or
 * staggered by a few KiB that are not a power of two, are the fastest.  A
 * caller that stages incoming chunks itself should space them accordingly;
 * issuing the peers' loads in an order that varies from workgroup to workgroup
 * was tried in the kernel and changes nothing. */
int hvdhip_reduce_sum_k(void* resident, const void* const* incoming, int k, int64_t num_elements,
                        int dtype, void* stream);

/* ------------------------------------------------------------------------ */
/* Adasum: Adasum<Comm>::FusedPairwiseReduceWithComm on one device          */
/* (ops/adasum/adasum.h:344-410)                                            */
/* ------------------------------------------------------------------------ */

/* An Adasum plan fixes the split of two equally long vectors into nlayers
 * consecutive slices of tensor_counts[i] elements (the tensor_counts vector of
 * adasum.h:344-351; zero-length slices are legal) and owns the device tables,
 * the per-workgroup partial sums, and the per-layer results.  dtype is
 * FLOAT16, FLOAT32 or FLOAT64 (adasum.h:101-140). */
typedef struct hvdhip_adasum_plan hvdhip_adasum_plan;

int hvdhip_adasum_plan_create(const int* tensor_counts, int nlayers, int dtype,
                              hvdhip_adasum_plan** plan);
int hvdhip_adasum_plan_destroy(hvdhip_adasum_plan* plan);

/* Per layer dot(a,b), |a|^2, |b|^2 accumulated in double
 * (ComputeDotAndNormSqrds, adasum.h:413-426), then the coefficients
 * ca = 1 - dot/|a|^2*0.5 and cb likewise, each 1 when its squared norm is
 * below sqrt(DBL_MIN) (adasum.h:397-404).  Results stay on the device inside
 * the plan.  The summation order is a fixed tree, so results are reproducible
 * from run to run. */
int hvdhip_adasum_dot_norms(hvdhip_adasum_plan* plan, const void* a, const void* b,
                            void* stream);

/* a[i] = ca*a[i] + cb*b[i] per layer with the plan's current coefficients,
 * evaluated in double and rounded once to the element type (ScaledAdd,
 * adasum.h:429-435).  For FLOAT16 the coefficients are narrowed to float and
 * the sum is fma(cb, b, ca*a) in fp32, rounded to half (adasum.h:482-500). */
int hvdhip_adasum_scaled_add(hvdhip_adasum_plan* plan, void* a, const void* b, void* stream);

/* dot_norms followed by scaled_add with no host round trip. */
int hvdhip_adasum_combine(hvdhip_adasum_plan* plan, void* a, const void* b, void* stream);

/* Copies the plan's {dot, |a|^2, |b|^2} (3*nlayers doubles) and/or {ca, cb}
 * (2*nlayers doubles) to host memory after the work queued on stream so far;
 * blocks until the copy is done.  Either pointer may be NULL. */
int hvdhip_adasum_read(hvdhip_adasum_plan* plan, double* normdots, double* coeffs, void* stream);

/* Replaces the plan's coefficients with 2*nlayers host doubles {ca, cb}: the
 * hook for a caller that sums the {dot, norms} triples across ranks before
 * the scaled add (adasum.h:380-382).  Ordered after the work queued on stream. */
int hvdhip_adasum_set_coeffs(hvdhip_adasum_plan* plan, const double* coeffs, void* stream);

/* Adasum::DispatchComputeDotAndNormSqrds (adasum.h:101-122) for one layer:
 * blocks until the three sums are in host memory. */
int hvdhip_adasum_dot_and_norm_sqrds(const void* a, const void* b, int dtype, int count,
                                     double* dot, double* anormsq, double* bnormsq,
                                     void* stream);

/* Adasum::DispatchScaledAdd (adasum.h:124-140) for one layer; asynchronous. */
int hvdhip_adasum_dispatch_scaled_add(int dtype, int count, double acoeff, void* a,
                                      double bcoeff, const void* b, void* stream);

/* hvdhip_adasum_combine for a single layer of count elements, for callers that cannot
 * allocate.  It has no counterpart in the reference: it exists for code under HIP graph
 * capture, tight serving loops and harnesses that forbid hipMalloc, which cannot create the
 * plan (device tables, partial sums) that hvdhip_adasum_combine works from.  The tables and
 * partial sums live in a fixed array of about 0.9 MiB inside the library's device code instead;
 * every device the library runs on holds its copy until the process ends.  The call only
 * launches kernels: no allocation, no free, no copy, no fill, no synchronisation.  (The first
 * call on a device looks the array's address up, which loads the library's device code if
 * nothing else has: make one call, count 0 will do, before capturing a graph.)
 *
 * a and b are device vectors of count elements of dtype (FLOAT16, FLOAT32, FLOAT64); a is
 * updated in place exactly as hvdhip_adasum_combine with a one-layer plan would.  results is
 * NULL or a device pointer to 5 doubles that receive {dot, |a|^2, |b|^2, ca, cb}.
 * Limit: count may need at most 16,384 chunks of 16 KiB, i.e. 2^26 FLOAT32, 2^27 FLOAT16 or
 * 2^25 FLOAT64 elements (256 MiB per vector); beyond that HVDHIP_ERR_TOO_LARGE is returned and
 * nothing is launched.  All calls on one device share the one array, which keeps the last
 * call's contents; the library therefore orders the calls on a device one behind the other,
 * whatever streams and threads they come from: a call records an event (made once per device,
 * with the address look-up) behind its last kernel, and a call on another stream first makes its
 * stream wait for that event.  The exception is a stream that is being captured: a capture can
 * neither wait for an event from outside it nor record one for later calls, so a call under
 * capture takes no part in that ordering, and whoever launches the graph keeps it apart from
 * other calls on the device (replays of one graph, or of graphs on one stream, are ordered by
 * the stream). */
int hvdhip_adasum_combine_static(void* a, const void* b, int dtype, int count, double* results,
                                 void* stream);

#ifdef __cplusplus
}
#endif

#endif /* HVDHIP_H */
