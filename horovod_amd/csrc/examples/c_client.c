/* c_client.c -- the library from plain C: no C++, no torch, no Python.
 *
 * Three tensors of different lengths are packed into a fusion buffer with a
 * prescale, summed with one peer buffer, and unpacked with a postscale, then
 * compared on the host with the same arithmetic in float.  Also times the host
 * side of one hvdhip_fusion_pack() call.
 *
 *   gcc -std=c99 -D__HIP_PLATFORM_AMD__ -I/opt/rocm/include -I../../include c_client.c \
 *       -L../lib -lhvdhip -L/opt/rocm/lib -lamdhip64 -Wl,-rpath,'$ORIGIN' -o ../lib/c_client   (what `make` in horovod_amd/csrc runs)
 */
#define _POSIX_C_SOURCE 199309L
#include <hip/hip_runtime_api.h>
#include <stdio.h>
#include <stdlib.h>
#include <time.h>

#include "hvdhip.h"

#define CHECK_HIP(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { \
  fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_)); return 2; } } while (0)
#define CHECK_HVD(x) do { int r_ = (x); if (r_ != 0) { \
  fprintf(stderr, "%s: %s (%s)\n", #x, hvdhip_error_string(r_), hvdhip_last_error()); return 3; } } while (0)

static double now_us(void) {
  struct timespec t;
  clock_gettime(CLOCK_MONOTONIC, &t);
  return t.tv_sec * 1e6 + t.tv_nsec * 1e-3;
}

int main(void) {
  enum { N = 3 };
  const int64_t counts[N] = {5, 70001, 4096};
  float* host[N];
  const void* tensors[N];
  void* outputs[N];
  int i;
  int64_t j, total = 0;
  for (i = 0; i < N; ++i) {
    void *t, *o;
    host[i] = (float*)malloc((size_t)counts[i] * sizeof(float));
    for (j = 0; j < counts[i]; ++j) host[i][j] = (float)((j * 37 + i * 11) % 201 - 100) * 0.25f;
    CHECK_HIP(hipMalloc(&t, (size_t)counts[i] * sizeof(float)));
    CHECK_HIP(hipMalloc(&o, (size_t)counts[i] * sizeof(float)));
    CHECK_HIP(hipMemcpy(t, host[i], (size_t)counts[i] * sizeof(float), hipMemcpyHostToDevice));
    tensors[i] = t;
    outputs[i] = o;
    total += counts[i];
  }

  hvdhip_fusion_plan* plan = NULL;
  CHECK_HVD(hvdhip_fusion_plan_create(tensors, outputs, counts, N, HVDHIP_FLOAT32, HVDHIP_FLOAT32, &plan));
  const int64_t len = hvdhip_fusion_plan_buffer_len(plan);
  int64_t offsets[N];
  CHECK_HVD(hvdhip_fusion_plan_offsets(plan, offsets));

  void *fusion = NULL, *peer = NULL, *stream = NULL;
  CHECK_HIP(hipMalloc(&fusion, (size_t)len));
  CHECK_HIP(hipMalloc(&peer, (size_t)len));
  float* peer_host = (float*)calloc((size_t)len / sizeof(float), sizeof(float));
  for (j = 0; j < len / (int64_t)sizeof(float); ++j) peer_host[j] = (float)(j % 17) - 8.0f;
  CHECK_HIP(hipMemcpy(peer, peer_host, (size_t)len, hipMemcpyHostToDevice));
  CHECK_HVD(hvdhip_stream_create(&stream));

  CHECK_HVD(hvdhip_fusion_pack(plan, fusion, 0.125, HVDHIP_PACK_DEFAULT, stream));
  CHECK_HVD(hvdhip_reduce_sum(fusion, peer, len / (int64_t)sizeof(float), HVDHIP_FLOAT32, stream));
  CHECK_HVD(hvdhip_fusion_unpack(plan, fusion, 0.5, stream));
  CHECK_HVD(hvdhip_stream_synchronize(stream));

  long bad = 0;
  for (i = 0; i < N; ++i) {
    float* got = (float*)malloc((size_t)counts[i] * sizeof(float));
    CHECK_HIP(hipMemcpy(got, outputs[i], (size_t)counts[i] * sizeof(float), hipMemcpyDeviceToHost));
    for (j = 0; j < counts[i]; ++j) {
      volatile float scaled = 0.125f * host[i][j];               /* one rounding per step, as on the device */
      volatile float summed = scaled + peer_host[offsets[i] / (int64_t)sizeof(float) + j];
      volatile float want = 0.5f * summed;
      if (got[j] != want) ++bad;
    }
    free(got);
  }

  /* host cost of queueing one pack */
  const int reps = 2000;
  double t0 = now_us();
  for (i = 0; i < reps; ++i) CHECK_HVD(hvdhip_fusion_pack(plan, fusion, 0.125, HVDHIP_PACK_DEFAULT, stream));
  double t1 = now_us();
  CHECK_HVD(hvdhip_stream_synchronize(stream));
  double t2 = now_us();

  printf("c_client: %lld elements in %d tensors, buffer_len %lld, mismatches %ld\n", (long long)total, N,
         (long long)len, bad);
  printf("c_client: hvdhip_fusion_pack host time %.2f us per call (%.2f us per call until the stream drained)\n",
         (t1 - t0) / reps, (t2 - t0) / reps);

  CHECK_HVD(hvdhip_fusion_plan_destroy(plan));
  CHECK_HVD(hvdhip_stream_destroy(stream));
  return bad == 0 ? 0 : 1;
}
