/* cache_stress.cc -- the library's host-side bookkeeping under load, from a native program:
 * the copy-table cache with limits so small that every call evicts (two threads on two streams,
 * a stream destroyed while tables remember it), the same cache at its default size (every set
 * misses once and hits afterwards), the single-layer Adasum plans beyond their capacity from two
 * threads, plan and event lifetimes, and the entry point that allocates nothing.  Passes when
 * every call succeeds and the cache counters add up.  Built without a sanitizer by the Makefile;
 * it is also the program to link against a host-AddressSanitizer build of the library
 * (hipcc ... -Xarch_host -fsanitize=address), which needs no preloaded runtime that way. */
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include <thread>
#include <unistd.h>
#include <vector>
#include "hvdhip.h"
#define CK(x) do { int rc_ = (x); if (rc_) { printf("FAIL %s -> %d (%s)\n", #x, rc_, hvdhip_last_error()); exit(1); } } while (0)
#define HK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("HIP FAIL %s -> %s\n", #x, hipGetErrorString(e_)); exit(1); } } while (0)

static void copy_sets(void* stream, char* src, char* dst, size_t arena, int sets, int per_set, unsigned seed) {
  std::vector<void*> out(per_set); std::vector<const void*> in(per_set); std::vector<size_t> sz(per_set);
  for (int round = 0; round < 3; ++round) {
    for (int s = 0; s < sets; ++s) {
      srand(seed + s);
      size_t at = 0;
      for (int i = 0; i < per_set; ++i) {
        size_t n = 4 * (1 + rand() % 3000);
        if (at + n > arena) n = 4;
        out[i] = dst + at; in[i] = src + at; sz[i] = n; at += (n + 255) / 256 * 256;
      }
      CK(hvdhip_batched_d2d_memcpy(out.data(), in.data(), sz.data(), per_set, stream));
      CK(hvdhip_batched_scaled_d2d_memcpy(out.data(), in.data(), sz.data(), per_set, 0.5, HVDHIP_FLOAT32, stream));
    }
  }
}

int main() {
  setvbuf(stdout, nullptr, _IONBF, 0);
  void *s1, *s2;
  CK(hvdhip_stream_create(&s1)); CK(hvdhip_stream_create(&s2));
  const size_t arena = 64u << 20;
  char *src, *dst1, *dst2;
  HK(hipMalloc(&src, arena)); HK(hipMalloc(&dst1, arena)); HK(hipMalloc(&dst2, arena));
  HK(hipMemset(src, 0, arena));
  // 1. copy-table cache: tiny limits so that every call evicts, two threads on two streams
  CK(hvdhip_copy_cache_set_limits(5, 1 << 20));
  std::thread t1(copy_sets, s1, src, dst1, arena, 40, 50, 1u), t2(copy_sets, s2, src, dst2, arena, 40, 50, 7u);
  t1.join(); t2.join();
  uint64_t h, m, e, n; CK(hvdhip_copy_cache_stats(&h, &m, &e, &n));
  printf("copy cache, 5 entries: hits %llu misses %llu evictions %llu entries %llu\n", (unsigned long long)h, (unsigned long long)m, (unsigned long long)e, (unsigned long long)n);
  if (h + m != 480 || n > 5 || e != m - n) { printf("FAIL: counters do not add up\n"); return 1; }
  // the same stream destroyed while entries remember it, then more evictions
  CK(hvdhip_stream_destroy(s2)); CK(hvdhip_stream_create(&s2));
  copy_sets(s1, src, dst1, arena, 20, 10, 99u);
  CK(hvdhip_copy_cache_set_limits(4096, 256u << 20));
  uint64_t h0, m0, e0;
  CK(hvdhip_copy_cache_stats(&h0, &m0, &e0, &n));
  copy_sets(s2, src, dst2, arena, 120, 30, 5u);
  CK(hvdhip_copy_cache_stats(&h, &m, &e, &n));
  printf("copy cache, default limits: hits +%llu misses +%llu evictions +%llu entries %llu\n", (unsigned long long)(h - h0), (unsigned long long)(m - m0), (unsigned long long)(e - e0), (unsigned long long)n);
  if (m - m0 != 240 || h - h0 != 480 || e != e0) { printf("FAIL: 120 sets x 2 kinds must miss once and hit twice\n"); return 1; }
  // 2. single-layer Adasum cache: more distinct counts than it holds, two threads
  auto adasum = [&](void* st, float* a, float* b, int base) {
    for (int i = 0; i < 300; ++i) {
      double d, an, bn;
      CK(hvdhip_adasum_dot_and_norm_sqrds(a, b, HVDHIP_FLOAT32, base + i * 17, &d, &an, &bn, st));
      CK(hvdhip_adasum_dispatch_scaled_add(HVDHIP_FLOAT32, base + i * 17, 0.5, a, 0.5, b, st));
    }
  };
  std::thread a1(adasum, s1, (float*)dst1, (float*)src, 1), a2(adasum, s2, (float*)dst2, (float*)src, 5);
  a1.join(); a2.join();
  // 3. plans: create, use, destroy; empty plan; many layers
  for (int rep = 0; rep < 20; ++rep) {
    std::vector<int> counts(100 + rep);
    for (size_t i = 0; i < counts.size(); ++i) counts[i] = (int)((i * 7919 + rep) % 5000);
    hvdhip_adasum_plan* p; CK(hvdhip_adasum_plan_create(counts.data(), (int)counts.size(), HVDHIP_FLOAT32, &p));
    CK(hvdhip_adasum_combine(p, dst1, src, s1));
    std::vector<double> nd(3 * counts.size()), co(2 * counts.size());
    CK(hvdhip_adasum_read(p, nd.data(), co.data(), s1));
    CK(hvdhip_adasum_plan_destroy(p));
    std::vector<const void*> tin(counts.size()); std::vector<void*> tout(counts.size()); std::vector<int64_t> c64(counts.size());
    size_t at = 0;
    for (size_t i = 0; i < counts.size(); ++i) { tin[i] = src + at; tout[i] = dst2 + at; c64[i] = counts[i]; at += ((size_t)counts[i] * 4 + 255) / 256 * 256; }
    hvdhip_fusion_plan* fp; CK(hvdhip_fusion_plan_create(tin.data(), tout.data(), c64.data(), (int)counts.size(), HVDHIP_FLOAT32, HVDHIP_FLOAT32, &fp));
    CK(hvdhip_fusion_pack(fp, dst1, 0.125, HVDHIP_PACK_DEFAULT, s1));
    void* ev; CK(hvdhip_event_acquire(s1, &ev));
    CK(hvdhip_fusion_unpack_record(fp, dst1, 1.0, s1, ev));
    CK(hvdhip_event_synchronize(ev)); CK(hvdhip_event_release(s1, ev));
    CK(hvdhip_fusion_plan_destroy(fp));
  }
  // 4. the entry point that allocates nothing, twice
  double* res; HK(hipMalloc(&res, 64));
  CK(hvdhip_adasum_combine_static(dst1, src, HVDHIP_FLOAT32, 1 << 20, res, s1));
  CK(hvdhip_adasum_combine_static(dst1, src, HVDHIP_FLOAT32, 1000, nullptr, s1));
  CK(hvdhip_stream_synchronize(s1)); CK(hvdhip_stream_synchronize(s2));
  CK(hvdhip_stream_destroy(s1)); CK(hvdhip_stream_destroy(s2));
  HK(hipFree(src)); HK(hipFree(dst1)); HK(hipFree(dst2)); HK(hipFree(res));
  printf("stress ok\n");
  _exit(0);  // the runtime's own teardown trips a check inside this sanitizer runtime
}
