// vecmem.h -- lane-level vector access to global memory (device code).
//
// A lane moves N elements of T as one 16- or 8-byte instruction whose address
// needs only the alignment of a single T: gfx950 serves multi-dword global
// accesses at any alignment, so callers need no alignment ladder and no head
// peeling, and naturally aligned data costs nothing extra.
#ifndef HVDHIP_VECMEM_H
#define HVDHIP_VECMEM_H

#include <hip/hip_runtime.h>

#include <cstdint>

namespace hvdhip {

typedef _Float16 half_t;

// Pointer into global (device) memory.  Addresses that arrive as integers
// from a table would otherwise be generic pointers and use flat instructions.
template <typename T>
using gptr = __attribute__((address_space(1))) T*;

template <typename T>
__device__ __forceinline__ gptr<T> as_global(uint64_t addr) {
  return reinterpret_cast<gptr<T>>(addr);
}
template <typename T>
__device__ __forceinline__ gptr<T> as_global(T* p) {
  return reinterpret_cast<gptr<T>>(reinterpret_cast<uint64_t>(p));
}

template <int BYTES>
struct RawSel;
template <>
struct RawSel<16> {
  typedef uint32_t type __attribute__((ext_vector_type(4)));
};
template <>
struct RawSel<8> {
  typedef uint32_t type __attribute__((ext_vector_type(2)));
};
// The same register type, declared with the alignment of one element.
template <int BYTES, int ALIGN>
struct Raw {
  typedef typename RawSel<BYTES>::type type __attribute__((aligned(ALIGN)));
};

// Returns x unchanged but hides where it came from.  Used between an fp32
// operation and a narrowing to fp16: without it the compiler fuses the pair
// into one mixed-precision fma with a +0 addend, which turns a -0 product
// into +0.  No instruction is emitted.
__device__ __forceinline__ float opaque(float x) {
  asm("" : "+v"(x));
  return x;
}

// N elements of T held in registers.
template <typename T, int N>
struct Arr {
  T v[N];
};

// Streaming data is touched once: the non-temporal hint keeps it from
// displacing useful lines in L2 and the Infinity Cache (+5-15 % measured against plain accesses).

// NT = false loads without the hint, for data that a later kernel reads again while it can
// still be in the Infinity Cache.
template <typename T, int N, bool NT = true>
__device__ __forceinline__ Arr<T, N> ldv(gptr<const T> p) {
  if constexpr (sizeof(T) * N == 32) {  // two 16-byte accesses
    Arr<T, N> out;
    const Arr<T, N / 2> lo = ldv<T, N / 2, NT>(p), hi = ldv<T, N / 2, NT>(p + N / 2);
    __builtin_memcpy(out.v, lo.v, 16);
    __builtin_memcpy(out.v + N / 2, hi.v, 16);
    return out;
  } else {
  typedef typename Raw<(int)sizeof(T) * N, (int)alignof(T)>::type R;
  typename RawSel<(int)sizeof(T) * N>::type r;
  if constexpr (NT) {
    r = __builtin_nontemporal_load(reinterpret_cast<gptr<const R>>(p));
  } else {
    r = *reinterpret_cast<gptr<const R>>(p);
  }
  return __builtin_bit_cast(Arr<T, N>, r);
  }
}

template <typename T, int N>
__device__ __forceinline__ void stv(gptr<T> p, const Arr<T, N>& a) {
  typedef typename Raw<(int)sizeof(T) * N, (int)alignof(T)>::type R;
  __builtin_nontemporal_store(__builtin_bit_cast(typename RawSel<(int)sizeof(T) * N>::type, a),
                              reinterpret_cast<gptr<R>>(p));
}

// Loads of one-byte elements.  The compiler drops the non-temporal hint from a vector load that
// is only byte-aligned (the instruction stays a 16-byte global load, the hint is gone), which
// costs the byte-typed kernels 15 % of their throughput.  A raw buffer load carries its cache
// policy as an immediate and has no alignment to declare, so byte elements are read through a
// window over the workgroup's source range (uniform base in scalar registers, byte offset per lane).
struct ReadWindow {
  __amdgpu_buffer_rsrc_t rsrc;
};

template <typename T>
__device__ __forceinline__ ReadWindow load_window(gptr<const T> base, uint32_t bytes) {
  ReadWindow w;
  w.rsrc = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(reinterpret_cast<uint64_t>(base)), 0,
                                             (int)bytes, 0x00020000);
  return w;
}

// Sixteen bytes at byte offset `off` of the window, non-temporal.
template <typename T, int N>
__device__ __forceinline__ Arr<T, N> ldw(const ReadWindow& w, uint32_t off) {
  static_assert(sizeof(T) * N == 16, "one 16-byte access");
  constexpr int kNonTemporal = 2;  // the nt bit of a buffer instruction's cache policy
  return __builtin_bit_cast(Arr<T, N>, __builtin_amdgcn_raw_buffer_load_b128(w.rsrc, (int)off, 0, kNonTemporal));
}

// How a streaming kernel stores.
//   kStoreNT: non-temporal global stores (the lines bypass the Infinity Cache on their way out).
//   kStoreWT: raw buffer stores with the sc0 and sc1 bits, which write the lines through L2 at once
//             and install them in the Infinity Cache, where the next kernel finds them.
// Which one streams faster depends on the kernel and on what runs around it (measured per kernel
// family; the table is in context.cc).  Plain stores, which leave the lines in L2 until they are
// written back, are slower than either once the data is not all zeros (a 62 MB reduce-sum: 29.8 us
// against 29.3 and 29.8; with zeros everywhere they measure 27.0 us, which is worth knowing before
// trusting a microbenchmark on freshly cleared memory) and cost a pipeline 4-7 %.
enum StorePolicy : int { kStoreNT = 0, kStoreWT = 1 };

// A window over a workgroup's destination range.  A buffer instruction takes its cache policy as
// an immediate, which is why the write-through path uses one; the window's base must be uniform
// over the wavefront (the resource lives in scalar registers), and stores beyond `bytes` are
// dropped by the hardware's range check.
struct Window {
  __amdgpu_buffer_rsrc_t rsrc;
  uint64_t base;
};

template <int ST, typename T>
__device__ __forceinline__ Window store_window(gptr<T> base, uint32_t bytes) {
  Window w;
  w.base = reinterpret_cast<uint64_t>(base);
  if constexpr (ST == kStoreWT) {
    // word 3: 32-bit data format, raw (unstrided, untyped) addressing
    w.rsrc = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(w.base), 0, (int)bytes, 0x00020000);
  }
  return w;
}

// Stores N elements of T at byte offset `off` of the window.
template <int ST, typename T, int N>
__device__ __forceinline__ void stw(const Window& w, uint32_t off, const Arr<T, N>& a) {
  if constexpr (sizeof(T) * N == 32) {  // two 16-byte accesses
    Arr<T, N / 2> lo, hi;
    __builtin_memcpy(lo.v, a.v, 16);
    __builtin_memcpy(hi.v, a.v + N / 2, 16);
    stw<ST, T, N / 2>(w, off, lo);
    stw<ST, T, N / 2>(w, off + 16, hi);
  } else if constexpr (ST == kStoreWT) {
    typedef typename RawSel<(int)sizeof(T) * N>::type R;
    // sc0 | sc1.  (sc1 alone measures the same, no bit at all -- plain write-back -- gains a third
    // as much, and sc1 with nt loses 5 % against non-temporal stores.)
    constexpr int kScopeBits = 1 | 16;
    const R r = __builtin_bit_cast(R, a);
    if constexpr (sizeof(T) * N == 16) {
      __builtin_amdgcn_raw_buffer_store_b128(r, w.rsrc, (int)off, 0, kScopeBits);
    } else {
      __builtin_amdgcn_raw_buffer_store_b64(r, w.rsrc, (int)off, 0, kScopeBits);
    }
  } else {
    stv<T, N>(reinterpret_cast<gptr<T>>(w.base + off), a);
  }
}

}  // namespace hvdhip

#endif  // HVDHIP_VECMEM_H
