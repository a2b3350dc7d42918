// internal.h -- shared declarations of the hvdhip library (not installed).
#ifndef HVDHIP_INTERNAL_H
#define HVDHIP_INTERNAL_H

#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <string>
#include <vector>

#include "hvdhip.h"

namespace hvdhip {

// Records a message for hvdhip_last_error() on the calling thread and returns code.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
// Clears the calling thread's message; returns 0.
int ok();

// Evaluates a HIP call; on failure records "<call> failed: <text>" and returns
// the hipError_t value from the enclosing function.
#define HVDHIP_CHECK(call)                                                          \
  do {                                                                              \
    hipError_t hvdhip_e_ = (call);                                                  \
    if (hvdhip_e_ != hipSuccess) {                                                  \
      (void)hipGetLastError(); /* the code is returned; leave no stale error behind */ \
      return ::hvdhip::fail((int)hvdhip_e_, "%s failed: %s", #call,                 \
                            hipGetErrorString(hvdhip_e_));                          \
    }                                                                               \
  } while (0)

// Checks the launch that has just been issued.
#define HVDHIP_CHECK_LAUNCH(name)                                                   \
  do {                                                                              \
    hipError_t hvdhip_e_ = hipGetLastError();                                       \
    if (hvdhip_e_ != hipSuccess)                                                    \
      return ::hvdhip::fail((int)hvdhip_e_, "%s launch failed: %s", name,           \
                            hipGetErrorString(hvdhip_e_));                          \
  } while (0)

inline int64_t dtype_size(int dtype) {
  switch (dtype) {
  case HVDHIP_UINT8: case HVDHIP_INT8: case HVDHIP_BOOL: return 1;
  case HVDHIP_UINT16: case HVDHIP_INT16: case HVDHIP_FLOAT16: return 2;
  case HVDHIP_INT32: case HVDHIP_FLOAT32: return 4;
  case HVDHIP_INT64: case HVDHIP_FLOAT64: return 8;
  default: return -1;
  }
}

// Threads per workgroup of every streaming kernel: four wave64 wavefronts.
constexpr int kWG = 256;

// Bytes of the wider side that one workgroup moves.  Read once from
// HVDHIP_CHUNK_BYTES (a multiple of 4096), default kDefaultChunkBytes.
constexpr uint32_t kDefaultChunkBytes = 32768;
uint32_t chunk_bytes();

// One contiguous run of elements to transfer.  `tensor` and `output` are
// absolute device addresses; `off` is a byte offset into the fusion buffer
// whose base address is given at launch.  `n` counts elements.
struct Seg {
  uint64_t tensor;
  uint64_t output;
  uint64_t off;
  uint64_t n;
};

// One workgroup's share: chunk number `idx` (in units of chunk_units
// elements) of segment `seg`.
struct Chunk {
  uint32_t seg;
  uint32_t idx;
};

// Device-resident segment and chunk tables of one plan.
struct DevTables {
  void* alloc = nullptr;  // one allocation holding both tables
  Seg* segs = nullptr;
  Chunk* chunks = nullptr;
  uint32_t nsegs = 0;
  uint32_t nchunks = 0;
  uint32_t chunk_units = 0;  // elements per chunk
};

// Builds the chunk table for `segs`, with chunk_units elements per chunk, and
// uploads both tables (allocates; synchronous).  Zero-length segments get no
// chunk.
int build_tables(const std::vector<Seg>& segs, uint32_t chunk_units, DevTables* out);
int free_tables(DevTables* t);

}  // namespace hvdhip

#endif  // HVDHIP_INTERNAL_H
