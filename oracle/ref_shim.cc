// ref_shim.cc -- C entry points over the reference's own fp16 routines.
//
// TEST INFRASTRUCTURE ONLY.  This file contains no reference code: it
// includes horovod/common/half.h from the read-only reference tree by path
// (given with -I on the command line) and is linked with the reference's own
// common/half.cc compiled in place.  The result, oracle/_ref/libhvdref.so, is
// used by the tests to validate the restatement in hvd_oracle.c.  It can only
// be built where the reference tree is mounted.
//
// The rest of the path (ScaleBufferCPUImpl in ops/collective_operations.h,
// Adasum in ops/adasum/adasum.h, FuseResponses in controller.cc) includes
// common.h / global_state.h, which need Eigen, Boost.Lockfree and FlatBuffers
// headers that are not present, so it is not buildable here.
#include <cstdint>

#include "half.h"  // horovod/common/half.h

using horovod::common::Float2HalfBits;
using horovod::common::HalfBits2Float;

extern "C" {

// HalfBits2Float, common/half.h:43-77
void ref_half2float(const uint16_t* src, float* dst, int64_t n) {
  for (int64_t i = 0; i < n; ++i) HalfBits2Float(src + i, dst + i);
}

// Float2HalfBits, common/half.h:79-139
void ref_float2half(const float* src, uint16_t* dst, int64_t n) {
  for (int64_t i = 0; i < n; ++i) Float2HalfBits(src + i, dst + i);
}

// float16_sum, common/half.cc:44-76 (the MPI user-op signature)
void ref_float16_sum(const uint16_t* in, uint16_t* inout, int64_t len) {
  while (len > 0) {
    int chunk = len > (1 << 30) ? (1 << 30) : (int)len;
    MPI_Datatype dt = MPI_DATATYPE_NULL;
    horovod::common::float16_sum((void*)in, (void*)inout, &chunk, &dt);
    in += chunk;
    inout += chunk;
    len -= chunk;
  }
}

}  // extern "C"
