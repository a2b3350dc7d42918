"""Thin Python handles over the C ABI, for tests and benchmarks.

Device memory comes from the caller (torch tensors here, the framework in
Horovod); these classes only pass raw addresses through.
"""
import array
import ctypes
from ctypes import c_double, c_float, c_int, c_int64, c_size_t, c_void_p

from ._lib import DTYPE, check, lib


def _ptr_array(values):
    """A C array of addresses; through array.array, which converts a list several times faster
    than filling a ctypes array element by element."""
    raw = array.array("Q", values)
    return (c_void_p * len(raw)).from_buffer(raw) if len(raw) else (c_void_p * 0)()


def _size_array(values):
    raw = array.array("Q", values)
    return (c_size_t * len(raw)).from_buffer(raw) if len(raw) else (c_size_t * 0)()


class Stream:
    """A stream of the library (GPUContext::StreamCreate)."""

    def __init__(self, handle=None):
        """Creates a stream, or wraps an existing hipStream_t address (not owned)."""
        self.owned = handle is None
        if handle is None:
            h = c_void_p()
            check(lib().hvdhip_stream_create(ctypes.byref(h)), "hvdhip_stream_create")
            self.handle = h
        else:
            self.handle = c_void_p(handle)

    def synchronize(self):
        check(lib().hvdhip_stream_synchronize(self.handle), "hvdhip_stream_synchronize")

    def destroy(self):
        if self.handle is not None and self.owned:
            check(lib().hvdhip_stream_destroy(self.handle), "hvdhip_stream_destroy")
        self.handle = None


class Timer:
    def __init__(self):
        h = c_void_p()
        check(lib().hvdhip_timer_create(ctypes.byref(h)), "hvdhip_timer_create")
        self.handle = h

    def start(self, stream):
        check(lib().hvdhip_timer_start(self.handle, stream.handle), "hvdhip_timer_start")

    def stop(self, stream):
        check(lib().hvdhip_timer_stop(self.handle, stream.handle), "hvdhip_timer_stop")

    def elapsed_ms(self):
        ms = c_float()
        check(lib().hvdhip_timer_elapsed_ms(self.handle, ctypes.byref(ms)), "hvdhip_timer_elapsed_ms")
        return ms.value

    def destroy(self):
        if self.handle is not None:
            lib().hvdhip_timer_destroy(self.handle)
            self.handle = None


class FusionPlan:
    """One fused response: tensors -> fusion buffer -> outputs."""

    def __init__(self, tensor_ptrs, output_ptrs, num_elements, tensor_dtype, buffer_dtype=None):
        if buffer_dtype is None:
            buffer_dtype = tensor_dtype
        n = len(tensor_ptrs)
        self.n = n
        counts = (c_int64 * n)(*num_elements)
        h = c_void_p()
        check(lib().hvdhip_fusion_plan_create(_ptr_array(tensor_ptrs), _ptr_array(output_ptrs), counts, n,
                                              int(tensor_dtype), int(buffer_dtype), ctypes.byref(h)),
              "hvdhip_fusion_plan_create")
        self.handle = h
        self.buffer_len = lib().hvdhip_fusion_plan_buffer_len(h)
        self.num_chunks = lib().hvdhip_fusion_plan_num_chunks(h)

    def offsets(self):
        out = (c_int64 * self.n)()
        check(lib().hvdhip_fusion_plan_offsets(self.handle, out), "hvdhip_fusion_plan_offsets")
        return list(out)

    def pack(self, buffer_ptr, scale, stream, flags=0):
        check(lib().hvdhip_fusion_pack(self.handle, buffer_ptr, float(scale), flags, stream.handle),
              "hvdhip_fusion_pack")

    def unpack(self, buffer_ptr, scale, stream, event=None):
        """event: a pooled event (ctypes.c_void_p) to be recorded behind the unpack as part of its launch."""
        if event is not None:
            check(lib().hvdhip_fusion_unpack_record(self.handle, buffer_ptr, float(scale), stream.handle, event),
                  "hvdhip_fusion_unpack_record")
            return
        check(lib().hvdhip_fusion_unpack(self.handle, buffer_ptr, float(scale), stream.handle),
              "hvdhip_fusion_unpack")

    def destroy(self):
        if self.handle is not None:
            check(lib().hvdhip_fusion_plan_destroy(self.handle), "hvdhip_fusion_plan_destroy")
            self.handle = None


class AdasumPlan:
    """Layer split of two vectors for the Adasum pairwise combine."""

    def __init__(self, tensor_counts, dtype):
        n = len(tensor_counts)
        self.nlayers = n
        counts = (c_int * n)(*[int(c) for c in tensor_counts])
        h = c_void_p()
        check(lib().hvdhip_adasum_plan_create(counts, n, int(dtype), ctypes.byref(h)),
              "hvdhip_adasum_plan_create")
        self.handle = h

    def dot_norms(self, a_ptr, b_ptr, stream):
        check(lib().hvdhip_adasum_dot_norms(self.handle, a_ptr, b_ptr, stream.handle), "hvdhip_adasum_dot_norms")

    def scaled_add(self, a_ptr, b_ptr, stream):
        check(lib().hvdhip_adasum_scaled_add(self.handle, a_ptr, b_ptr, stream.handle), "hvdhip_adasum_scaled_add")

    def combine(self, a_ptr, b_ptr, stream):
        check(lib().hvdhip_adasum_combine(self.handle, a_ptr, b_ptr, stream.handle), "hvdhip_adasum_combine")

    def read(self, stream):
        nd = (c_double * (3 * self.nlayers))()
        co = (c_double * (2 * self.nlayers))()
        check(lib().hvdhip_adasum_read(self.handle, nd, co, stream.handle), "hvdhip_adasum_read")
        return list(nd), list(co)

    def set_coeffs(self, coeffs, stream):
        arr = (c_double * (2 * self.nlayers))(*coeffs)
        check(lib().hvdhip_adasum_set_coeffs(self.handle, arr, stream.handle), "hvdhip_adasum_set_coeffs")

    def destroy(self):
        if self.handle is not None:
            check(lib().hvdhip_adasum_plan_destroy(self.handle), "hvdhip_adasum_plan_destroy")
            self.handle = None


def batched_d2d_memcpy(out_ptrs, in_ptrs, sizes, stream):
    n = len(sizes)
    check(lib().hvdhip_batched_d2d_memcpy(_ptr_array(out_ptrs), _ptr_array(in_ptrs), _size_array(sizes), n,
                                          stream.handle), "hvdhip_batched_d2d_memcpy")


def batched_scaled_d2d_memcpy(out_ptrs, in_ptrs, sizes, scale, dtype, stream):
    n = len(sizes)
    check(lib().hvdhip_batched_scaled_d2d_memcpy(_ptr_array(out_ptrs), _ptr_array(in_ptrs),
                                                 _size_array(sizes), n, float(scale), int(dtype),
                                                 stream.handle), "hvdhip_batched_scaled_d2d_memcpy")


def scale_buffer(in_ptr, out_ptr, n, scale, dtype, stream):
    check(lib().hvdhip_scale_buffer(in_ptr, out_ptr, n, float(scale), int(dtype), stream.handle),
          "hvdhip_scale_buffer")


def reduce_sum(resident_ptr, incoming_ptr, n, dtype, stream):
    check(lib().hvdhip_reduce_sum(resident_ptr, incoming_ptr, n, int(dtype), stream.handle), "hvdhip_reduce_sum")


def reduce_sum_k(resident_ptr, incoming_ptrs, n, dtype, stream):
    check(lib().hvdhip_reduce_sum_k(resident_ptr, _ptr_array(incoming_ptrs), len(incoming_ptrs), n, int(dtype),
                                    stream.handle), "hvdhip_reduce_sum_k")


FP16_SCALE_FP32_FACTOR = 0  # ScaleBufferCPUImpl<unsigned short, float>, ops/collective_operations.h:99-127
FP16_SCALE_HALF_FACTOR = 1  # scale_buffer_k<__half>, ops/cuda/cuda_kernels.cu:96-136,167


def set_fp16_scale_mode(mode):
    check(lib().hvdhip_set_fp16_scale_mode(int(mode)), "hvdhip_set_fp16_scale_mode")


def get_fp16_scale_mode():
    return int(lib().hvdhip_get_fp16_scale_mode())


__all__ = ["Stream", "Timer", "FusionPlan", "AdasumPlan", "batched_d2d_memcpy", "batched_scaled_d2d_memcpy",
           "scale_buffer", "reduce_sum", "reduce_sum_k", "DTYPE", "FP16_SCALE_FP32_FACTOR", "FP16_SCALE_HALF_FACTOR",
           "set_fp16_scale_mode", "get_fp16_scale_mode"]
