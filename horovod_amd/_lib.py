"""ctypes binding of libhvdhip.so: one prototype per function of include/hvdhip.h."""
import ctypes
import os
from ctypes import (POINTER, c_char_p, c_double, c_float, c_int, c_int64, c_size_t,
                    c_uint, c_uint64, c_void_p)

_HERE = os.path.dirname(os.path.abspath(__file__))

# horovod::common::DataType values (common/message.h:30-41 of the reference).
DTYPE = {
    "uint8": 0, "int8": 1, "uint16": 2, "int16": 3, "int32": 4, "int64": 5,
    "float16": 6, "float32": 7, "float64": 8, "bool": 9,
}
_SIZES = {0: 1, 1: 1, 2: 2, 3: 2, 4: 4, 5: 8, 6: 2, 7: 4, 8: 8, 9: 1}


def dtype_size(dtype):
    return _SIZES[int(dtype)]


class HvdHipError(RuntimeError):
    """A non-zero return code of the C ABI; mirrors the reference's
    std::logic_error("<op> failed: <text>") (ops/cuda_operations.cc:82-86)."""

    def __init__(self, code, what, detail):
        self.code = code
        super().__init__("%s failed: %s%s" % (what, detail[0], (" (" + detail[1] + ")") if detail[1] else ""))


def lib_path():
    """The in-tree library, or the file named by HVDHIP_LIBRARY."""
    return os.environ.get("HVDHIP_LIBRARY") or os.path.join(_HERE, "lib", "libhvdhip.so")


_PV = POINTER(c_void_p)
_PROTOTYPES = {
    "hvdhip_error_string": (c_char_p, [c_int]),
    "hvdhip_last_error": (c_char_p, []),
    "hvdhip_set_fp16_scale_mode": (c_int, [c_int]),
    "hvdhip_get_fp16_scale_mode": (c_int, []),
    "hvdhip_dtype_size": (c_int64, [c_int]),
    "hvdhip_get_device": (c_int, [POINTER(c_int)]),
    "hvdhip_set_device": (c_int, [c_int]),
    "hvdhip_stream_create": (c_int, [_PV]),
    "hvdhip_stream_destroy": (c_int, [c_void_p]),
    "hvdhip_stream_forget": (c_int, [c_void_p]),
    "hvdhip_stream_synchronize": (c_int, [c_void_p]),
    "hvdhip_stream_wait_event": (c_int, [c_void_p, c_void_p]),
    "hvdhip_event_acquire": (c_int, [c_void_p, _PV]),
    "hvdhip_event_record": (c_int, [c_void_p, c_void_p]),
    "hvdhip_event_query": (c_int, [c_void_p, POINTER(c_int)]),
    "hvdhip_event_synchronize": (c_int, [c_void_p]),
    "hvdhip_event_release": (c_int, [c_void_p, c_void_p]),
    "hvdhip_event_pool_size": (c_int, [c_void_p, POINTER(c_int)]),
    "hvdhip_memcpy_async": (c_int, [c_void_p, c_void_p, c_size_t, c_int, c_void_p]),
    "hvdhip_timer_create": (c_int, [_PV]),
    "hvdhip_timer_start": (c_int, [c_void_p, c_void_p]),
    "hvdhip_timer_stop": (c_int, [c_void_p, c_void_p]),
    "hvdhip_timer_elapsed_ms": (c_int, [c_void_p, POINTER(c_float)]),
    "hvdhip_timer_destroy": (c_int, [c_void_p]),
    "hvdhip_batched_d2d_memcpy": (c_int, [_PV, _PV, POINTER(c_size_t), c_int, c_void_p]),
    "hvdhip_batched_scaled_d2d_memcpy": (c_int, [_PV, _PV, POINTER(c_size_t), c_int, c_double, c_int, c_void_p]),
    "hvdhip_copy_cache_stats": (c_int, [POINTER(c_uint64)] * 4),
    "hvdhip_copy_cache_set_limits": (c_int, [c_uint64, c_uint64]),
    "hvdhip_scale_buffer": (c_int, [c_void_p, c_void_p, c_int64, c_double, c_int, c_void_p]),
    "hvdhip_fusion_plan_create": (c_int, [_PV, _PV, POINTER(c_int64), c_int, c_int, c_int, _PV]),
    "hvdhip_fusion_plan_destroy": (c_int, [c_void_p]),
    "hvdhip_fusion_plan_buffer_len": (c_int64, [c_void_p]),
    "hvdhip_fusion_plan_offsets": (c_int, [c_void_p, POINTER(c_int64)]),
    "hvdhip_fusion_plan_num_chunks": (c_int64, [c_void_p]),
    "hvdhip_fusion_pack": (c_int, [c_void_p, c_void_p, c_double, c_uint, c_void_p]),
    "hvdhip_fusion_unpack": (c_int, [c_void_p, c_void_p, c_double, c_void_p]),
    "hvdhip_fusion_unpack_record": (c_int, [c_void_p, c_void_p, c_double, c_void_p, c_void_p]),
    "hvdhip_reduce_sum": (c_int, [c_void_p, c_void_p, c_int64, c_int, c_void_p]),
    "hvdhip_reduce_sum_k": (c_int, [c_void_p, _PV, c_int, c_int64, c_int, c_void_p]),
    "hvdhip_adasum_plan_create": (c_int, [POINTER(c_int), c_int, c_int, _PV]),
    "hvdhip_adasum_plan_destroy": (c_int, [c_void_p]),
    "hvdhip_adasum_dot_norms": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p]),
    "hvdhip_adasum_scaled_add": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p]),
    "hvdhip_adasum_combine": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p]),
    "hvdhip_adasum_read": (c_int, [c_void_p, POINTER(c_double), POINTER(c_double), c_void_p]),
    "hvdhip_adasum_set_coeffs": (c_int, [c_void_p, POINTER(c_double), c_void_p]),
    "hvdhip_adasum_dot_and_norm_sqrds": (c_int, [c_void_p, c_void_p, c_int, c_int, POINTER(c_double),
                                                 POINTER(c_double), POINTER(c_double), c_void_p]),
    "hvdhip_adasum_dispatch_scaled_add": (c_int, [c_int, c_int, c_double, c_void_p, c_double, c_void_p, c_void_p]),
    "hvdhip_adasum_combine_static": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p]),
}

_lib = None


def lib():
    """Loads libhvdhip.so (once).  Raises if it has not been built: there is
    no fallback implementation."""
    global _lib
    if _lib is not None:
        return _lib
    path = lib_path()
    if not os.path.exists(path):
        raise RuntimeError(
            "%s is missing: build it with `make -C horovod_amd/csrc` "
            "(or __graft_entry__.build()); there is no fallback path" % path)
    # torch ships its own HIP runtime under the same soname; import it first so
    # that one runtime serves both torch's allocations and this library.
    try:
        import torch  # noqa: F401
    except Exception:  # pragma: no cover - torch is only needed for device memory
        pass
    cdll = ctypes.CDLL(path)
    for name, (res, args) in _PROTOTYPES.items():
        fn = getattr(cdll, name)
        fn.restype = res
        fn.argtypes = args
    _lib = cdll
    return _lib


_adapter = None


def adapter_lib():
    """libhvdhip_adapter.so: the C++ mirror of the reference's op-layer classes, with the
    plain-C surface the Python callers use (keyed response fusion among others)."""
    global _adapter
    if _adapter is not None:
        return _adapter
    lib()  # the adapter links libhvdhip.so; load that one (and torch's HIP runtime) first
    path = os.path.join(_HERE, "lib", "libhvdhip_adapter.so")
    if not os.path.exists(path):
        raise RuntimeError("%s is missing: build it with `make -C horovod_amd/csrc`; "
                           "there is no fallback path" % path)
    cdll = ctypes.CDLL(path)
    cdll.hvd_adapter_fuse_keyed.restype = c_int
    cdll.hvd_adapter_fuse_keyed.argtypes = [POINTER(c_int64), POINTER(c_int), c_int, c_int64, c_int, POINTER(c_int)]
    _adapter = cdll
    return _adapter


def check(code, what):
    if code != 0:
        L = lib()
        raise HvdHipError(code, what, (L.hvdhip_error_string(code).decode(), L.hvdhip_last_error().decode()))
