"""ctypes access to the CPU oracle (oracle/liborc.so) for the tests.

The oracle is the checker only: nothing here is used by the library under test.
"""
import ctypes
import os
import subprocess
from ctypes import c_double, c_float, c_int, c_int64, c_void_p

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")

U8, I8, U16, I16, I32, I64, F16, F32, F64, BOOL = range(10)
NP_OF = {U8: np.uint8, I8: np.int8, U16: np.uint16, I16: np.int16, I32: np.int32, I64: np.int64,
         F16: np.float16, F32: np.float32, F64: np.float64, BOOL: np.bool_}
SIZE_OF = {U8: 1, I8: 1, U16: 2, I16: 2, I32: 4, I64: 8, F16: 2, F32: 4, F64: 8, BOOL: 1}


def _p(a):
    return c_void_p(a.ctypes.data)


def _ensure_built():
    so = os.path.join(ORACLE_DIR, "liborc.so")
    src = os.path.join(ORACLE_DIR, "hvd_oracle.c")
    if not os.path.exists(so) or os.path.getmtime(so) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", ORACLE_DIR, "liborc.so"], stdout=subprocess.DEVNULL)
    return so


def load_ref():
    so = os.path.join(ORACLE_DIR, "_ref", "libhvdref.so")
    if not os.path.exists(so):
        return None
    lib = ctypes.CDLL(so)
    return Ref(lib)


class Ref:
    def __init__(self, lib):
        self.lib = lib

    def half2float(self, h):
        h = np.ascontiguousarray(h, np.uint16)
        out = np.empty(h.shape, np.float32)
        self.lib.ref_half2float(_p(h), _p(out), c_int64(h.size))
        return out

    def float2half(self, f):
        f = np.ascontiguousarray(f, np.float32)
        out = np.empty(f.shape, np.uint16)
        self.lib.ref_float2half(_p(f), _p(out), c_int64(f.size))
        return out

    def float16_sum(self, inp, inout):
        inp = np.ascontiguousarray(inp, np.uint16)
        out = np.array(inout, np.uint16, copy=True)
        self.lib.ref_float16_sum(_p(inp), _p(out), c_int64(out.size))
        return out


class Oracle:
    def __init__(self):
        self.lib = ctypes.CDLL(_ensure_built())
        L = self.lib
        L.orc_pack.restype = c_int64
        L.orc_pack_padded.restype = c_int64
        L.orc_padded_offsets.restype = c_int64
        L.orc_fusion_threshold.restype = c_int64
        L.orc_dtype_size.restype = c_int64

    # ---- fp16 ----
    def half2float(self, h, f16c=False):
        h = np.ascontiguousarray(h, np.uint16)
        out = np.empty(h.shape, np.float32)
        fn = self.lib.orc_half2float_f16c if f16c else self.lib.orc_half2float
        fn(_p(h), _p(out), c_int64(h.size))
        return out

    def float2half(self, f, f16c=False):
        f = np.ascontiguousarray(f, np.float32)
        out = np.empty(f.shape, np.uint16)
        fn = self.lib.orc_float2half_f16c if f16c else self.lib.orc_float2half
        fn(_p(f), _p(out), c_int64(f.size))
        return out

    # ---- pack / unpack ----
    @staticmethod
    def _ptrs(arrays):
        arr = (c_void_p * len(arrays))()
        for i, a in enumerate(arrays):
            arr[i] = a.ctypes.data
        return arr

    def pack(self, tensors, padded=False):
        """tensors: list of contiguous numpy arrays.  Returns (buffer bytes, buffer_len)."""
        nb = np.array([t.nbytes for t in tensors], np.int64)
        cap = int(sum(16 * ((int(x) + 15) // 16) for x in nb)) + 16
        buf = np.full(cap, 0xAB, np.uint8)
        fn = self.lib.orc_pack_padded if padded else self.lib.orc_pack
        n = fn(self._ptrs(tensors), _p(nb), c_int(len(tensors)), _p(buf))
        return buf, int(n)

    def unpack(self, buf, outputs, padded=False):
        nb = np.array([t.nbytes for t in outputs], np.int64)
        fn = self.lib.orc_unpack_padded if padded else self.lib.orc_unpack
        fn(_p(buf), self._ptrs(outputs), _p(nb), c_int(len(outputs)))

    def padded_offsets(self, nbytes):
        nb = np.array(nbytes, np.int64)
        offs = np.empty(len(nb) + 1, np.int64)
        self.lib.orc_padded_offsets(_p(nb), c_int(len(nb)), _p(offs))
        return offs

    # ---- scale ----
    def scale_buffer(self, x, scale, dtype):
        x = np.ascontiguousarray(x)
        out = np.empty_like(x)
        rc = self.lib.orc_scale_buffer(_p(x), _p(out), c_int64(x.size), c_double(scale), c_int(dtype))
        if rc != 0:
            raise ValueError("dtype %d not supported by ScaleBuffer" % dtype)
        return out

    def scale_half_scalar(self, h, factor):
        h = np.ascontiguousarray(h, np.uint16)
        out = np.empty_like(h)
        self.lib.orc_scale_half_scalar(_p(h), _p(out), c_int64(h.size), c_float(factor))
        return out

    def scale_half_cuda(self, h, scale):
        h = np.ascontiguousarray(h, np.uint16)
        out = np.empty_like(h)
        self.lib.orc_scale_half_cuda(_p(h), _p(out), c_int64(h.size), c_double(scale))
        return out

    def scale_cast_f32_to_f16(self, x, scale, cast_first=False, f16c=False):
        x = np.ascontiguousarray(x, np.float32)
        out = np.empty(x.shape, np.uint16)
        fn = self.lib.orc_cast_then_scale_f32_to_f16 if cast_first else self.lib.orc_scale_cast_f32_to_f16
        if f16c:
            fn = self.lib.orc_scale_cast_f32_to_f16_f16c
        fn(_p(x), _p(out), c_int64(x.size), c_double(scale))
        return out

    def scale_cast_f16_to_f32(self, h, scale, f16c=False):
        h = np.ascontiguousarray(h, np.uint16)
        out = np.empty(h.shape, np.float32)
        fn = self.lib.orc_scale_cast_f16_to_f32_f16c if f16c else self.lib.orc_scale_cast_f16_to_f32
        fn(_p(h), _p(out), c_int64(h.size), c_double(scale))
        return out

    # ---- sum ----
    def sum(self, inp, inout, dtype):
        """Returns inout + inp (a new array); inout is left untouched."""
        inp = np.ascontiguousarray(inp)
        out = np.array(inout, copy=True)
        rc = self.lib.orc_sum(_p(inp), _p(out), c_int64(out.size), c_int(dtype))
        if rc != 0:
            raise ValueError("dtype %d cannot be summed" % dtype)
        return out

    def float16_sum(self, inp, inout, scalar=False):
        inp = np.ascontiguousarray(inp, np.uint16)
        out = np.array(inout, np.uint16, copy=True)
        fn = self.lib.orc_float16_sum_scalar if scalar else self.lib.orc_float16_sum
        fn(_p(inp), _p(out), c_int64(out.size))
        return out

    # ---- adasum ----
    def adasum_dot_norms(self, a, b, dtype):
        a = np.ascontiguousarray(a)
        b = np.ascontiguousarray(b)
        out = np.zeros(3, np.float64)
        rc = self.lib.orc_adasum_dot_norms(_p(a), _p(b), c_int(a.size), c_int(dtype), _p(out))
        if rc != 0:
            raise ValueError("dtype")
        return out

    def adasum_coeffs(self, dot, an, bn):
        ca, cb = c_double(), c_double()
        self.lib.orc_adasum_coeffs(c_double(dot), c_double(an), c_double(bn), ctypes.byref(ca), ctypes.byref(cb))
        return ca.value, cb.value

    def adasum_scaled_add(self, a, b, ca, cb, dtype):
        out = np.array(a, copy=True)
        b = np.ascontiguousarray(b)
        self.lib.orc_adasum_scaled_add(c_int(dtype), c_int(out.size), c_double(ca), _p(out), c_double(cb), _p(b))
        return out

    def adasum_pairwise(self, a, b, counts, dtype):
        """Returns (new a, normdots[3L], coeffs[2L])."""
        out = np.array(a, copy=True)
        b = np.ascontiguousarray(b)
        counts = np.array(counts, np.int32)
        nd = np.zeros(3 * len(counts), np.float64)
        co = np.zeros(2 * len(counts), np.float64)
        rc = self.lib.orc_adasum_pairwise(_p(out), _p(b), c_int(dtype), _p(counts), c_int(len(counts)),
                                          _p(nd), _p(co))
        if rc != 0:
            raise ValueError("dtype")
        return out, nd, co

    # ---- allgather fusion ----
    def allgather(self, per_rank_tensors, dtype):
        """per_rank_tensors[rank][entry] -> list of outputs (one per entry), via the oracle's
        displacement / offset / pack / unpack restatement, every rank packing into one buffer."""
        size, n = len(per_rank_tensors), len(per_rank_tensors[0])
        es = SIZE_OF[dtype]
        sizes = np.array([[per_rank_tensors[rc][ec].size for rc in range(size)] for ec in range(n)], np.int64)
        recv = np.array([int(sizes[:, rc].sum()) for rc in range(size)], np.int32)
        displ = np.zeros(size, np.int32)
        self.lib.orc_allgather_displacements(_p(recv), _p(displ), c_int(size))
        offs = np.zeros((n, size), np.int64)
        self.lib.orc_allgather_component_offsets(_p(sizes), c_int(n), c_int(size), _p(recv), _p(offs))
        buf = np.full(int(recv.sum()) * es + 16, 0xEE, np.uint8)
        for rc in range(size):
            ts = [np.ascontiguousarray(t) for t in per_rank_tensors[rc]]
            nb = np.array([t.nbytes for t in ts], np.int64)
            self.lib.orc_allgather_pack(self._ptrs(ts), _p(nb), c_int(n), _p(displ), c_int(rc), c_int(es), _p(buf))
        outs = [np.zeros(int(sizes[ec].sum()), per_rank_tensors[0][ec].dtype) for ec in range(n)]
        self.lib.orc_allgather_unpack(_p(offs), _p(sizes), c_int(n), c_int(size), _p(buf), c_int(es),
                                      self._ptrs(outs))
        return outs, displ, offs

    # ---- planning ----
    def fusion_threshold(self, proposed, local_size, homogeneous=True):
        return int(self.lib.orc_fusion_threshold(c_int64(proposed), c_int(local_size), c_int(int(homogeneous))))

    def fuse_responses(self, tensor_bytes, threshold, pad16=True, keys=None):
        tb = np.array(tensor_bytes, np.int64)
        keys = np.zeros(len(tb), np.int32) if keys is None else np.array(keys, np.int32)
        groups = np.empty(len(tb), np.int32)
        n = self.lib.orc_fuse_responses(_p(tb), _p(keys), c_int(len(tb)), c_int64(threshold), c_int(int(pad16)),
                                        _p(groups))
        return int(n), groups
