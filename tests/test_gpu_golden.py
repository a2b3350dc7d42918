"""The HIP path against the committed golden vectors directly (tests/golden/half_golden.npz:
outputs of the reference's own common/half.h and common/half.cc, compiled in place), without
the oracle in between: the fp32 -> fp16 rounding of the converting pack, the fp16 -> fp32
widening of the converting unpack, and the fp16 sum of the reduce kernel."""
import os

import numpy as np
import pytest

from oracle_util import F16, F32

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "half_golden.npz")


@pytest.fixture(scope="module")
def golden():
    return np.load(GOLDEN)  # plain arrays, no pickled objects


def _not_nan16(h):
    return (h & 0x7fff) <= 0x7c00


def test_converting_pack_rounds_like_float2halfbits(gpu, golden):
    """Float2HalfBits (common/half.h:79-139) on the fixture's fp32 patterns: normals, subnormal
    results, ties, overflow to infinity.  NaNs are left out: the software converter canonicalises
    them, the hardware keeps the payload."""
    x = golden["f2h_in"].view(np.float32)
    want = golden["f2h_out"]
    keep = ~np.isnan(x)
    x, want = np.ascontiguousarray(x[keep]), want[keep]
    n = x.size
    src, out = gpu.upload(x), gpu.empty(4 * n)
    plan = gpu.H.FusionPlan([src.data_ptr()], [out.data_ptr()], [n], F32, F16)
    try:
        fb = gpu.empty(plan.buffer_len)
        plan.pack(fb.data_ptr(), 1.0, gpu.stream)
        got = gpu.download(fb)[:2 * n].view(np.uint16)
        assert np.array_equal(got, want), "%d of %d halves differ" % (int((got != want).sum()), n)
    finally:
        plan.destroy()


def test_converting_unpack_widens_like_halfbits2float(gpu, golden):
    """HalfBits2Float (common/half.h:43-77) on all 65,536 halves (NaNs aside)."""
    h = np.arange(65536, dtype=np.uint16)
    want = golden["h2f_out"]
    keep = _not_nan16(h)
    h, want = np.ascontiguousarray(h[keep]), want[keep]
    n = h.size
    tensors, out = gpu.empty(4 * n, fill=0), gpu.empty(4 * n, fill=0x5A)
    plan = gpu.H.FusionPlan([tensors.data_ptr()], [out.data_ptr()], [n], F32, F16)
    try:
        assert plan.buffer_len >= 2 * n
        fb = gpu.upload(np.concatenate([h, np.zeros((plan.buffer_len - 2 * n) // 2, np.uint16)]))
        plan.unpack(fb.data_ptr(), 1.0, gpu.stream)
        got = gpu.download(out)[:4 * n].view(np.uint32)
        assert np.array_equal(got, want), "%d of %d values differ" % (int((got != want).sum()), n)
    finally:
        plan.destroy()


def test_fp16_reduce_sums_like_float16_sum(gpu, golden):
    """float16_sum (common/half.cc:44-76): inout = RNE16(fp32(in) + fp32(inout))."""
    a, b, want = golden["sum_a"], golden["sum_b"], golden["sum_out"]
    keep = _not_nan16(a) & _not_nan16(b) & _not_nan16(want)  # inf - inf gives a NaN whose bits are unspecified
    a, b, want = np.ascontiguousarray(a[keep]), np.ascontiguousarray(b[keep]), want[keep]
    resident, incoming = gpu.upload(b), gpu.upload(a)
    gpu.H.reduce_sum(resident.data_ptr(), incoming.data_ptr(), a.size, F16, gpu.stream)
    got = gpu.download(resident)[:2 * a.size].view(np.uint16)
    assert np.array_equal(got, want), "%d of %d sums differ" % (int((got != want).sum()), a.size)
