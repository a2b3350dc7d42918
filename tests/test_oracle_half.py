"""Pins the oracle's fp16 routines: against the committed golden vectors taken
from the reference's own common/half.h and half.cc, against oracle/_ref where it
is built, against F16C hardware conversion and against numpy float16."""
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "half_golden.npz")


@pytest.fixture(scope="module")
def golden():
    return np.load(GOLDEN)


def test_half2float_all_values_match_golden(orc, golden):
    h = np.arange(65536, dtype=np.uint16)
    got = orc.half2float(h).view(np.uint32)
    assert np.array_equal(got, golden["h2f_out"])


def test_half2float_nan_is_canonical(orc):
    # common/half.h:69-70: every NaN becomes 0x7fffffff, sign dropped
    h = np.array([0x7c01, 0x7e00, 0xfe00, 0xffff], np.uint16)
    assert list(orc.half2float(h).view(np.uint32)) == [0x7fffffff] * 4


def test_half2float_matches_numpy_and_f16c(orc):
    h = np.arange(65536, dtype=np.uint16)
    want = h.view(np.float16).astype(np.float32)
    ok = ~np.isnan(want)
    assert np.array_equal(orc.half2float(h).view(np.uint32)[ok], want.view(np.uint32)[ok])
    assert np.array_equal(orc.half2float(h, f16c=True).view(np.uint32)[ok], want.view(np.uint32)[ok])


def test_float2half_matches_golden(orc, golden):
    got = orc.float2half(golden["f2h_in"].view(np.float32))
    assert np.array_equal(got, golden["f2h_out"])


def test_float2half_special_values(orc):
    f = np.array([0x00000000, 0x80000000, 0x7f800000, 0xff800000, 0x7fc00000, 0xffc00000, 0x477ff000,
                  0x477fefff, 0x33800000, 0x33000000, 0x33000001], np.uint32).view(np.float32)
    # +-0, +-inf, NaN -> 0x7fff (sign dropped, common/half.h:94-96), 65520 -> inf (tie to even),
    # just below -> 65504, 2^-24 -> smallest subnormal, 2^-25 tie -> 0, just above -> 1
    want = [0x0000, 0x8000, 0x7c00, 0xfc00, 0x7fff, 0x7fff, 0x7c00, 0x7bff, 0x0001, 0x0000, 0x0001]
    assert list(orc.float2half(f)) == want


def test_float2half_flushes_fp32_subnormals_to_signed_zero(orc):
    f = np.array([0x00000001, 0x007fffff, 0x80000001], np.uint32).view(np.float32)
    assert list(orc.float2half(f)) == [0x0000, 0x0000, 0x8000]


def test_float2half_strided_sweep_matches_numpy_and_f16c(orc):
    # every 4099th fp32 pattern (about 1M cases), NaNs excluded
    u = np.arange(0, 1 << 32, 4099, dtype=np.uint64).astype(np.uint32)
    f = u.view(np.float32)
    ok = ~np.isnan(f)
    sw = orc.float2half(f)
    with np.errstate(over="ignore"):
        want = f.astype(np.float16).view(np.uint16)
    assert np.array_equal(sw[ok], want[ok])
    assert np.array_equal(sw[ok], orc.float2half(f, f16c=True)[ok])


def test_float2half_matches_reference_build(orc, ref):
    rng = np.random.default_rng(5)
    u = rng.integers(0, 1 << 32, 1 << 20, dtype=np.uint64).astype(np.uint32)
    assert np.array_equal(orc.float2half(u.view(np.float32)), ref.float2half(u.view(np.float32)))
    h = np.arange(65536, dtype=np.uint16)
    assert np.array_equal(orc.half2float(h).view(np.uint32), ref.half2float(h).view(np.uint32))


def test_float16_sum_matches_golden(orc, golden):
    got = orc.float16_sum(golden["sum_a"], golden["sum_b"])
    assert np.array_equal(got, golden["sum_out"])
    got = orc.float16_sum(golden["sum_a"], golden["sum_b"], scalar=True)
    assert np.array_equal(got, golden["sum_out"])


def test_float16_sum_is_fp32_add_rounded_to_half(orc):
    rng = np.random.default_rng(9)
    a = (rng.standard_normal(100003) * 1e-4).astype(np.float16)
    b = (rng.standard_normal(100003) * 1e-4).astype(np.float16)
    want = (a.astype(np.float32) + b.astype(np.float32)).astype(np.float16)
    got = orc.float16_sum(a.view(np.uint16), b.view(np.uint16))
    assert np.array_equal(got, want.view(np.uint16))
    # 24 >= 2*11+2: the fp32 detour is a correctly rounded fp16 add
    assert np.array_equal(got, (a + b).view(np.uint16))


def test_float16_sum_matches_reference_build(orc, ref):
    rng = np.random.default_rng(10)
    a = rng.integers(0, 1 << 16, 200001, dtype=np.uint32).astype(np.uint16)
    b = rng.integers(0, 1 << 16, 200001, dtype=np.uint32).astype(np.uint16)
    keep = ~(np.isnan(a.view(np.float16)) | np.isnan(b.view(np.float16)))
    a, b = a[keep], b[keep]
    want = ref.float16_sum(a, b)
    got = orc.float16_sum(a, b)
    nan = np.isnan(want.view(np.float16))  # inf + -inf
    assert np.array_equal(got[~nan], want[~nan])
    assert np.array_equal(np.isnan(got.view(np.float16)), nan)
