"""Pins the oracle's ScaleBuffer (ops/collective_operations.h:91-127,
collective_operations.cc:114-146) and element-wise sum by IEEE closed forms."""
import numpy as np
import pytest

from oracle_util import F16, F32, F64, I8, I32, I64, U8, U16, I16, BOOL

FACTORS = [0.125, 1.0 / 3.0, 2.5, -0.7, 1e-3, 1.0]


@pytest.mark.parametrize("factor", FACTORS)
def test_scale_f32_is_one_single_precision_multiply(orc, factor):
    rng = np.random.default_rng(1)
    x = np.concatenate([rng.standard_normal(10007).astype(np.float32) * 1e-3,
                        np.array([0.0, -0.0, 1e-40, -1e-40, 3e38, np.inf], np.float32)])
    want = np.float32(factor) * x
    assert np.array_equal(orc.scale_buffer(x, factor, F32).view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("factor", FACTORS)
def test_scale_f64(orc, factor):
    rng = np.random.default_rng(2)
    x = rng.standard_normal(5003)
    assert np.array_equal(orc.scale_buffer(x, factor, F64), factor * x)


@pytest.mark.parametrize("dtype,np_t,lo,hi", [(U8, np.uint8, 0, 256), (I8, np.int8, -128, 128),
                                              (I32, np.int32, -2**31, 2**31), (I64, np.int64, -2**53, 2**53)])
@pytest.mark.parametrize("factor", [0.3, 0.125, 0.999, 1.0 / 3.0])
def test_scale_int_is_double_product_truncated_toward_zero(orc, dtype, np_t, lo, hi, factor):
    rng = np.random.default_rng(3)
    x = rng.integers(lo, hi, 4099, dtype=np.int64).astype(np_t)
    want = np.trunc(np.float64(factor) * x.astype(np.float64)).astype(np_t)
    assert np.array_equal(orc.scale_buffer(x, factor, dtype), want)


def test_scale_int_examples(orc):
    # 7*0.3 = 2.1 -> 2 ; -7*0.3 = -2.1 -> -2 (toward zero, not floor)
    assert list(orc.scale_buffer(np.array([7, -7], np.int32), 0.3, I32)) == [2, -2]


@pytest.mark.parametrize("factor", FACTORS)
def test_scale_f16_goes_through_fp32_with_fp32_factor(orc, factor):
    h = np.arange(65536, dtype=np.uint16)
    h = h[~np.isnan(h.view(np.float16))]
    with np.errstate(over="ignore"):
        want = (np.float32(factor) * h.view(np.float16).astype(np.float32)).astype(np.float16).view(np.uint16)
    got = orc.scale_buffer(h, factor, F16)
    assert np.array_equal(got, want)
    # the 8-wide F16C path and the software tail of the reference agree everywhere
    assert np.array_equal(got, orc.scale_half_scalar(h, factor))
    for n in (1, 7, 8, 9, 15, 17):
        assert np.array_equal(orc.scale_buffer(h[:n], factor, F16), want[:n])


@pytest.mark.parametrize("factor", FACTORS + [0.1915194503788923])
def test_scale_f16_cuda_arithmetic_rounds_the_factor_to_half_first(orc, factor):
    """ops/cuda/cuda_kernels.cu:96-136,167: half(factor) * x in half arithmetic.  numpy's
    float16 product is the exact product rounded once, like __hmul."""
    h = np.arange(65536, dtype=np.uint16)
    h = h[~np.isnan(h.view(np.float16))]
    with np.errstate(over="ignore"):
        want = (np.float16(np.float32(factor)) * h.view(np.float16)).view(np.uint16)
    got = orc.scale_half_cuda(h, factor)
    assert np.array_equal(got, want)
    if float(np.float16(np.float32(factor))) == factor:
        # a factor that a half holds exactly: both arithmetics of the reference agree
        assert np.array_equal(got, orc.scale_buffer(h, factor, F16))
    else:
        assert not np.array_equal(got, orc.scale_buffer(h, factor, F16))


def test_scale_f16_cuda_arithmetic_on_the_reference_test_vector(orc):
    """test/parallel/test_torch.py:339-388 for device half tensors: integers in [-100, 100)
    times np.random.seed(1234); np.random.uniform(), expected as
    (factor.type(half) * tensor.type(half)); for host half tensors the expectation is the
    fp32 product rounded to half."""
    np.random.seed(1234)
    factor = np.random.uniform()
    assert factor == 0.1915194503788923
    x = np.arange(-100, 100).astype(np.float16)
    want_device = np.float16(factor) * x
    want_host = (np.float32(factor) * x.astype(np.float32)).astype(np.float16)
    assert np.array_equal(orc.scale_half_cuda(x.view(np.uint16), factor), want_device.view(np.uint16))
    assert np.array_equal(orc.scale_buffer(x.view(np.uint16), factor, F16), want_host.view(np.uint16))
    assert not np.array_equal(want_device, want_host)  # the two expectations really differ on this vector


@pytest.mark.parametrize("dtype", [U16, I16, BOOL])
def test_scale_rejects_types_the_reference_rejects(orc, dtype):
    with pytest.raises(ValueError):
        orc.scale_buffer(np.zeros(4, np.uint16), 0.5, dtype)


def test_prescale_then_cast_is_a_single_rounding(orc):
    rng = np.random.default_rng(4)
    x = (rng.standard_normal(200003) * 1e-4).astype(np.float32)  # results are mostly subnormal halves
    want = (np.float32(0.125) * x).astype(np.float16).view(np.uint16)
    assert np.array_equal(orc.scale_cast_f32_to_f16(x, 0.125), want)
    f = 1.0 / 3.0
    want = (np.float32(f) * x).astype(np.float16).view(np.uint16)
    assert np.array_equal(orc.scale_cast_f32_to_f16(x, f), want)
    # scale 1.0 skips the multiply
    assert np.array_equal(orc.scale_cast_f32_to_f16(x, 1.0), x.astype(np.float16).view(np.uint16))


def test_cast_then_scale_is_two_roundings_and_differs(orc):
    rng = np.random.default_rng(4)
    x = (rng.standard_normal(200003) * 1e-4).astype(np.float32)
    h = x.astype(np.float16)
    want = (np.float32(0.125) * h.astype(np.float32)).astype(np.float16).view(np.uint16)
    got = orc.scale_cast_f32_to_f16(x, 0.125, cast_first=True)
    assert np.array_equal(got, want)
    assert not np.array_equal(got, orc.scale_cast_f32_to_f16(x, 0.125))


def test_postscale_and_widen(orc):
    h = np.arange(65536, dtype=np.uint16)
    h = h[~np.isnan(h.view(np.float16))]
    for f in (1.0, 0.5, 4.0, 1.0 / 3.0):
        with np.errstate(over="ignore"):
            want = (np.float32(f) * h.view(np.float16).astype(np.float32)).astype(np.float16).astype(np.float32)
        assert np.array_equal(orc.scale_cast_f16_to_f32(h, f).view(np.uint32), want.view(np.uint32))


def test_f16c_casts_for_the_cpu_timing_equal_the_software_casts(orc):
    """The 8-wide variants that the benchmark times on the CPU give the values of the software
    versions: random magnitudes from subnormal halves to overflow, every non-NaN half, odd lengths."""
    rng = np.random.default_rng(9)
    x = (rng.standard_normal(100003) * np.exp(rng.uniform(-20, 12, 100003))).astype(np.float32)
    x[:6] = [0.0, -0.0, np.inf, -np.inf, 65504.0, 65520.0]
    for f in (0.125, 1.0, 1.0 / 3.0, -7.5):
        for n in (0, 1, 7, 8, 9, x.size):
            assert np.array_equal(orc.scale_cast_f32_to_f16(x[:n], f, f16c=True), orc.scale_cast_f32_to_f16(x[:n], f))
    h = np.arange(65536, dtype=np.uint16)
    h = h[~np.isnan(h.view(np.float16))]
    for f in (1.0, 0.5, 1.0 / 3.0, 1e4):
        for n in (5, h.size):
            assert np.array_equal(orc.scale_cast_f16_to_f32(h[:n], f, f16c=True).view(np.uint32),
                                  orc.scale_cast_f16_to_f32(h[:n], f).view(np.uint32))


@pytest.mark.parametrize("dtype,np_t", [(U8, np.uint8), (I8, np.int8), (U16, np.uint16), (I16, np.int16),
                                        (I32, np.int32), (I64, np.int64)])
def test_sum_integers_wrap(orc, dtype, np_t):
    rng = np.random.default_rng(6)
    info = np.iinfo(np_t)
    a = rng.integers(info.min, int(info.max) + 1, 5001, dtype=np.int64 if np_t != np.int64 else np.int64).astype(np_t)
    b = rng.integers(info.min, int(info.max) + 1, 5001, dtype=np.int64).astype(np_t)
    with np.errstate(over="ignore"):
        want = (a + b).astype(np_t)
    assert np.array_equal(orc.sum(a, b, dtype), want)


@pytest.mark.parametrize("dtype,np_t", [(F32, np.float32), (F64, np.float64)])
def test_sum_float_is_one_ieee_add(orc, dtype, np_t):
    rng = np.random.default_rng(7)
    a = (rng.standard_normal(10001) * 1e-3).astype(np_t)
    b = (rng.standard_normal(10001) * 1e-3).astype(np_t)
    assert np.array_equal(orc.sum(a, b, dtype), a + b)


def test_sum_f16_dispatches_to_float16_sum(orc):
    rng = np.random.default_rng(8)
    a = (rng.standard_normal(10001) * 1e-4).astype(np.float16)
    b = (rng.standard_normal(10001) * 1e-4).astype(np.float16)
    got = orc.sum(a.view(np.uint16), b.view(np.uint16), F16)
    assert np.array_equal(got, (a + b).view(np.uint16))
