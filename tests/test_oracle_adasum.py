"""Pins the oracle's Adasum (ops/adasum/adasum.h:344-435,439-500): exact sums,
the closed-form pairwise operation that the reference's own test restates
(test/parallel/test_adasum_tensorflow.py:29-44), and the algebraic invariants of
test/parallel/test_adasum_pytorch.py:46-211."""
import math

import numpy as np
import pytest

from oracle_util import F16, F32, F64


def _pairwise_closed_form(a, b):
    """a, b float64.  The operation of test_adasum_tensorflow.py:29-44."""
    an, bn, dot = float(np.inner(a, a)), float(np.inner(b, b)), float(np.dot(a, b))
    ca = 1.0 - dot / an * 0.5 if an != 0 else 1.0
    cb = 1.0 - dot / bn * 0.5 if bn != 0 else 1.0
    return ca * a + cb * b


def _diff_ratio(true_vec, comp_vec):
    # test_adasum_pytorch.py:38-44
    return np.linalg.norm(true_vec - comp_vec) / np.linalg.norm(true_vec) / 100.0


@pytest.mark.parametrize("dtype,np_t", [(F32, np.float32), (F64, np.float64), (F16, np.float16)])
def test_dot_norms_match_exact_sums(orc, dtype, np_t):
    rng = np.random.default_rng(11)
    for n in (1, 2, 7, 8, 9, 1000, 65537):
        a = rng.standard_normal(n).astype(np_t)
        b = rng.standard_normal(n).astype(np_t)
        got = orc.adasum_dot_norms(a.view(np.uint16) if np_t == np.float16 else a,
                                   b.view(np.uint16) if np_t == np.float16 else b, dtype)
        a64, b64 = a.astype(np.float64), b.astype(np.float64)
        want = [math.fsum(a64 * b64), math.fsum(a64 * a64), math.fsum(b64 * b64)]
        # products of narrower floats are exact in double; only the order of additions differs
        for g, w, scale in zip(got, want, [math.fsum(np.abs(a64 * b64)), want[1], want[2]]):
            assert abs(g - w) <= 1e-13 * scale + 1e-300


def test_dot_norms_catch_swapped_or_dropped_terms(orc):
    a = np.array([1.0, 2.0, 3.0], np.float32)
    b = np.array([-4.0, 5.0, 0.5], np.float32)
    assert list(orc.adasum_dot_norms(a, b, F32)) == [-4.0 + 10.0 + 1.5, 14.0, 16.0 + 25.0 + 0.25]


def test_coeffs_closed_form_and_guard(orc):
    assert orc.adasum_coeffs(3.0, 4.0, 8.0) == (1.0 - 3.0 / 4.0 * 0.5, 1.0 - 3.0 / 8.0 * 0.5)
    guard = math.sqrt(2.2250738585072014e-308)
    # below sqrt(DBL_MIN) the coefficient stays 1 (adasum.h:399-404)
    ca, cb = orc.adasum_coeffs(1e-200, guard * 0.999, 4.0)
    assert ca == 1.0 and cb == 1.0 - 1e-200 / 4.0 * 0.5
    ca, cb = orc.adasum_coeffs(0.0, guard, guard)
    assert (ca, cb) == (1.0, 1.0)
    assert orc.adasum_coeffs(0.0, 0.0, 0.0) == (1.0, 1.0)


@pytest.mark.parametrize("dtype,np_t,tol", [(F32, np.float32, 1), (F64, np.float64, 2)])
def test_pairwise_matches_closed_form(orc, dtype, np_t, tol):
    rng = np.random.default_rng(12)
    counts = [5, 0, 1, 1000, 17, 4096]
    n = sum(counts)
    a = rng.standard_normal(n).astype(np_t)
    b = (0.3 * a + rng.standard_normal(n)).astype(np_t)
    got, nd, co = orc.adasum_pairwise(a, b, counts, dtype)
    off = 0
    for i, c in enumerate(counts):
        sa, sb = a[off:off + c].astype(np.float64), b[off:off + c].astype(np.float64)
        if c:
            want = _pairwise_closed_form(sa, sb).astype(np_t)
            if np_t == np.float64:
                # the closed form's own coefficients carry a few ulps from numpy's summation order
                bound = 8 * np.finfo(np.float64).eps * (np.abs(sa) + np.abs(sb))
            else:
                bound = tol * np.spacing(np.abs(want).astype(np_t))
            assert np.all(np.abs(got[off:off + c].astype(np.float64) - want) <= bound)
            assert abs(co[2 * i] - (1.0 - np.dot(sa, sb) / np.dot(sa, sa) * 0.5)) < 1e-12
        else:
            assert (co[2 * i], co[2 * i + 1]) == (1.0, 1.0) and list(nd[3 * i:3 * i + 3]) == [0, 0, 0]
        off += c


@pytest.mark.parametrize("dtype,np_t", [(F32, np.float32), (F64, np.float64)])
def test_scaled_add_is_two_products_and_a_sum(orc, dtype, np_t):
    # adasum.h:429-435 as written: acoeff * a[i] + bcoeff * b[i] in double, three roundings, then the
    # conversion to T.  numpy evaluates each operation on its own (no contraction), so a fused
    # multiply-add in the oracle would show here as last-bit differences.
    rng = np.random.default_rng(17)
    for n in (1, 7, 100003):
        a = rng.standard_normal(n).astype(np_t)
        b = rng.standard_normal(n).astype(np_t)
        ca, cb = 0.8312345678901234, 0.9123456789012345
        want = (np.float64(ca) * a.astype(np.float64) + np.float64(cb) * b.astype(np.float64)).astype(np_t)
        got = orc.adasum_scaled_add(a, b, ca, cb, dtype)
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8))
    # a contracted evaluation, fma(ca, a, cb*b), computed exactly with rationals, differs from the
    # above on some of these inputs: the check can tell the two apart
    from fractions import Fraction
    a = rng.standard_normal(3000)
    b = rng.standard_normal(3000)
    plain = np.float64(ca) * a + np.float64(cb) * b
    fused = np.array([float(Fraction(ca) * Fraction(float(x)) + Fraction(float(np.float64(cb) * y)))
                      for x, y in zip(a, b)])
    assert 0 < np.count_nonzero(plain != fused) < 1500
    assert np.array_equal(orc.adasum_scaled_add(a, b, ca, cb, F64), plain)


def test_fp16_scaled_add_formula(orc):
    # adasum.h:482-500: float coefficients, t = ca*a rounded to fp32, fma(cb, b, t), RNE to half
    rng = np.random.default_rng(13)
    for n in (3, 8, 13, 1001):
        a = rng.standard_normal(n).astype(np.float16)
        b = rng.standard_normal(n).astype(np.float16)
        ca, cb = 0.8312345678, 0.9123456789
        t = np.float32(ca) * a.astype(np.float32)
        # fma in fp32 == the double expression rounded once (the product of two fp32 is exact in double,
        # and the sum of that with an fp32 is exact enough that one rounding decides)
        r = (np.float32(cb).astype(np.float64) * b.astype(np.float64) + t.astype(np.float64)).astype(np.float32)
        want = r.astype(np.float16)
        got = orc.adasum_scaled_add(a.view(np.uint16), b.view(np.uint16), ca, cb, F16)
        assert np.array_equal(got, want.view(np.uint16))


@pytest.mark.parametrize("dtype,np_t", [(F32, np.float32), (F16, np.float16)])
def test_orthogonal_vectors_add(orc, dtype, np_t):
    # test_adasum_pytorch.py:46-91: orthogonal gradients -> plain sum
    rng = np.random.default_rng(2)
    for n in (23, 5, 4, 2 ** 12):
        q, _ = np.linalg.qr(rng.standard_normal((n, 2)))
        q = q.astype(np_t)
        a, b = np.ascontiguousarray(q[:, 0]), np.ascontiguousarray(q[:, 1])
        raw = (lambda v: v.view(np.uint16)) if np_t == np.float16 else (lambda v: v)
        got, _, _ = orc.adasum_pairwise(raw(a), raw(b), [n], dtype)
        got = got.view(np_t).astype(np.float64)
        want = q.astype(np.float64).sum(axis=1)
        assert _diff_ratio(want, got) < np.finfo(np_t).eps


@pytest.mark.parametrize("dtype,np_t", [(F32, np.float32), (F16, np.float16)])
def test_parallel_vectors_average(orc, dtype, np_t):
    # test_adasum_pytorch.py:93-138: identical gradients -> the gradient itself
    rng = np.random.default_rng(3)
    a = rng.standard_normal(1000).astype(np_t)
    raw = (lambda v: v.view(np.uint16)) if np_t == np.float16 else (lambda v: v)
    got, _, co = orc.adasum_pairwise(raw(a), raw(a.copy()), [1000], dtype)
    assert abs(co[0] - 0.5) < 1e-12 and abs(co[1] - 0.5) < 1e-12
    assert _diff_ratio(a.astype(np.float64), got.view(np_t).astype(np.float64)) < np.finfo(np_t).eps


def test_scale_stability(orc):
    # test_adasum_pytorch.py:140-211: tiny magnitudes do not lose the direction
    rng = np.random.default_rng(4)
    a = rng.standard_normal(1000)
    b = 0.3 * a + rng.standard_normal(1000)
    base, _, _ = orc.adasum_pairwise(a.astype(np.float32), b.astype(np.float32), [1000], F32)
    for s in (1e-15, 1e-8, 1e6):
        got, _, _ = orc.adasum_pairwise((a * s).astype(np.float32), (b * s).astype(np.float32), [1000], F32)
        assert _diff_ratio(base.astype(np.float64) * s, got.astype(np.float64)) < np.finfo(np.float32).eps
