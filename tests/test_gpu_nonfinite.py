"""Infinities, NaNs and overflow through every kernel family, against the oracle.

Copies move bytes, so NaN payloads survive them bit for bit.  Arithmetic kernels must produce a NaN
exactly where the reference's CPU path does and the oracle's bits everywhere else (infinities from
overflow included); which NaN it is stays open, because the reference's software half converters
canonicalise NaNs (common/half.h:69-70,94-96) where hardware keeps payloads.
"""
import numpy as np
import pytest

from oracle_util import F16, F32, F64, NP_OF, SIZE_OF

pytestmark = pytest.mark.gpu

RAW_OF = {F16: np.uint16, F32: np.uint32, F64: np.uint64}


def _raw(v):
    return v.view(np.uint16) if v.dtype == np.float16 else v


def _specials(dtype, n, seed):
    """n values: ordinary ones with infinities, NaNs (quiet, with payload), zeros of both signs,
    the largest finite value and subnormals sprinkled in."""
    np_t = NP_OF[dtype]
    rng = np.random.default_rng(seed)
    v = rng.standard_normal(n).astype(np_t)
    info = np.finfo(np_t)
    bits = v.view(RAW_OF[dtype]).copy()
    nan_payload = {F16: 0x7e55, F32: 0x7fc12345, F64: 0x7ff8000012345678}[dtype]
    neg_nan = {F16: 0xfe01, F32: 0xffc00001, F64: 0xfff8000000000001}[dtype]
    special = [np.array(x, np_t).view(RAW_OF[dtype]) for x in
               (np.inf, -np.inf, 0.0, -0.0, info.max, -info.max, info.tiny, info.smallest_subnormal)]
    special += [np.array(nan_payload, RAW_OF[dtype]), np.array(neg_nan, RAW_OF[dtype])]
    where = rng.choice(n, size=min(n, 10 * len(special)), replace=False)
    for j, w in enumerate(where):
        bits[w] = special[j % len(special)]
    return bits.view(np_t)


def _same_but_for_nan_bits(got, want, np_t, what):
    """got and want are raw bit arrays of np_t values."""
    g, w = got.view(np_t), want.view(np_t)
    nan = np.isnan(w)
    assert np.array_equal(np.isnan(g), nan), "%s: NaNs in other places than the reference's" % what
    assert np.array_equal(got[~nan], want[~nan]), "%s: finite or infinite results differ" % what


@pytest.mark.parametrize("dtype", [F16, F32, F64])
def test_copies_keep_nan_payloads(gpu, dtype):
    v = _specials(dtype, 50001, 1)
    es = SIZE_OF[dtype]
    d_in = gpu.upload(v)
    plan = gpu.H.FusionPlan([d_in.data_ptr()], [d_in.data_ptr()], [v.size], dtype)
    try:
        buf = gpu.empty(plan.buffer_len, fill=0x11)
        plan.pack(buf.data_ptr(), 1.0, gpu.stream)
        got = gpu.download(buf)
        assert np.array_equal(got[:v.size * es], v.view(np.uint8))
    finally:
        plan.destroy()
    out = gpu.empty(v.size * es, fill=0x22)
    gpu.H.batched_d2d_memcpy([out.data_ptr()], [d_in.data_ptr()], [v.size * es], gpu.stream)
    assert np.array_equal(gpu.download(out), v.view(np.uint8))


@pytest.mark.parametrize("dtype", [F16, F32, F64])
@pytest.mark.parametrize("factor", [0.125, 2.5, 1e6, 0.0, -3.0])
def test_scale_with_nonfinite_values(gpu, orc, dtype, factor):
    # 2.5 and 1e6 overflow the largest values to infinity; 0 turns infinities into NaNs
    v = _specials(dtype, 20003, 2)
    d = gpu.upload(v)
    out = gpu.empty(v.nbytes)
    gpu.H.scale_buffer(d.data_ptr(), out.data_ptr(), v.size, factor, dtype, gpu.stream)
    got = gpu.download(out, RAW_OF[dtype])
    want = orc.scale_buffer(_raw(v), factor, dtype).view(RAW_OF[dtype])
    _same_but_for_nan_bits(got, want, NP_OF[dtype], "scale by %r" % factor)


@pytest.mark.parametrize("dtype", [F16, F32, F64])
@pytest.mark.parametrize("k", [1, 3, 7])
def test_reduce_sum_with_nonfinite_values(gpu, orc, dtype, k):
    # inf + -inf gives NaN; max + max overflows to inf; a NaN stays one through every later peer
    n = 30011
    res = _specials(dtype, n, 3)
    peers = [_specials(dtype, n, 10 + i) for i in range(k)]
    # line the specials of some peers up with those of the resident chunk
    peers[0][:200] = -res[:200]
    want = _raw(res).copy()
    for p in peers:
        want = orc.sum(_raw(p), want, dtype)
    d_res = gpu.upload(res)
    d_peers = [gpu.upload(p) for p in peers]
    gpu.H.reduce_sum_k(d_res.data_ptr(), [p.data_ptr() for p in d_peers], n, dtype, gpu.stream)
    got = gpu.download(d_res, RAW_OF[dtype])
    _same_but_for_nan_bits(got, want.view(RAW_OF[dtype]), NP_OF[dtype], "sum of %d peers" % k)


@pytest.mark.parametrize("cast_first", [False, True])
@pytest.mark.parametrize("factor", [0.125, 1.0, 4.0])
def test_narrowing_pack_overflows_to_infinity_like_the_reference(gpu, orc, cast_first, factor):
    # Float2HalfBits (common/half.h:79-139): beyond 65504 + half an ulp a value becomes infinity,
    # 65520 exactly ties to infinity, NaN stays NaN
    v = _specials(F32, 40009, 4)
    edge = np.array([65504.0, 65519.99, 65520.0, 65536.0, 1e5, -65520.0, -1e38, 5.9e-8, 2.98e-8, 2.9802322e-8,
                     524160.0, 524159.0, 8 * 65520.0, 16380.0, 16379.9], np.float32)
    v[:edge.size] = edge
    d = gpu.upload(v)
    plan = gpu.H.FusionPlan([d.data_ptr()], [d.data_ptr()], [v.size], F32, F16)
    try:
        buf = gpu.empty(plan.buffer_len, fill=0x33)
        plan.pack(buf.data_ptr(), factor, gpu.stream, flags=1 if cast_first else 0)
        got = gpu.download(buf, np.uint16)[:v.size]
    finally:
        plan.destroy()
    want = orc.scale_cast_f32_to_f16(v, factor, cast_first=cast_first)
    _same_but_for_nan_bits(got, want, np.float16, "narrowing pack, factor %r" % factor)


@pytest.mark.parametrize("factor", [1.0, 0.5, 3.0, 1e4])
def test_widening_unpack_with_nonfinite_values(gpu, orc, factor):
    h = np.arange(65536, dtype=np.uint16)  # every half, NaNs included
    d_buf = gpu.upload(h)
    out = gpu.empty(h.size * 4, fill=0x44)
    plan = gpu.H.FusionPlan([out.data_ptr()], [out.data_ptr()], [h.size], F32, F16)
    try:
        plan.unpack(d_buf.data_ptr(), factor, gpu.stream)
        got = gpu.download(out, np.uint32)
    finally:
        plan.destroy()
    want = orc.scale_cast_f16_to_f32(h, factor).view(np.uint32)
    _same_but_for_nan_bits(got, want, np.float32, "widening unpack, factor %r" % factor)


@pytest.mark.parametrize("dtype", [F32, F64, F16])
def test_adasum_layers_with_nonfinite_values(gpu, orc, dtype):
    """The coefficient guard of adasum.h:397-404 is written as `norm >= sqrt(DBL_MIN)`, which a NaN
    norm fails: that side's coefficient stays 1 while the other one becomes NaN.  A layer with a NaN
    or an infinity must come out as it does on the CPU, and must not leak into its neighbours."""
    np_t = NP_OF[dtype]
    counts = [1000, 20000, 17, 9000, 40000, 300, 5000]
    rng = np.random.default_rng(5)
    n = sum(counts)
    a = rng.standard_normal(n).astype(np_t)
    b = (0.3 * a.astype(np.float64) + rng.standard_normal(n)).astype(np_t)
    starts = np.concatenate([[0], np.cumsum(counts)])
    a[starts[1] + 7] = np.nan                      # layer 1: NaN in a only
    b[starts[2] + 3] = np.nan                      # layer 2: NaN in b only
    a[starts[3] + 5] = np.nan                      # layer 3: NaN in both
    b[starts[3] + 6] = np.nan
    a[starts[4] + 11] = np.inf                     # layer 4: infinity in a
    b[starts[5] + 1] = -np.inf                     # layer 5: infinity in b
    want, nd_w, co_w = orc.adasum_pairwise(_raw(a), _raw(b), counts, dtype)
    d_a, d_b = gpu.upload(a), gpu.upload(b)
    plan = gpu.H.AdasumPlan(counts, dtype)
    try:
        plan.combine(d_a.data_ptr(), d_b.data_ptr(), gpu.stream)
        nd, co = plan.read(gpu.stream)
    finally:
        plan.destroy()
    nd, co = np.array(nd), np.array(co)
    assert np.array_equal(np.isnan(nd), np.isnan(nd_w)), "sums: NaN in other places"
    assert np.array_equal(np.isinf(nd), np.isinf(nd_w)), "sums: infinity in other places"
    assert np.array_equal(np.isnan(co), np.isnan(co_w)), "coefficients: NaN in other places"
    fin = np.isfinite(co_w)
    assert np.all(np.abs(co[fin] - co_w[fin]) <= 1e-6 * np.abs(co_w[fin]))
    assert np.array_equal(co[~fin & ~np.isnan(co_w)], co_w[~fin & ~np.isnan(co_w)])
    got = gpu.download(d_a, RAW_OF[dtype]).view(np_t)
    w = want.view(np_t)
    assert np.array_equal(np.isnan(got), np.isnan(w)), "results: NaN in other places"
    ok = ~np.isnan(w)
    if dtype == F16:
        assert np.array_equal(got.view(np.uint16)[ok], w.view(np.uint16)[ok])
    else:
        inf = np.isinf(w)
        assert np.array_equal(got[inf], w[inf])
        ok &= ~inf
        tol = (1e-6 if dtype == F32 else 1e-11) * (np.abs(a[ok].astype(np.float64)) + np.abs(b[ok].astype(np.float64)))
        assert np.all(np.abs(got[ok].astype(np.float64) - w[ok].astype(np.float64)) <= tol)
    # the untouched layers are what they are without any special value around them
    for layer in (0, 6):
        s, e = starts[layer], starts[layer + 1]
        alone, _, _ = orc.adasum_pairwise(_raw(a[s:e]), _raw(b[s:e]), [e - s], dtype)
        assert np.array_equal(want[s:e], alone)
