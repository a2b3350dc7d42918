"""Parity of the HIP Adasum path with the oracle: coefficients to 1e-6 relative
(observed ~1e-13), results within 1 ulp for fp32/fp64 and bit-exact for fp16."""
import math

import numpy as np
import pytest

from oracle_util import F16, F32, F64, NP_OF, SIZE_OF

pytestmark = pytest.mark.gpu


def _raw(v):
    return v.view(np.uint16) if v.dtype == np.float16 else v


def _ulp_diff(got, want):
    """Distance in units in the last place between two float arrays of the same dtype."""
    it = {2: np.int16, 4: np.int32, 8: np.int64}[got.dtype.itemsize]
    g, w = got.view(it).astype(np.int64), want.view(it).astype(np.int64)
    top = np.int64(1) << (8 * got.dtype.itemsize - 1)
    g = np.where(g < 0, -(g + top), g)  # sign-magnitude -> monotone integers
    w = np.where(w < 0, -(w + top), w)
    return np.abs(g - w)


def _pair(rng, n, np_t, corr=0.3):
    a = rng.standard_normal(n)
    b = corr * a + math.sqrt(1 - corr * corr) * rng.standard_normal(n)
    return a.astype(np_t), b.astype(np_t)


COUNTS = [5, 0, 1, 1000, 17, 8192, 8193, 3, 100003, 0, 2 * 8192, 65537]


@pytest.mark.parametrize("dtype", [F32, F64, F16])
def test_combine_matches_oracle(gpu, orc, dtype):
    rng = np.random.default_rng(1)
    np_t = NP_OF[dtype]
    n = sum(COUNTS)
    a, b = _pair(rng, n, np_t)
    want, nd_w, co_w = orc.adasum_pairwise(_raw(a), _raw(b), COUNTS, dtype)
    es = SIZE_OF[dtype]
    # vectors start one element past a 16-byte boundary: layer starts are only element-aligned anyway
    pad = np.zeros(1, np_t)
    d_a, d_b = gpu.upload(np.concatenate([pad, a, pad])), gpu.upload(np.concatenate([pad, b]))
    plan = gpu.H.AdasumPlan(COUNTS, dtype)
    try:
        plan.combine(d_a.data_ptr() + es, d_b.data_ptr() + es, gpu.stream)
        nd, co = plan.read(gpu.stream)
        nd, co = np.array(nd), np.array(co)
        for i, c in enumerate(COUNTS):
            a64 = a[sum(COUNTS[:i]):sum(COUNTS[:i + 1])].astype(np.float64)
            b64 = b[sum(COUNTS[:i]):sum(COUNTS[:i + 1])].astype(np.float64)
            mag = [math.fsum(np.abs(a64 * b64)), nd_w[3 * i + 1], nd_w[3 * i + 2]]
            for j in range(3):
                assert abs(nd[3 * i + j] - nd_w[3 * i + j]) <= 1e-12 * mag[j] + 1e-300, (i, j)
        assert np.all(np.abs(co - co_w) <= 1e-6 * np.abs(co_w)), "coefficients beyond 1e-6 relative"
        assert np.all(np.abs(co - co_w) <= 1e-11 * np.abs(co_w))
        got = gpu.download(d_a, np_t if np_t != np.float16 else np.uint16)
        assert got[0] == 0 and got[-1] == 0, "wrote outside the vector"
        got = got[1:-1]
        if dtype == F16:
            # fp16: float coefficients (identical after rounding 1e-13-close doubles, barring a tie) and
            # exact fp32 mul + fma: bit-exact
            assert np.array_equal(got, want)
        else:
            # The scaled add itself is pinned to the bit: with the coefficients the device computed,
            # the result is acoeff * a + bcoeff * b as adasum.h:429-435 states it (two rounded double
            # products, their rounded sum, one conversion), which numpy evaluates without contraction.
            off = 0
            for i, c in enumerate(COUNTS):
                x, y = a[off:off + c].astype(np.float64), b[off:off + c].astype(np.float64)
                exact = (np.float64(co[2 * i]) * x + np.float64(co[2 * i + 1]) * y).astype(np_t)
                assert np.array_equal(got[off:off + c].view(np.uint8), exact.view(np.uint8)), i
                off += c
            # Against the oracle's own coefficients (sequential sums; 1e-13 apart from the tree sums):
            if dtype == F32:
                assert _ulp_diff(got, want).max() <= 1
            else:
                bound = 1e-11 * (np.abs(a.astype(np.float64)) + np.abs(b.astype(np.float64)))
                assert np.all(np.abs(got - want) <= bound)
    finally:
        plan.destroy()


@pytest.mark.parametrize("dtype", [F32, F16])
def test_dot_norms_then_host_coeffs_then_scaled_add(gpu, orc, dtype):
    # the split form: a caller sums the triples across ranks, then sets coefficients
    rng = np.random.default_rng(2)
    np_t = NP_OF[dtype]
    counts = [4097, 33, 70000]
    a, b = _pair(rng, sum(counts), np_t, corr=-0.5)
    d_a, d_b = gpu.upload(a), gpu.upload(b)
    plan = gpu.H.AdasumPlan(counts, dtype)
    try:
        plan.dot_norms(d_a.data_ptr(), d_b.data_ptr(), gpu.stream)
        nd, _ = plan.read(gpu.stream)
        coeffs = []
        for i in range(len(counts)):
            coeffs += list(orc.adasum_coeffs(2 * nd[3 * i], 2 * nd[3 * i + 1], 2 * nd[3 * i + 2]))  # "two ranks"
        plan.set_coeffs(coeffs, gpu.stream)
        plan.scaled_add(d_a.data_ptr(), d_b.data_ptr(), gpu.stream)
        got = gpu.download(d_a, np_t if np_t != np.float16 else np.uint16)
        off = 0
        for i, c in enumerate(counts):
            want = orc.adasum_scaled_add(_raw(a[off:off + c]), _raw(b[off:off + c]), coeffs[2 * i],
                                         coeffs[2 * i + 1], dtype)
            if dtype == F16:
                assert np.array_equal(got[off:off + c], want)
            else:
                assert _ulp_diff(got[off:off + c], want).max() <= 1
            off += c
    finally:
        plan.destroy()


def test_dispatch_hooks_single_layer(gpu, orc):
    # the shapes of Adasum::DispatchComputeDotAndNormSqrds / DispatchScaledAdd (adasum.h:101-140)
    import ctypes
    import horovod_amd
    L = horovod_amd.lib()
    rng = np.random.default_rng(3)
    for n in (0, 1, 1000, 50001):
        a, b = _pair(rng, max(n, 1), np.float32)
        a, b = a[:n], b[:n]
        d_a, d_b = gpu.upload(np.concatenate([a, [0]]).astype(np.float32)), gpu.upload(np.concatenate([b, [0]]).astype(np.float32))
        dot, an, bn = ctypes.c_double(-1), ctypes.c_double(-1), ctypes.c_double(-1)
        horovod_amd.check(L.hvdhip_adasum_dot_and_norm_sqrds(d_a.data_ptr(), d_b.data_ptr(), F32, n,
                                                             ctypes.byref(dot), ctypes.byref(an), ctypes.byref(bn),
                                                             gpu.stream.handle), "dot")
        w = orc.adasum_dot_norms(a, b, F32) if n else np.zeros(3)
        assert np.allclose([dot.value, an.value, bn.value], w, rtol=1e-12, atol=0)
        horovod_amd.check(L.hvdhip_adasum_dispatch_scaled_add(F32, n, 0.75, d_a.data_ptr(), 1.25, d_b.data_ptr(),
                                                              gpu.stream.handle), "scaled_add")
        got = gpu.download(d_a, np.float32)
        want = orc.adasum_scaled_add(a, b, 0.75, 1.25, F32)
        assert got[n] == 0
        if n:
            assert _ulp_diff(got[:n], want).max() <= 1


def test_dispatch_hooks_from_two_threads_on_two_streams(gpu, orc):
    # The per-layer hooks keep their single-layer plans in a shared cache.  Two threads, each with
    # a stream of its own and the same layer sizes, must neither wait for each other's blocking
    # read nor see each other's partial sums.
    import ctypes
    import threading
    import horovod_amd
    L = horovod_amd.lib()
    rng = np.random.default_rng(31)
    sizes = [70001, 1000, 70001, 333333, 1000]
    data = []
    for t in range(2):
        per = []
        for n in sizes:
            a, b = _pair(rng, n, np.float32, corr=0.2 + 0.5 * t)
            per.append((a, b, gpu.upload(a), gpu.upload(b)))
        data.append(per)
    errors, results = [], [[], []]

    def worker(t):
        try:
            L.hvdhip_set_device(0)
            st = horovod_amd.Stream()
            for rep in range(6):
                for a, b, d_a, d_b in data[t]:
                    dot, an, bn = ctypes.c_double(), ctypes.c_double(), ctypes.c_double()
                    horovod_amd.check(L.hvdhip_adasum_dot_and_norm_sqrds(
                        d_a.data_ptr(), d_b.data_ptr(), F32, a.size, ctypes.byref(dot), ctypes.byref(an),
                        ctypes.byref(bn), st.handle), "dot")
                    results[t].append((a.size, dot.value, an.value, bn.value))
            st.destroy()
        except Exception as e:  # pragma: no cover
            errors.append(e)

    ts = [threading.Thread(target=worker, args=(t,)) for t in range(2)]
    [t.start() for t in ts]
    [t.join() for t in ts]
    assert not errors, errors
    for t in range(2):
        assert len(results[t]) == 6 * len(sizes)
        for k, (n, dot, an, bn) in enumerate(results[t]):
            a, b, _, _ = data[t][k % len(sizes)]
            w = orc.adasum_dot_norms(a, b, F32)
            assert np.allclose([dot, an, bn], w, rtol=1e-12, atol=0), (t, k)
        # the same layer gives the same bits every time (fixed summation tree)
        firsts = {}
        for k, r in enumerate(results[t]):
            assert firsts.setdefault(k % len(sizes), r) == r


def test_tiny_norms_keep_coefficient_one(gpu, orc):
    # |a|^2 below sqrt(DBL_MIN): coefficient 1 (adasum.h:399-404)
    a = np.full(64, 1e-40, np.float32)  # fp32 subnormal; |a|^2 = 64e-80 >= 1.5e-154, so not guarded
    b = np.zeros(64, np.float32)
    z = np.zeros(64, np.float64)
    tiny = np.full(64, 1e-80, np.float64)  # |a|^2 = 6.4e-159 < sqrt(DBL_MIN): guarded
    for x, y, dtype in ((a, b, F32), (tiny, z + 1.0, F64), (z, z, F64)):
        d_a, d_b = gpu.upload(x), gpu.upload(y)
        plan = gpu.H.AdasumPlan([64], dtype)
        plan.combine(d_a.data_ptr(), d_b.data_ptr(), gpu.stream)
        _, co = plan.read(gpu.stream)
        want, _, co_w = orc.adasum_pairwise(x, y, [64], dtype)
        assert co == list(co_w)
        got = gpu.download(d_a, x.dtype)
        assert _ulp_diff(got, want).max() <= 1
        plan.destroy()


@pytest.mark.parametrize("dtype", [F32, F16])
def test_invariants_orthogonal_and_parallel(gpu, dtype):
    # test/parallel/test_adasum_pytorch.py:46-138 on the device
    np_t = NP_OF[dtype]
    rng = np.random.default_rng(4)
    n = 2 ** 19
    q, _ = np.linalg.qr(rng.standard_normal((n, 2)))
    q = q.astype(np_t)
    a, b = np.ascontiguousarray(q[:, 0]), np.ascontiguousarray(q[:, 1])
    d_a, d_b = gpu.upload(a), gpu.upload(b)
    plan = gpu.H.AdasumPlan([n], dtype)
    plan.combine(d_a.data_ptr(), d_b.data_ptr(), gpu.stream)
    got = gpu.download(d_a, np_t).astype(np.float64)
    want = q.astype(np.float64).sum(axis=1)
    assert np.linalg.norm(want - got) / np.linalg.norm(want) / 100.0 < np.finfo(np_t).eps
    d_a, d_b = gpu.upload(a), gpu.upload(a)
    plan.combine(d_a.data_ptr(), d_b.data_ptr(), gpu.stream)
    got = gpu.download(d_a, np_t).astype(np.float64)
    assert np.linalg.norm(a.astype(np.float64) - got) / np.linalg.norm(a.astype(np.float64)) / 100.0 < np.finfo(np_t).eps
    plan.destroy()


def test_results_are_reproducible_run_to_run(gpu):
    rng = np.random.default_rng(5)
    counts = [300001, 7, 123457]
    a, b = _pair(rng, sum(counts), np.float32)
    d_a, d_b = gpu.upload(a), gpu.upload(b)
    plan = gpu.H.AdasumPlan(counts, F32)
    seen = set()
    for _ in range(5):
        plan.dot_norms(d_a.data_ptr(), d_b.data_ptr(), gpu.stream)
        nd, co = plan.read(gpu.stream)
        seen.add((tuple(nd), tuple(co)))
    assert len(seen) == 1
    plan.destroy()


@pytest.mark.parametrize("dtype", [F32, F64, F16])
@pytest.mark.parametrize("big", [False, True])
def test_combine_equals_split_sequence_bit_for_bit(gpu, dtype, big):
    """combine() sums each layer's partial results inside the scaled add when every layer is
    small enough, and launches the separate summing kernel otherwise (big: one layer beyond
    that limit).  Both must give exactly what dot_norms() followed by scaled_add() gives:
    same sums, same coefficients, same vector, to the bit, with empty layers reported as
    sums 0 and coefficients 1."""
    rng = np.random.default_rng(11)
    np_t = NP_OF[dtype]
    counts = [0, 5, 0, 70001, 16384 // SIZE_OF[dtype] * 512, 1, 0]  # fifth layer: exactly 512 chunks
    if big:
        counts[3] = 16384 // SIZE_OF[dtype] * 512 + 1  # 513 chunks
    n = sum(counts)
    a, b = _pair(rng, n, np_t)
    d_a1, d_a2, d_b = gpu.upload(a), gpu.upload(a), gpu.upload(b)
    plan1, plan2 = gpu.H.AdasumPlan(counts, dtype), gpu.H.AdasumPlan(counts, dtype)
    try:
        plan1.dot_norms(d_a1.data_ptr(), d_b.data_ptr(), gpu.stream)
        plan1.scaled_add(d_a1.data_ptr(), d_b.data_ptr(), gpu.stream)
        nd1, co1 = plan1.read(gpu.stream)
        plan2.combine(d_a2.data_ptr(), d_b.data_ptr(), gpu.stream)
        nd2, co2 = plan2.read(gpu.stream)
        assert np.array_equal(np.array(nd1).view(np.uint64), np.array(nd2).view(np.uint64))
        assert np.array_equal(np.array(co1).view(np.uint64), np.array(co2).view(np.uint64))
        for i, c in enumerate(counts):
            if c == 0:
                assert list(nd2[3 * i:3 * i + 3]) == [0.0, 0.0, 0.0] and list(co2[2 * i:2 * i + 2]) == [1.0, 1.0]
        raw = np.uint16 if np_t == np.float16 else np_t
        g1, g2 = gpu.download(d_a1, raw), gpu.download(d_a2, raw)
        assert np.array_equal(g1.view(np.uint8), g2.view(np.uint8))
        assert not np.array_equal(g2.view(np.uint8), _raw(a).view(np.uint8)), "combine left the vector untouched"
    finally:
        plan1.destroy()
        plan2.destroy()


def test_rejects_integer_dtypes(gpu):
    import horovod_amd
    with pytest.raises(horovod_amd.HvdHipError) as e:
        gpu.H.AdasumPlan([4], 4)
    assert e.value.code == -2
