"""Parity of hvdhip_scale_buffer and hvdhip_reduce_sum{,_k} with the oracle."""
import numpy as np
import pytest

from oracle_util import F16, F32, F64, I8, I16, I32, I64, U8, U16, NP_OF, SIZE_OF

pytestmark = pytest.mark.gpu

SIZES = [1, 2, 3, 4, 5, 7, 8, 9, 63, 64, 65, 2047, 2048, 2049, 8191, 8192, 8193, 65537, 300001]


def _vals(rng, n, dtype, scale=1.0):
    np_t = NP_OF[dtype]
    if dtype in (F32, F64, F16):
        return (rng.standard_normal(n) * scale).astype(np_t)
    if dtype == I64:
        return rng.integers(-2 ** 40, 2 ** 40, n, dtype=np.int64)
    info = np.iinfo(np_t)
    return rng.integers(info.min, int(info.max) + 1, n, dtype=np.int64).astype(np_t)


def _raw(v):
    return v.view(np.uint16) if v.dtype == np.float16 else v


@pytest.mark.parametrize("dtype", [U8, I8, I32, I64, F16, F32, F64])
@pytest.mark.parametrize("factor", [0.125, 1.0 / 3.0, 2.5, 1.0])
def test_scale_buffer(gpu, orc, dtype, factor):
    rng = np.random.default_rng(1)
    es = SIZE_OF[dtype]
    for n in SIZES:
        v = _vals(rng, n, dtype, 1e-3 if dtype == F16 else 1.0)
        if dtype in (I32,):
            v = (v // 4).astype(np.int32)  # keep factor*x inside the type
        if dtype in (U8, I8) and factor > 1:
            v = (v // 4).astype(v.dtype)
        # out of place, input offset by one element to break 16-byte alignment
        pad = np.zeros(1, v.dtype)
        d_in = gpu.upload(np.concatenate([pad, v]))
        d_out = gpu.empty((n + 2) * es, fill=0x5A)
        gpu.H.scale_buffer(d_in.data_ptr() + es, d_out.data_ptr(), n, factor, dtype, gpu.stream)
        out = gpu.download(d_out)
        want = orc.scale_buffer(_raw(v), factor, dtype)
        assert np.array_equal(out[:n * es], want.view(np.uint8)), "n=%d" % n
        assert np.all(out[n * es:] == 0x5A)
        # in place
        gpu.H.scale_buffer(d_in.data_ptr() + es, d_in.data_ptr() + es, n, factor, dtype, gpu.stream)
        got = gpu.download(d_in)[es:]
        assert np.array_equal(got, want.view(np.uint8)), "in place n=%d" % n


def test_scale_buffer_fp16_subnormal_results_and_odd_factor(gpu, orc):
    # every finite half times a non-representable factor: results cover the subnormal range
    h = np.arange(65536, dtype=np.uint16)
    h = h[~np.isnan(h.view(np.float16))]
    d = gpu.upload(h)
    for factor in (1.0 / 3.0, 1e-3, 0.1, 7.7):
        out = gpu.empty(h.nbytes)
        gpu.H.scale_buffer(d.data_ptr(), out.data_ptr(), h.size, factor, F16, gpu.stream)
        got = gpu.download(out, np.uint16)
        want = orc.scale_buffer(h, factor, F16)
        assert np.array_equal(got, want), "factor %r: %d differ" % (factor, int((got != want).sum()))


def test_scale_buffer_fp32_denormals_are_kept(gpu, orc):
    v = np.array([1e-38, -1e-38, 1.5e-45, 3e-39, 1.17549435e-38], np.float32)
    d = gpu.upload(v)
    gpu.H.scale_buffer(d.data_ptr(), d.data_ptr(), v.size, 0.125, F32, gpu.stream)
    got = gpu.download(d, np.uint32)
    assert np.array_equal(got, orc.scale_buffer(v, 0.125, F32).view(np.uint32))


@pytest.mark.parametrize("dtype", [U8, I8, U16, I16, I32, I64, F16, F32, F64])
def test_reduce_sum(gpu, orc, dtype):
    rng = np.random.default_rng(2)
    es = SIZE_OF[dtype]
    for n in SIZES:
        a = _vals(rng, n, dtype, 1e-4 if dtype == F16 else 1e-3)
        b = _vals(rng, n, dtype, 1e-4 if dtype == F16 else 1e-3)
        pad = np.zeros(1, a.dtype)
        d_res = gpu.upload(np.concatenate([pad, a, pad]))
        d_in = gpu.upload(np.concatenate([pad, pad, b]))
        gpu.H.reduce_sum(d_res.data_ptr() + es, d_in.data_ptr() + 2 * es, n, dtype, gpu.stream)
        got = gpu.download(d_res)
        want = orc.sum(_raw(b), _raw(a), dtype)
        assert np.array_equal(got[es:es + n * es], want.view(np.uint8)), "n=%d" % n
        assert np.all(got[:es] == 0) and np.all(got[es + n * es:] == 0), "wrote outside the chunk"


def test_reduce_sum_fp16_all_pairs_sample(gpu, orc):
    # a dense sample of half x half, including subnormals, max, infinities
    rng = np.random.default_rng(3)
    a = rng.integers(0, 1 << 16, 1 << 20, dtype=np.uint32).astype(np.uint16)
    b = rng.integers(0, 1 << 16, 1 << 20, dtype=np.uint32).astype(np.uint16)
    keep = ~(np.isnan(a.view(np.float16)) | np.isnan(b.view(np.float16)))
    a, b = a[keep], b[keep]
    want = orc.float16_sum(b, a)
    nan = np.isnan(want.view(np.float16))
    d_res, d_in = gpu.upload(a), gpu.upload(b)
    gpu.H.reduce_sum(d_res.data_ptr(), d_in.data_ptr(), a.size, F16, gpu.stream)
    got = gpu.download(d_res, np.uint16)
    assert np.array_equal(got[~nan], want[~nan])
    assert np.all(np.isnan(got.view(np.float16)[nan]))


@pytest.mark.parametrize("dtype", [F16, F32, F64, I32])
@pytest.mark.parametrize("k", [1, 2, 3, 7, 8, 9, 16])
def test_reduce_sum_k_equals_k_successive_sums(gpu, orc, dtype, k):
    rng = np.random.default_rng(4 + k)
    es = SIZE_OF[dtype]
    for n in (5, 8193, 100003):
        res = _vals(rng, n, dtype, 1e-4 if dtype == F16 else 1e-3)
        peers = [_vals(rng, n, dtype, 1e-4 if dtype == F16 else 1e-3) for _ in range(k)]
        want = _raw(res).copy()
        for p in peers:
            want = orc.sum(_raw(p), want, dtype)  # rounded to the element type after every peer
        d_res = gpu.upload(res)
        d_peers = [gpu.upload(p) for p in peers]
        gpu.H.reduce_sum_k(d_res.data_ptr(), [d.data_ptr() for d in d_peers], n, dtype, gpu.stream)
        got = gpu.download(d_res)
        assert np.array_equal(got, want.view(np.uint8)), "n=%d k=%d" % (n, k)


def test_reduce_rejects_bool_and_bad_k(gpu):
    import horovod_amd
    t = gpu.empty(64)
    with pytest.raises(horovod_amd.HvdHipError) as e:
        gpu.H.reduce_sum(t.data_ptr(), t.data_ptr(), 4, 9, gpu.stream)
    assert e.value.code == -2
    with pytest.raises(horovod_amd.HvdHipError):
        gpu.H.reduce_sum_k(t.data_ptr(), [t.data_ptr()] * 17, 4, F32, gpu.stream)


@pytest.mark.parametrize("dtype", [F32, F16])
@pytest.mark.parametrize("n_tiles", [512, 513, 1024 + 300, 5 * 512 + 1])
def test_tile_order_across_xcd_groups(gpu, orc, dtype, n_tiles):
    """Contiguous kernels hand tiles to workgroups in groups of 512 so that each XCD walks runs of 64
    consecutive tiles, and leave a ragged last group in natural order: whole groups, a group plus
    one tile, and sizes that end inside a tile must all give the oracle's values."""
    rng = np.random.default_rng(n_tiles)
    es = SIZE_OF[dtype]
    n = n_tiles * (4096 // es) - 37
    v = _vals(rng, n, dtype, 1e-2 if dtype == F16 else 1.0)
    p = _vals(rng, n, dtype, 1e-2 if dtype == F16 else 1.0)
    d_v, d_p, d_o = gpu.upload(_raw(v)), gpu.upload(_raw(p)), gpu.empty(n * es + 64, fill=0x5A)
    gpu.H.scale_buffer(d_v.data_ptr(), d_o.data_ptr(), n, 0.125, dtype, gpu.stream)
    out = gpu.download(d_o)
    assert np.array_equal(out[:n * es], orc.scale_buffer(_raw(v), 0.125, dtype).view(np.uint8))
    assert np.all(out[n * es:] == 0x5A)
    gpu.H.reduce_sum(d_v.data_ptr(), d_p.data_ptr(), n, dtype, gpu.stream)
    assert np.array_equal(gpu.download(d_v)[:n * es], orc.sum(_raw(p), _raw(v), dtype).view(np.uint8))
