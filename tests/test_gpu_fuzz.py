"""Seeded random fused responses (dtype, tensor sizes, source/output misalignment, scale
factors, peers) through pack -> k-way reduce -> unpack, against the oracle.  Deterministic."""
import numpy as np
import pytest

from oracle_util import F16, F32, F64, I8, I32, I64, U8, NP_OF, SIZE_OF

pytestmark = pytest.mark.gpu

from gpu_util import Arena  # noqa: E402


def _vals(rng, n, dtype):
    np_t = NP_OF[dtype]
    if dtype in (F32, F64):
        return (rng.standard_normal(n) * 10.0 ** rng.integers(-6, 2)).astype(np_t)
    if dtype == F16:
        return (rng.standard_normal(n) * 10.0 ** rng.integers(-6, 0)).astype(np.float16)
    if dtype == I64:
        return rng.integers(-2 ** 40, 2 ** 40, n, dtype=np.int64)
    if dtype == I32:
        return rng.integers(-2 ** 27, 2 ** 27, n, dtype=np.int64).astype(np.int32)
    info = np.iinfo(np_t)
    return (rng.integers(info.min, int(info.max) + 1, n, dtype=np.int64) // 8).astype(np_t)


def _raw(v):
    return v.view(np.uint16) if v.dtype == np.float16 else v


@pytest.mark.parametrize("seed", range(40))
def test_random_fused_response(gpu, orc, seed):
    rng = np.random.default_rng(1000 + seed)
    dtype = [F32, F16, F64, I32, I64, U8, I8][seed % 7]
    es = SIZE_OF[dtype]
    n = int(rng.integers(1, 40))
    # a mix of tiny, chunk-boundary and large tensors
    counts = []
    for _ in range(n):
        kind = rng.integers(0, 4)
        if kind == 0:
            counts.append(int(rng.integers(0, 64)))
        elif kind == 1:
            counts.append(int(4096 // es * rng.integers(1, 5) + rng.integers(-3, 4)))
        elif kind == 2:
            counts.append(int(rng.integers(100, 50000)))
        else:
            counts.append(int(rng.integers(50000, 400000)))
    counts = [max(c, 0) for c in counts]
    prescale = float(rng.choice([1.0, 0.125, 1.0 / 3.0, 0.3, 0.75]))
    postscale = float(rng.choice([1.0, 0.5, 1.0 / 7.0]))
    if dtype in (U8, I8, I32, I64):
        prescale, postscale = min(prescale, 1.0), min(postscale, 1.0)  # keep products inside the type
    k = int(rng.integers(0, 4))
    total = sum(c * es for c in counts) + 512 * (n + 2)
    src, dst = Arena(total), Arena(total, fill=0x5A)
    so, do, vals = [], [], []
    for c in counts:
        so.append(src.alloc(c * es, misalign=int(rng.integers(0, 16 // es)) * es))
        do.append(dst.alloc(c * es, misalign=int(rng.integers(0, 16 // es)) * es))
        v = _vals(rng, c, dtype)
        src.host[so[-1]:so[-1] + c * es] = v.view(np.uint8)
        vals.append(v)
    src.upload(), dst.upload()
    plan = gpu.H.FusionPlan([src.ptr(o) for o in so], [dst.ptr(o) for o in do], counts, dtype)
    try:
        offs = plan.offsets()
        fb = gpu.empty(plan.buffer_len + 64, fill=0xCD)
        nbuf = plan.buffer_len // es
        peer_host = [np.zeros(nbuf, NP_OF[dtype]) for _ in range(k)]
        for ph in peer_host:
            for o, c in zip(offs, counts):
                ph[o // es:o // es + c] = _vals(rng, c, dtype) if dtype not in (U8, I8, I32, I64) else _vals(rng, c, dtype) // 4
        peers = [gpu.upload(ph) for ph in peer_host]
        plan.pack(fb.data_ptr(), prescale, gpu.stream)
        if k:
            gpu.H.reduce_sum_k(fb.data_ptr(), [p.data_ptr() for p in peers], nbuf, dtype, gpu.stream)
        plan.unpack(fb.data_ptr(), postscale, gpu.stream)
        gpu.sync()
        out = dst.download()
        assert np.all(gpu.download(fb)[plan.buffer_len:] == 0xCD)
        touched = np.zeros(out.size, bool)
        for i, (c, v) in enumerate(zip(counts, vals)):
            w = _raw(v) if prescale == 1.0 else orc.scale_buffer(_raw(v), prescale, dtype)
            for ph in peer_host:
                w = orc.sum(_raw(ph[offs[i] // es:offs[i] // es + c]), w, dtype)
            w = w if postscale == 1.0 else orc.scale_buffer(w, postscale, dtype)
            got = out[do[i]:do[i] + c * es]
            assert np.array_equal(got, w.view(np.uint8)), "seed %d tensor %d (%d elements)" % (seed, i, c)
            touched[do[i]:do[i] + c * es] = True
        assert np.all(out[~touched] == 0x5A)
    finally:
        plan.destroy()
