"""hvdhip_adasum_combine_static, the Adasum combine that allocates nothing (its tables and
partial sums live in a fixed array inside the library's device code), against
hvdhip_adasum_combine with a one-layer plan: same kernels, same tables, so the vector, the sums
and the coefficients must agree to the bit.  Two calls in a row share the array; the second is
smaller, so it runs over what the first left behind."""
import ctypes

import numpy as np
import pytest
import torch

from oracle_util import F16, F32, F64, NP_OF

pytestmark = pytest.mark.gpu


def _pair(rng, n, np_t, corr=0.3):
    a = rng.standard_normal(n)
    b = corr * a + np.sqrt(1 - corr * corr) * rng.standard_normal(n)
    return a.astype(np_t), b.astype(np_t)


def _static(gpu, d_a, d_b, dtype, n, d_res):
    import horovod_amd
    horovod_amd.check(horovod_amd.lib().hvdhip_adasum_combine_static(
        d_a.data_ptr(), d_b.data_ptr(), dtype, n, d_res.data_ptr() if d_res is not None else None,
        gpu.stream.handle), "hvdhip_adasum_combine_static")


def _planned(gpu, d_a, d_b, dtype, n):
    plan = gpu.H.AdasumPlan([n], dtype)
    try:
        plan.combine(d_a.data_ptr(), d_b.data_ptr(), gpu.stream)
        nd, co = plan.read(gpu.stream)
    finally:
        plan.destroy()
    return np.array(nd + co)


@pytest.mark.parametrize("dtype", [F32, F16, F64])
def test_two_calls_in_a_row_match_the_planned_combine(gpu, orc, dtype):
    rng = np.random.default_rng(41)
    np_t = NP_OF[dtype]
    raw = np.uint16 if np_t == np.float16 else np_t
    per_chunk = 16384 // np.dtype(np_t).itemsize
    # first call: 700 chunks (the sums get a launch of their own) and a ragged tail;
    # second call: 37 chunks (summed inside the scaled add), over the first call's leftovers;
    # then the empty layer and a single element
    for n in (700 * per_chunk + 1234, 37 * per_chunk - 5, 0, 1):
        a, b = _pair(rng, max(n, 1), np_t)
        a, b = a[:n], b[:n]
        guard = np.full(8, 7, np_t)
        d_a1 = gpu.upload(np.concatenate([a, guard]))
        d_a2 = gpu.upload(np.concatenate([a, guard]))
        d_b = gpu.upload(np.concatenate([b, guard]))
        d_res = torch.full((5,), -1.0, dtype=torch.float64, device="cuda")
        torch.cuda.synchronize()
        want5 = _planned(gpu, d_a1, d_b, dtype, n)
        _static(gpu, d_a2, d_b, dtype, n, d_res)
        got = gpu.download(d_a2, raw)
        want = gpu.download(d_a1, raw)
        assert np.array_equal(got, want), "vector differs from the planned combine (n=%d)" % n
        assert np.array_equal(got[n:], guard.view(raw)), "wrote past the vector"
        got5 = d_res.cpu().numpy()
        assert np.array_equal(got5.view(np.uint64), want5.view(np.uint64)), (n, got5, want5)
        if n:
            # and the planned combine is what the oracle computes (coefficients to 1e-6)
            _, _, co_w = orc.adasum_pairwise(a.view(raw), b.view(raw), [n], dtype)
            assert np.all(np.abs(got5[3:] - co_w) <= 1e-6 * np.abs(co_w))
            assert not np.array_equal(got[:n], a.view(raw)), "the vector was left untouched"


def test_results_pointer_is_optional_and_limit_is_enforced(gpu):
    import horovod_amd
    rng = np.random.default_rng(42)
    n = 100000
    a, b = _pair(rng, n, np.float32)
    d_a1, d_a2, d_b = gpu.upload(a), gpu.upload(a), gpu.upload(b)
    _planned(gpu, d_a1, d_b, F32, n)
    _static(gpu, d_a2, d_b, F32, n, None)
    assert np.array_equal(gpu.download(d_a2, np.float32), gpu.download(d_a1, np.float32))
    # one element beyond 16,384 chunks of 4,096 floats: refused, nothing launched
    with pytest.raises(horovod_amd.HvdHipError) as e:
        _static(gpu, d_a2, d_b, F32, (1 << 26) + 1, None)
    assert e.value.code == -4
    with pytest.raises(horovod_amd.HvdHipError) as e:
        _static(gpu, d_a2, d_b, 4, 16, None)  # INT32
    assert e.value.code == -2


def test_largest_size_runs(gpu):
    # exactly the limit for fp32: 2^26 elements, 16,384 chunks; identical vectors give the vector back
    n = 1 << 26
    x = torch.ones(n, dtype=torch.float32, device="cuda")
    y = torch.ones(n, dtype=torch.float32, device="cuda")
    d_res = torch.zeros(5, dtype=torch.float64, device="cuda")
    torch.cuda.synchronize()
    _static(gpu, x, y, F32, n, d_res)
    gpu.sync()
    assert d_res.cpu().tolist() == [float(n)] * 3 + [0.5, 0.5]
    assert int((x != 1).sum()) == 0


@pytest.mark.parametrize("chunks", [37, 700])
def test_a_captured_call_replays_like_the_eager_one(gpu, chunks):
    """The property the entry point exists for.  Under stream capture (torch's default, global mode)
    an allocation, a free, a blocking copy or a synchronisation on any thread is refused, so a
    call that did any of those would fail the capture; the recorded graph holds kernels only.  It is
    replayed three times on fresh inputs, with eager work and synchronisations in between, and every
    replay must equal the planned combine of the same inputs to the bit (vector, sums, coefficients).
    37 chunks take the path that sums inside the scaled add, 700 the one with a sum launch of its own."""
    import horovod_amd
    n = chunks * 4096 - 5
    side = torch.cuda.Stream()
    s = horovod_amd.Stream(side.cuda_stream)
    a = torch.zeros(n, device="cuda")
    b = torch.zeros(n, device="cuda")
    a2 = torch.zeros(n, device="cuda")
    res = torch.zeros(5, dtype=torch.float64, device="cuda")
    static = horovod_amd.lib().hvdhip_adasum_combine_static

    def call():
        horovod_amd.check(static(a.data_ptr(), b.data_ptr(), F32, n, res.data_ptr(), s.handle),
                          "hvdhip_adasum_combine_static")

    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        call()  # warm-up outside the capture: the scratch array's address is looked up on the first call
        side.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            call()
        side.synchronize()
    gen = torch.Generator(device="cuda")
    for replay in range(3):
        gen.manual_seed(50 + replay)
        a.copy_(torch.randn(n, generator=gen, device="cuda"))
        b.copy_(0.3 * a + torch.randn(n, generator=gen, device="cuda"))
        a2.copy_(a)
        res.fill_(-1.0)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        want5 = _planned(gpu, a2, b, F32, n)  # eager, with its own plan and its own synchronisations
        torch.cuda.synchronize()
        assert torch.equal(a.view(torch.int32), a2.view(torch.int32)), "replay %d" % replay
        assert np.array_equal(res.cpu().numpy().view(np.uint64), want5.view(np.uint64)), "replay %d" % replay
        assert not torch.equal(a, b)


def test_eager_calls_leave_the_device_memory_as_it_was(gpu):
    """hipMemGetInfo's free bytes before and after 100 calls (after one warm-up call): the entry
    point takes nothing from the device allocator, whatever the sizes it is called with."""
    rng = np.random.default_rng(43)
    sizes = [1, 4096 * 37 - 5, 4096 * 700 + 1234, 1 << 22, 17]
    n_max = max(sizes)
    a, b = _pair(rng, n_max, np.float32)
    d_a, d_b = gpu.upload(a), gpu.upload(b)
    d_res = torch.zeros(5, dtype=torch.float64, device="cuda")
    _static(gpu, d_a, d_b, F32, sizes[1], d_res)
    gpu.sync()
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    for i in range(100):
        _static(gpu, d_a, d_b, F32, sizes[i % len(sizes)], d_res)
    gpu.sync()
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before


def test_calls_from_two_streams_are_ordered_by_the_library(gpu):
    """All calls on a device share one scratch array, so the library puts each behind the one
    before it (an event behind every call, a stream wait in the next call from another stream).
    Two streams call alternately, 40 times each, on vectors of their own and of different sizes
    (one with a sum launch of its own, one that sums inside the scaled add), nothing synchronised in
    between; each vector must come out exactly as 40 planned combines in a row leave it."""
    import horovod_amd
    rng = np.random.default_rng(44)
    s1, s2 = horovod_amd.Stream(), horovod_amd.Stream()
    sizes = (700 * 4096 + 99, 37 * 4096 - 5)
    data = []
    for n in sizes:
        a, b = _pair(rng, n, np.float32)
        data.append((gpu.upload(a), gpu.upload(a), gpu.upload(b), n))
    static = horovod_amd.lib().hvdhip_adasum_combine_static
    try:
        torch.cuda.synchronize()
        for _ in range(40):
            for (d_a, _, d_b, n), s in zip(data, (s1, s2)):
                horovod_amd.check(static(d_a.data_ptr(), d_b.data_ptr(), F32, n, None, s.handle),
                                  "hvdhip_adasum_combine_static")
        s1.synchronize()
        s2.synchronize()
        for d_a, d_ref, d_b, n in data:
            plan = gpu.H.AdasumPlan([n], F32)
            try:
                for _ in range(40):
                    plan.combine(d_ref.data_ptr(), d_b.data_ptr(), gpu.stream)
                gpu.sync()
            finally:
                plan.destroy()
            assert np.array_equal(gpu.download(d_a, np.uint32), gpu.download(d_ref, np.uint32)), n
    finally:
        s1.destroy()
        s2.destroy()
