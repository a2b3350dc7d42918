"""Sizes beyond 32-bit byte counts, and replay from a captured HIP graph."""
import numpy as np
import pytest
import torch

from oracle_util import F16, F32, I8, U8

pytestmark = pytest.mark.gpu


def test_tensor_larger_than_4_gib(gpu, orc):
    # one 4.5 GiB entry: more than 2^32 bytes, 1.2 M workgroups; checked by sampled windows and checksums
    n = (9 << 29) + 12345
    g = torch.Generator(device="cuda")
    g.manual_seed(3)
    src = torch.randint(0, 256, (n,), generator=g, device="cuda", dtype=torch.uint8)
    dst = torch.zeros(n + 64, dtype=torch.uint8, device="cuda")
    plan = gpu.H.FusionPlan([src.data_ptr()], [dst.data_ptr()], [n], U8)
    assert plan.buffer_len == (n + 15) // 16 * 16
    fb = torch.full((plan.buffer_len + 64,), 0xCD, dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()
    plan.pack(fb.data_ptr(), 1.0, gpu.stream)
    plan.unpack(fb.data_ptr(), 1.0, gpu.stream)
    gpu.sync()
    assert torch.equal(fb[:n], src) and torch.equal(dst[:n], src)
    assert int(fb[n:plan.buffer_len].max()) == 0 and int(fb[plan.buffer_len:].min()) == 0xCD
    assert int(dst[n:].max()) == 0
    plan.destroy()
    del fb, dst
    torch.cuda.empty_cache()
    # whole-buffer scale over more than 2^32 int8 elements, in place, against the oracle on windows
    x = (src.view(torch.int8) // 4)
    keep = x.clone()
    torch.cuda.synchronize()  # torch's stream and the library's stream are unordered otherwise
    gpu.H.scale_buffer(x.data_ptr(), x.data_ptr(), n, 2.5, I8, gpu.stream)
    gpu.sync()
    for start in (0, (1 << 32) - 1000, n - 5000):
        w = keep[start:start + 4000].cpu().numpy()
        assert np.array_equal(x[start:start + 4000].cpu().numpy(), orc.scale_buffer(w, 2.5, I8))
    want_sum = torch.trunc(keep[::4099].double() * 2.5).sum()
    assert x[::4099].double().sum() == want_sum


def test_reduce_and_adasum_beyond_2_31_elements(gpu, orc):
    n = (1 << 31) + 4096 + 3
    a = torch.full((n,), 3, dtype=torch.int8, device="cuda")
    b = torch.full((n,), 5, dtype=torch.int8, device="cuda")
    b[-1] = 120
    torch.cuda.synchronize()
    gpu.H.reduce_sum(a.data_ptr(), b.data_ptr(), n, I8, gpu.stream)
    gpu.sync()
    assert int(a[:-1].min()) == 8 and int(a[:-1].max()) == 8 and int(a[-1]) == 123
    del a, b
    torch.cuda.empty_cache()
    # Adasum layer counts are ints (adasum.h:413: `int count`): two layers of 2^30 halves sum past 2^31 elements
    counts = [1 << 30, (1 << 30) + 7]
    x = torch.ones(sum(counts), dtype=torch.float16, device="cuda")
    y = torch.ones(sum(counts), dtype=torch.float16, device="cuda")
    plan = gpu.H.AdasumPlan(counts, F16)
    torch.cuda.synchronize()
    plan.combine(x.data_ptr(), y.data_ptr(), gpu.stream)
    nd, co = plan.read(gpu.stream)
    assert nd == [float(counts[0])] * 3 + [float(counts[1])] * 3  # exact in double
    assert co == [0.5, 0.5, 0.5, 0.5]
    assert int((x != 1).sum()) == 0  # identical vectors: the average is the vector itself
    plan.destroy()


def test_contiguous_kernels_slice_beyond_one_launch(gpu):
    # 33 GiB of int8: more than 2^23 workgroups of 4 KiB, so scale and reduce run as two launches each
    n = (33 << 30) + 777
    x = torch.full((n,), 4, dtype=torch.int8, device="cuda")
    y = torch.full((n,), 7, dtype=torch.int8, device="cuda")
    x[-1] = 8
    torch.cuda.synchronize()
    gpu.H.scale_buffer(x.data_ptr(), x.data_ptr(), n, 2.5, I8, gpu.stream)
    gpu.sync()
    assert int(x[:-1].min()) == 10 and int(x[:-1].max()) == 10 and int(x[-1]) == 20
    gpu.H.reduce_sum(x.data_ptr(), y.data_ptr(), n, I8, gpu.stream)
    gpu.sync()
    assert int(x[:-1].min()) == 17 and int(x[:-1].max()) == 17 and int(x[-1]) == 27
    # a plan of that size is refused rather than mis-launched
    import horovod_amd
    with pytest.raises(horovod_amd.HvdHipError) as e:
        gpu.H.FusionPlan([x.data_ptr()], [y.data_ptr()], [n], U8)
    assert e.value.code == -4


def test_pipeline_replays_from_a_hip_graph(gpu, orc):
    """pack -> reduce -> unpack captured once and replayed: the entry points only launch kernels
    (no allocation, no memset), so they can be captured; every replay must equal the eager result."""
    rng = np.random.default_rng(11)
    counts = [1, 4097, 70001, 255, 33000]
    vals = [rng.standard_normal(c).astype(np.float32) for c in counts]
    d_in = [torch.from_numpy(v).cuda() for v in vals]
    d_out = [torch.zeros(c, dtype=torch.float32, device="cuda") for c in counts]
    plan = gpu.H.FusionPlan([t.data_ptr() for t in d_in], [t.data_ptr() for t in d_out], counts, F32)
    fb = torch.zeros(plan.buffer_len, dtype=torch.uint8, device="cuda")
    peer = torch.from_numpy(rng.standard_normal(plan.buffer_len // 4).astype(np.float32)).cuda()
    offs = plan.offsets()
    peer_host = peer.cpu().numpy()

    def expected():
        out = []
        for v, o in zip(vals, offs):
            w = orc.sum(peer_host[o // 4:o // 4 + v.size], orc.scale_buffer(v, 0.125, F32), F32)
            out.append(orc.scale_buffer(w, 0.5, F32))
        return out

    side = torch.cuda.Stream()
    cap = gpu.H.Stream(side.cuda_stream)
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        # eager once on the capture stream (plans are built, nothing is left to allocate)
        plan.pack(fb.data_ptr(), 0.125, cap)
        gpu.H.reduce_sum(fb.data_ptr(), peer.data_ptr(), plan.buffer_len // 4, F32, cap)
        plan.unpack(fb.data_ptr(), 0.5, cap)
        side.synchronize()
        eager = [t.clone() for t in d_out]
        with torch.cuda.graph(graph, stream=side):
            plan.pack(fb.data_ptr(), 0.125, cap)
            gpu.H.reduce_sum(fb.data_ptr(), peer.data_ptr(), plan.buffer_len // 4, F32, cap)
            plan.unpack(fb.data_ptr(), 0.5, cap)
    torch.cuda.synchronize()
    for e, w in zip(eager, expected()):
        assert np.array_equal(e.cpu().numpy().view(np.uint32), w.view(np.uint32))
    for rep in range(4):
        # new inputs between replays, written by ordinary eager work
        vals = [rng.standard_normal(c).astype(np.float32) for c in counts]
        for t, v in zip(d_in, vals):
            t.copy_(torch.from_numpy(v))
        for t in d_out:
            t.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for t, w in zip(d_out, expected()):
            assert np.array_equal(t.cpu().numpy().view(np.uint32), w.view(np.uint32)), "replay %d" % rep
    plan.destroy()
