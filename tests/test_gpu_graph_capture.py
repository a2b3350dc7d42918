"""Plan-based entry points launch kernels and nothing else (no allocation, no memset, no
synchronisation), so a caller may record them into a HIP graph.  One fused cycle and one
Adasum combine are captured on a side stream and replayed with fresh inputs; every replay
must equal what the same calls give eagerly."""
import numpy as np
import pytest
import torch

from oracle_util import F16, F32

pytestmark = pytest.mark.gpu


def test_captured_cycle_replays_like_the_eager_calls(gpu):
    import horovod_amd
    counts = [5, 1000, 3, 70001, 256, 1, 4099]
    side = torch.cuda.Stream()
    s = horovod_amd.Stream(side.cuda_stream)
    srcs = [torch.zeros(c, device="cuda") for c in counts]
    outs = [torch.zeros(c, device="cuda") for c in counts]
    eager_outs = [torch.zeros(c, device="cuda") for c in counts]
    plan = gpu.H.FusionPlan([t.data_ptr() for t in srcs], [t.data_ptr() for t in outs], counts, F32, F16)
    eager = gpu.H.FusionPlan([t.data_ptr() for t in srcs], [t.data_ptr() for t in eager_outs], counts, F32, F16)
    fb = torch.empty(plan.buffer_len, dtype=torch.uint8, device="cuda")
    fb2 = torch.empty(plan.buffer_len, dtype=torch.uint8, device="cuda")
    peers = [torch.zeros(plan.buffer_len // 2, dtype=torch.float16, device="cuda") for _ in range(3)]
    n = plan.buffer_len // 2

    def cycle(p, buf):
        p.pack(buf.data_ptr(), 0.125, s)
        gpu.H.reduce_sum_k(buf.data_ptr(), [t.data_ptr() for t in peers], n, F16, s)
        gpu.H.scale_buffer(buf.data_ptr(), buf.data_ptr(), n, 0.5, F16, s)
        p.unpack(buf.data_ptr(), 2.0, s)

    try:
        torch.cuda.synchronize()
        with torch.cuda.stream(side):
            cycle(plan, fb)  # warm-up outside the capture
            side.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=side):
                cycle(plan, fb)
            side.synchronize()
        gen = torch.Generator(device="cuda")
        for replay in range(4):
            gen.manual_seed(replay)
            for t in srcs:
                t.copy_(torch.randn(t.shape, generator=gen, device="cuda") * 1e-2)
            for t in peers:
                t.copy_((torch.randn(t.shape, generator=gen, device="cuda") * 1e-2).half())
            for t in outs:
                t.fill_(-1.0)
            torch.cuda.synchronize()
            g.replay()
            torch.cuda.synchronize()
            cycle(eager, fb2)
            s.synchronize()
            torch.cuda.synchronize()
            for a, b in zip(outs, eager_outs):
                assert torch.equal(a.view(torch.int32), b.view(torch.int32)), "replay %d" % replay
            assert any(float(t.abs().sum()) > 0 for t in outs)
    finally:
        torch.cuda.synchronize()
        plan.destroy()
        eager.destroy()


def test_captured_adasum_combine_replays_like_the_eager_call(gpu):
    import horovod_amd
    counts = [4099, 7, 0, 100000]
    total = sum(counts)
    side = torch.cuda.Stream()
    s = horovod_amd.Stream(side.cuda_stream)
    a, b, a2 = (torch.zeros(total, device="cuda") for _ in range(3))
    plan, eager = gpu.H.AdasumPlan(counts, F32), gpu.H.AdasumPlan(counts, F32)
    try:
        torch.cuda.synchronize()
        with torch.cuda.stream(side):
            plan.combine(a.data_ptr(), b.data_ptr(), s)
            side.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=side):
                plan.combine(a.data_ptr(), b.data_ptr(), s)
            side.synchronize()
        gen = torch.Generator(device="cuda")
        for replay in range(4):
            gen.manual_seed(10 + replay)
            a.copy_(torch.randn(total, generator=gen, device="cuda"))
            b.copy_(0.3 * a + torch.randn(total, generator=gen, device="cuda"))
            a2.copy_(a)
            torch.cuda.synchronize()
            g.replay()
            torch.cuda.synchronize()
            eager.combine(a2.data_ptr(), b.data_ptr(), s)
            s.synchronize()
            nd1, co1 = plan.read(s)
            nd2, co2 = eager.read(s)
            assert np.array_equal(np.array(nd1), np.array(nd2)) and np.array_equal(np.array(co1), np.array(co2))
            assert torch.equal(a.view(torch.int32), a2.view(torch.int32)), "replay %d" % replay
    finally:
        torch.cuda.synchronize()
        plan.destroy()
        eager.destroy()
