"""Streams, pooled events and async copies: the member set of GPUContext::impl
(ops/cuda_operations.cc:28-210) behind the C ABI."""
import ctypes
import threading

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_device_and_stream(gpu):
    import horovod_amd
    L = horovod_amd.lib()
    dev = ctypes.c_int(-1)
    horovod_amd.check(L.hvdhip_get_device(ctypes.byref(dev)), "get_device")
    assert dev.value == 0
    horovod_amd.check(L.hvdhip_set_device(0), "set_device")
    assert L.hvdhip_set_device(1 << 20) > 0  # a hipError_t, reported not thrown
    assert b"hipSetDevice" in L.hvdhip_last_error()
    s = horovod_amd.Stream()
    s.synchronize()
    s.destroy()


def test_event_pool_prepopulates_128_and_recycles(gpu):
    import horovod_amd
    L = horovod_amd.lib()
    s = horovod_amd.Stream()
    n = ctypes.c_int()
    L.hvdhip_event_pool_size(s.handle, ctypes.byref(n))
    assert n.value == 0
    ev = ctypes.c_void_p()
    horovod_amd.check(L.hvdhip_event_acquire(s.handle, ctypes.byref(ev)), "acquire")
    L.hvdhip_event_pool_size(s.handle, ctypes.byref(n))
    assert n.value == 127  # N_CUDA_EVENTS_PREPOPULATE = 128, one taken
    horovod_amd.check(L.hvdhip_event_record(ev, s.handle), "record")
    horovod_amd.check(L.hvdhip_event_synchronize(ev), "sync")
    done = ctypes.c_int(-1)
    horovod_amd.check(L.hvdhip_event_query(ev, ctypes.byref(done)), "query")
    assert done.value == 1
    horovod_amd.check(L.hvdhip_event_release(s.handle, ev), "release")
    L.hvdhip_event_pool_size(s.handle, ctypes.byref(n))
    assert n.value == 128
    # drain past the pool: the 129th event is created on demand
    taken = []
    for _ in range(130):
        e = ctypes.c_void_p()
        horovod_amd.check(L.hvdhip_event_acquire(s.handle, ctypes.byref(e)), "acquire")
        taken.append(e)
    assert len({e.value for e in taken}) == 130
    for e in taken:
        L.hvdhip_event_release(s.handle, e)
    L.hvdhip_event_pool_size(s.handle, ctypes.byref(n))
    assert n.value == 130
    s.destroy()


def test_event_pool_is_thread_safe(gpu):
    # finalizer threads release while the background thread acquires (ops/gpu_operations.cc:72-99)
    import horovod_amd
    L = horovod_amd.lib()
    s = horovod_amd.Stream()
    errors = []

    def worker():
        try:
            L.hvdhip_set_device(0)
            for _ in range(300):
                e = ctypes.c_void_p()
                assert L.hvdhip_event_acquire(s.handle, ctypes.byref(e)) == 0
                assert L.hvdhip_event_record(e, s.handle) == 0
                assert L.hvdhip_event_synchronize(e) == 0
                assert L.hvdhip_event_release(s.handle, e) == 0
        except Exception as ex:  # pragma: no cover
            errors.append(ex)

    ts = [threading.Thread(target=worker) for _ in range(4)]
    [t.start() for t in ts]
    [t.join() for t in ts]
    assert not errors
    n = ctypes.c_int()
    L.hvdhip_event_pool_size(s.handle, ctypes.byref(n))
    assert n.value >= 128
    s.destroy()


def test_stream_wait_event_orders_two_streams(gpu, orc):
    # pack on stream A, record; stream B waits on the event and unpacks: no host sync in between
    import horovod_amd
    from oracle_util import F32
    L = horovod_amd.lib()
    a, b = horovod_amd.Stream(), horovod_amd.Stream()
    rng = np.random.default_rng(1)
    x = rng.standard_normal(1 << 20).astype(np.float32)
    d_x, d_y = gpu.upload(x), gpu.empty(x.nbytes, fill=0)
    plan = gpu.H.FusionPlan([d_x.data_ptr()], [d_y.data_ptr()], [x.size], F32)
    fb = gpu.empty(plan.buffer_len)
    ev = ctypes.c_void_p()
    horovod_amd.check(L.hvdhip_event_acquire(a.handle, ctypes.byref(ev)), "acquire")
    for _ in range(3):
        plan.pack(fb.data_ptr(), 0.125, a)
        horovod_amd.check(L.hvdhip_event_record(ev, a.handle), "record")
        horovod_amd.check(L.hvdhip_stream_wait_event(b.handle, ev), "wait")
        plan.unpack(fb.data_ptr(), 1.0, b)
        b.synchronize()
    got = gpu.download(d_y, np.float32)
    assert np.array_equal(got, orc.scale_buffer(x, 0.125, F32))
    L.hvdhip_event_release(a.handle, ev)
    plan.destroy()
    a.destroy(), b.destroy()


def test_memcpy_async_kinds(gpu):
    import horovod_amd
    import torch
    L = horovod_amd.lib()
    x = torch.arange(4096, dtype=torch.float32).pin_memory()
    y = torch.zeros(4096, dtype=torch.float32).pin_memory()
    d1, d2 = gpu.empty(x.numel() * 4), gpu.empty(x.numel() * 4)
    s = gpu.stream
    horovod_amd.check(L.hvdhip_memcpy_async(d1.data_ptr(), x.data_ptr(), 16384, 1, s.handle), "h2d")
    horovod_amd.check(L.hvdhip_memcpy_async(d2.data_ptr(), d1.data_ptr(), 16384, 3, s.handle), "d2d")
    horovod_amd.check(L.hvdhip_memcpy_async(y.data_ptr(), d2.data_ptr(), 16384, 2, s.handle), "d2h")
    s.synchronize()
    assert torch.equal(x, y)
    assert L.hvdhip_memcpy_async(y.data_ptr(), d2.data_ptr(), 16, 99, s.handle) == -1


def test_timer_measures_stream_time(gpu):
    import horovod_amd
    from oracle_util import F32
    t = horovod_amd.Timer()
    d = gpu.empty(64 << 20)
    t.start(gpu.stream)
    for _ in range(10):
        gpu.H.scale_buffer(d.data_ptr(), d.data_ptr(), (64 << 20) // 4, 1.0001, F32, gpu.stream)
    t.stop(gpu.stream)
    ms = t.elapsed_ms()
    assert 0.0 < ms < 1000.0
    t.destroy()


def test_a_callers_stream_is_forgotten_and_usable_again(gpu, orc):
    """hvdhip_stream_forget on a stream that the caller owns (torch's here): work queued on it
    finishes first, the stream's pooled events go, and the entry points that remember streams
    (pooled events, cached copy tables, the single-layer Adasum plans) work on it afterwards as on a
    stream they have never seen."""
    import horovod_amd
    import torch
    from oracle_util import F32
    L = horovod_amd.lib()
    side = torch.cuda.Stream()
    s = horovod_amd.Stream(side.cuda_stream)
    rng = np.random.default_rng(5)
    sizes = [int(x) for x in rng.integers(1, 200000, 300)]
    offs = np.concatenate([[0], np.cumsum([(x + 15) // 16 * 16 for x in sizes])]).astype(np.int64)
    host = rng.integers(0, 256, int(offs[-1]), dtype=np.uint8)
    src = gpu.upload(host)
    a = rng.standard_normal(50001).astype(np.float32)
    b = rng.standard_normal(50001).astype(np.float32)
    d_a, d_b = gpu.upload(a), gpu.upload(b)
    n = ctypes.c_int()
    for rep in range(2):
        dst = gpu.empty(int(offs[-1]), fill=0)
        torch.cuda.synchronize()
        ev = ctypes.c_void_p()
        horovod_amd.check(L.hvdhip_event_acquire(s.handle, ctypes.byref(ev)), "acquire")
        L.hvdhip_event_pool_size(s.handle, ctypes.byref(n))
        assert n.value == 127  # a fresh pool both times
        gpu.H.batched_d2d_memcpy([dst.data_ptr() + int(o) for o in offs[:-1]],
                                 [src.data_ptr() + int(o) for o in offs[:-1]], sizes, s)
        horovod_amd.check(L.hvdhip_event_record(ev, s.handle), "record")
        dot, an, bn = ctypes.c_double(), ctypes.c_double(), ctypes.c_double()
        horovod_amd.check(L.hvdhip_adasum_dot_and_norm_sqrds(d_a.data_ptr(), d_b.data_ptr(), F32, a.size,
                                                             ctypes.byref(dot), ctypes.byref(an), ctypes.byref(bn),
                                                             s.handle), "dot")
        assert np.allclose([dot.value, an.value, bn.value], orc.adasum_dot_norms(a, b, F32), rtol=1e-12, atol=0)
        # one more copy left queued: forget waits for it
        gpu.H.batched_d2d_memcpy([dst.data_ptr() + int(o) for o in offs[:-1]],
                                 [src.data_ptr() + int(o) for o in offs[:-1]], sizes, s)
        horovod_amd.check(L.hvdhip_event_release(s.handle, ev), "release")
        horovod_amd.check(L.hvdhip_stream_forget(s.handle), "forget")
        assert side.query()  # nothing left running on the stream
        L.hvdhip_event_pool_size(s.handle, ctypes.byref(n))
        assert n.value == 0
        out = dst.cpu().numpy()
        for o, x in zip(offs[:-1], sizes):
            assert np.array_equal(out[o:o + x], host[o:o + x])
