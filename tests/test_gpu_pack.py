"""Parity of the HIP pack / unpack / batched-copy path with the CPU oracle,
through the C ABI.  Bit-exact for copies; scaled values compared bit-for-bit
with the oracle's ScaleBuffer on the same seeded inputs."""
import numpy as np
import pytest

from oracle_util import F16, F32, F64, I8, I32, I64, U8, U16, NP_OF, SIZE_OF

pytestmark = pytest.mark.gpu

from gpu_util import Arena  # noqa: E402

EDGE_BYTES = [0, 1, 2, 3, 15, 16, 17, 31, 32, 33, 255, 256, 257, 4095, 4096, 4097, 32767, 32768, 32769,
              65536 + 5, 3 * 32768 + 1]


def _rand_values(rng, n, dtype):
    np_t = NP_OF[dtype]
    if dtype in (F32, F64):
        return rng.uniform(-1, 1, n).astype(np_t)
    if dtype == F16:
        return rng.uniform(-1, 1, n).astype(np.float16)
    if dtype == I64:
        return rng.integers(-2 ** 40, 2 ** 40, n, dtype=np.int64)
    info = np.iinfo(np_t)
    return rng.integers(info.min, int(info.max) + 1, n, dtype=np.int64).astype(np_t)


def _build(gpu, rng, counts, dtype, misalign=None, out_misalign=None):
    """Places tensors (seeded values) and zeroed outputs in arenas; returns everything a test needs."""
    es = SIZE_OF[dtype]
    total = sum(c * es for c in counts) + 512 * (len(counts) + 2)
    src, dst = Arena(total), Arena(total, fill=0x5A)
    offs, ooffs, vals = [], [], []
    for i, c in enumerate(counts):
        m = 0 if misalign is None else misalign[i % len(misalign)]
        om = 0 if out_misalign is None else out_misalign[i % len(out_misalign)]
        o = src.alloc(c * es, misalign=m)
        oo = dst.alloc(c * es, misalign=om)
        v = _rand_values(rng, c, dtype)
        src.host[o:o + c * es] = v.view(np.uint8)
        offs.append(o)
        ooffs.append(oo)
        vals.append(v)
    src.upload()
    dst.upload()
    return src, dst, offs, ooffs, vals


def _raw(v):
    return v.view(np.uint16) if v.dtype == np.float16 else v


def _check_round_trip(gpu, orc, counts, dtype, prescale, postscale, misalign=None, out_misalign=None, seed=0):
    rng = np.random.default_rng(seed)
    es = SIZE_OF[dtype]
    src, dst, offs, ooffs, vals = _build(gpu, rng, counts, dtype, misalign, out_misalign)
    plan = gpu.H.FusionPlan([src.ptr(o) for o in offs], [dst.ptr(o) for o in ooffs], counts, dtype)
    try:
        want_offs = orc.padded_offsets([c * es for c in counts])
        assert plan.buffer_len == want_offs[-1]
        assert plan.offsets() == list(want_offs[:-1])
        fb = gpu.empty(plan.buffer_len + 64, fill=0xCD)
        plan.pack(fb.data_ptr(), prescale, gpu.stream)
        buf = gpu.download(fb)
        # per-tensor parity of the buffer contents with the oracle's ScaleBuffer
        scaled = []
        for i, (c, v) in enumerate(zip(counts, vals)):
            w = _raw(v) if prescale == 1.0 else orc.scale_buffer(_raw(v), prescale, dtype)
            scaled.append(w)
            got = buf[want_offs[i]:want_offs[i] + c * es]
            assert np.array_equal(got, w.view(np.uint8)), "pack: tensor %d of %d elements" % (i, c)
            pad = buf[want_offs[i] + c * es:want_offs[i + 1]]
            assert np.all(pad == 0), "pad bytes after tensor %d" % i
        assert np.all(buf[plan.buffer_len:] == 0xCD), "wrote past buffer_len"
        plan.unpack(fb.data_ptr(), postscale, gpu.stream)
        gpu.sync()
        out = dst.download()
        touched = np.zeros(out.size, bool)
        for i, (c, w) in enumerate(zip(counts, scaled)):
            z = w if postscale == 1.0 else orc.scale_buffer(w, postscale, dtype)
            got = out[ooffs[i]:ooffs[i] + c * es]
            assert np.array_equal(got, z.view(np.uint8)), "unpack: tensor %d of %d elements" % (i, c)
            touched[ooffs[i]:ooffs[i] + c * es] = True
        assert np.all(out[~touched] == 0x5A), "unpack wrote outside the outputs"
    finally:
        plan.destroy()


@pytest.mark.parametrize("dtype", [U8, I8, U16, I32, I64, F16, F32, F64])
def test_pack_unpack_copy_edge_sizes(gpu, orc, dtype):
    es = SIZE_OF[dtype]
    counts = [b // es for b in EDGE_BYTES]
    _check_round_trip(gpu, orc, counts, dtype, 1.0, 1.0, seed=1)


@pytest.mark.parametrize("dtype", [U8, I8, I32, I64, F16, F32, F64])
@pytest.mark.parametrize("prescale,postscale", [(0.125, 1.0), (1.0 / 3.0, 2.5), (0.3, 0.999)])
def test_pack_unpack_scaled_edge_sizes(gpu, orc, dtype, prescale, postscale):
    es = SIZE_OF[dtype]
    counts = [b // es for b in EDGE_BYTES]
    _check_round_trip(gpu, orc, counts, dtype, prescale, postscale, seed=2)


@pytest.mark.parametrize("dtype", [U8, F16, F32, F64])
def test_pack_unpack_every_misalignment(gpu, orc, dtype):
    # source and output tensors at every element-aligned offset within 16 bytes
    es = SIZE_OF[dtype]
    mis = list(range(0, 16, es))
    counts = [(1000 + 37 * i) // es + 1 for i in range(2 * len(mis))] + [40000 // es + 3]
    _check_round_trip(gpu, orc, counts, dtype, 1.0, 1.0, misalign=mis, out_misalign=mis[::-1], seed=3)
    if dtype != U8:
        _check_round_trip(gpu, orc, counts, dtype, 0.125, 1.0 / 3.0, misalign=mis, out_misalign=mis[::-1], seed=4)


def test_more_entries_than_the_reference_batch_capacity(gpu, orc):
    # 1,000 entries: the reference needs ceil(1000/160) launches (ops/gpu_operations.cc:145)
    rng = np.random.default_rng(5)
    counts = [int(x) for x in rng.integers(1, 3000, 1000)]
    _check_round_trip(gpu, orc, counts, F32, 0.125, 1.0, seed=5)


@pytest.mark.parametrize("dtype", [F16, F32])
def test_twenty_thousand_tiny_tensors(gpu, orc, dtype):
    """A response of very many very small tensors (0 to 40 elements, so most are shorter than
    the 16-byte pad unit and none fills a vector loop), packed misaligned to both sides."""
    rng = np.random.default_rng(21)
    counts = [int(c) for c in rng.integers(0, 41, 20000)]
    es = SIZE_OF[dtype]
    _check_round_trip(gpu, orc, counts, dtype, 0.125, 3.0, misalign=[0, es, 2 * es, 3 * es],
                      out_misalign=[3 * es, 0, es], seed=22)


def test_in_place_outputs_alias_tensors(gpu, orc):
    # allreduce_async_ passes output == tensor (torch/mpi_ops.py:265)
    rng = np.random.default_rng(6)
    counts = [1, 1023, 70001, 16]
    src, _, offs, _, vals = _build(gpu, rng, counts, F32)
    ptrs = [src.ptr(o) for o in offs]
    plan = gpu.H.FusionPlan(ptrs, ptrs, counts, F32)
    try:
        fb = gpu.empty(plan.buffer_len)
        plan.pack(fb.data_ptr(), 0.5, gpu.stream)
        plan.unpack(fb.data_ptr(), 3.0, gpu.stream)
        gpu.sync()
        out = src.download()
        for o, c, v in zip(offs, counts, vals):
            want = orc.scale_buffer(orc.scale_buffer(v, 0.5, F32), 3.0, F32)
            assert np.array_equal(out[o:o + 4 * c], want.view(np.uint8))
    finally:
        plan.destroy()


def test_empty_plan_and_zero_length_entries(gpu, orc):
    plan = gpu.H.FusionPlan([], [], [], F32)
    assert plan.buffer_len == 0 and plan.num_chunks == 0
    plan.pack(0, 0.5, gpu.stream)
    plan.unpack(0, 0.5, gpu.stream)
    gpu.sync()
    plan.destroy()
    _check_round_trip(gpu, orc, [0, 5, 0, 0, 9, 0], F32, 0.125, 1.0, seed=7)


@pytest.mark.parametrize("prescale", [0.125, 1.0, 1.0 / 3.0, 1e-3])
@pytest.mark.parametrize("flags", [0, 1])
def test_converting_pack_fp32_to_fp16(gpu, orc, prescale, flags):
    # values N(0,1e-4): after the prescale most results are subnormal halves
    rng = np.random.default_rng(8)
    counts = [b // 4 for b in EDGE_BYTES] + [100003]
    src = Arena(sum(counts) * 4 + 512 * (len(counts) + 2))
    dst = Arena(src.capacity, fill=0x5A)
    offs, ooffs, vals = [], [], []
    for i, c in enumerate(counts):
        o, oo = src.alloc(c * 4, misalign=4 * (i % 4)), dst.alloc(c * 4, misalign=4 * ((i + 1) % 4))
        v = (rng.standard_normal(c) * 1e-4).astype(np.float32)
        if c > 8:
            v[:8] = [0.0, -0.0, 65504.0, 65520.0, -1e9, 6.1e-5, 5.96e-8, 2.98e-8]
        src.host[o:o + 4 * c] = v.view(np.uint8)
        offs.append(o), ooffs.append(oo), vals.append(v)
    src.upload(), dst.upload()
    plan = gpu.H.FusionPlan([src.ptr(o) for o in offs], [dst.ptr(o) for o in ooffs], counts, F32, F16)
    try:
        want_offs = orc.padded_offsets([2 * c for c in counts])
        assert plan.buffer_len == want_offs[-1]
        fb = gpu.empty(plan.buffer_len + 64, fill=0xCD)
        plan.pack(fb.data_ptr(), prescale, gpu.stream, flags=flags)
        buf = gpu.download(fb)
        halves = []
        for i, (c, v) in enumerate(zip(counts, vals)):
            w = orc.scale_cast_f32_to_f16(v, prescale, cast_first=bool(flags))
            halves.append(w)
            got = buf[want_offs[i]:want_offs[i] + 2 * c].view(np.uint16)
            assert np.array_equal(got, w), "tensor %d: %d of %d halves differ" % (i, int((got != w).sum()), c)
            assert np.all(buf[want_offs[i] + 2 * c:want_offs[i + 1]] == 0)
        assert np.all(buf[plan.buffer_len:] == 0xCD)
        for postscale in (1.0, 4.0, 1.0 / 3.0):
            plan.unpack(fb.data_ptr(), postscale, gpu.stream)
            gpu.sync()
            out = dst.download()
            for i, (c, w) in enumerate(zip(counts, halves)):
                want = orc.scale_cast_f16_to_f32(w, postscale)
                got = out[ooffs[i]:ooffs[i] + 4 * c].view(np.uint32)
                assert np.array_equal(got, want.view(np.uint32)), "unpack tensor %d postscale %r" % (i, postscale)
    finally:
        plan.destroy()


def test_batched_d2d_memcpy_arbitrary_bytes(gpu, orc):
    # the byte-granular entry point: any size, any alignment on either side
    rng = np.random.default_rng(9)
    sizes = [0, 1, 2, 3, 5, 15, 16, 17, 100, 4097, 32768, 32771, 100001]
    sizes = sizes + sizes
    src = Arena(sum(sizes) + 512 * (len(sizes) + 2))
    dst = Arena(src.capacity, fill=0x5A)
    so, do = [], []
    for i, n in enumerate(sizes):
        so.append(src.alloc(n, misalign=i % 16))
        do.append(dst.alloc(n, misalign=(7 * i + 3) % 16))
        src.host[so[-1]:so[-1] + n] = rng.integers(0, 256, n, dtype=np.uint8)
    src.upload(), dst.upload()
    for rep in range(2):  # second call hits the table cache
        gpu.H.batched_d2d_memcpy([dst.ptr(o) for o in do], [src.ptr(o) for o in so], sizes, gpu.stream)
    gpu.sync()
    out = dst.download()
    touched = np.zeros(out.size, bool)
    for s, d, n in zip(so, do, sizes):
        assert np.array_equal(out[d:d + n], src.host[s:s + n])
        touched[d:d + n] = True
    assert np.all(out[~touched] == 0x5A)


@pytest.mark.parametrize("dtype,scale", [(F32, 0.125), (F32, 1.0), (F16, 1.0 / 3.0), (I32, 0.3), (F64, 0.7)])
def test_batched_scaled_d2d_memcpy(gpu, orc, dtype, scale):
    rng = np.random.default_rng(10)
    es = SIZE_OF[dtype]
    counts = [1, 3, 4, 5, 1000, 8193, 70001]
    src, dst, offs, ooffs, vals = _build(gpu, rng, counts, dtype, misalign=[0, es], out_misalign=[es, 0])
    gpu.H.batched_scaled_d2d_memcpy([dst.ptr(o) for o in ooffs], [src.ptr(o) for o in offs],
                                    [c * es for c in counts], scale, dtype, gpu.stream)
    gpu.sync()
    out = dst.download()
    for o, c, v in zip(ooffs, counts, vals):
        want = _raw(v) if scale == 1.0 else orc.scale_buffer(_raw(v), scale, dtype)
        assert np.array_equal(out[o:o + c * es], want.view(np.uint8))


def _cache_stats():
    import ctypes
    import horovod_amd
    v = [ctypes.c_uint64() for _ in range(4)]
    horovod_amd.check(horovod_amd.lib().hvdhip_copy_cache_stats(*[ctypes.byref(x) for x in v]), "stats")
    return dict(zip(("hits", "misses", "evictions", "entries"), [x.value for x in v]))


def _cache_limits(entries, nbytes):
    import horovod_amd
    horovod_amd.check(horovod_amd.lib().hvdhip_copy_cache_set_limits(entries, nbytes), "set_limits")


def test_batched_copy_tables_stay_resident_over_a_gpt2_sized_step(gpu):
    """A GPT-2 XL step has 49 fusion cycles, each with a copy set in and a copy set out: 98 distinct
    (out, in, sizes) sets through the array-taking entry points, alternating over two streams.  Every
    set builds its table in the first step and finds it in every later one; nothing is evicted."""
    import horovod_amd
    rng = np.random.default_rng(21)
    nsets, per = 98, 12
    src = Arena(24 << 20)
    dst = Arena(24 << 20, fill=0x5A)
    sets = []
    for _ in range(nsets):
        sizes = [4 * int(x) for x in rng.integers(1, 4000, per)]
        so = [src.alloc(n, align=16) for n in sizes]
        do = [dst.alloc(n, align=16) for n in sizes]
        for o, n in zip(so, sizes):
            src.host[o:o + n] = rng.integers(0, 256, n, dtype=np.uint8)
        sets.append((None, so, do, sizes))
    src.upload(), dst.upload()
    streams = [horovod_amd.Stream(), horovod_amd.Stream()]
    before = _cache_stats()
    after_step = []
    for step in range(3):
        for i, (_, so, do, sizes) in enumerate(sets):
            st = streams[i % 2]
            if i % 3 == 0:  # a third of the sets go through the scaled entry point
                gpu.H.batched_scaled_d2d_memcpy([dst.ptr(o) for o in do], [src.ptr(o) for o in so], sizes, 1.0,
                                                F32, st)
            else:
                gpu.H.batched_d2d_memcpy([dst.ptr(o) for o in do], [src.ptr(o) for o in so], sizes, st)
        after_step.append(_cache_stats())
    for st in streams:
        st.synchronize()
    assert after_step[0]["misses"] - before["misses"] == nsets
    assert after_step[1]["misses"] == after_step[0]["misses"], "tables were rebuilt in the second step"
    assert after_step[2]["misses"] == after_step[0]["misses"], "tables were rebuilt in the third step"
    assert after_step[2]["hits"] - after_step[0]["hits"] == 2 * nsets
    assert after_step[2]["evictions"] == before["evictions"]
    out = dst.download()
    for _, so, do, sizes in sets:
        for s_, d_, n in zip(so, do, sizes):
            assert np.array_equal(out[d_:d_ + n], src.host[s_:s_ + n])
    for st in streams:
        st.destroy()


def test_batched_copy_cache_eviction_from_several_threads(gpu):
    # more distinct copy sets than the table cache may hold (limited to 64 here), issued from four
    # threads on four streams: tables are evicted and their buffers reused while launches are in flight
    import threading
    import horovod_amd
    _cache_limits(64, 256 << 20)
    evicted_before = _cache_stats()["evictions"]
    rng = np.random.default_rng(12)
    nsets, per = 40, 6
    src = Arena(4 << 20)
    dst = Arena(4 << 20, fill=0x5A)
    sets = []
    for s_ in range(4 * nsets):
        sizes = [int(x) for x in rng.integers(1, 3000, per)]
        so = [src.alloc(n, align=16) for n in sizes]
        do = [dst.alloc(n, align=16) for n in sizes]
        for o, n in zip(so, sizes):
            src.host[o:o + n] = rng.integers(0, 256, n, dtype=np.uint8)
        sets.append((so, do, sizes))
    src.upload(), dst.upload()
    errors = []

    def worker(t):
        try:
            horovod_amd.lib().hvdhip_set_device(0)
            st = horovod_amd.Stream()
            for rep in range(2):
                for so, do, sizes in sets[t * nsets:(t + 1) * nsets]:
                    gpu.H.batched_d2d_memcpy([dst.ptr(o) for o in do], [src.ptr(o) for o in so], sizes, st)
            st.synchronize()
            st.destroy()
        except Exception as e:  # pragma: no cover
            errors.append(e)

    ts = [threading.Thread(target=worker, args=(t,)) for t in range(4)]
    [t.start() for t in ts]
    [t.join() for t in ts]
    stats = _cache_stats()
    _cache_limits(4096, 256 << 20)
    assert not errors, errors
    assert stats["evictions"] - evicted_before >= 4 * nsets - 64 and stats["entries"] <= 64
    out = dst.download()
    for so, do, sizes in sets:
        for s_, d_, n in zip(so, do, sizes):
            assert np.array_equal(out[d_:d_ + n], src.host[s_:s_ + n])


def test_batched_copy_cache_bounded_by_bytes(gpu):
    # the limit that matters is the device memory the tables take: with room for three 4 KiB tables,
    # five sets evict, and every copy is still right
    rng = np.random.default_rng(14)
    _cache_limits(4096, 3 * 4096)
    before = _cache_stats()
    src = Arena(1 << 20)
    dst = Arena(1 << 20, fill=0x5A)
    sets = []
    for _ in range(5):
        sizes = [int(x) for x in rng.integers(1, 5000, 9)]
        so = [src.alloc(n, align=16) for n in sizes]
        do = [dst.alloc(n, align=16) for n in sizes]
        for o, n in zip(so, sizes):
            src.host[o:o + n] = rng.integers(0, 256, n, dtype=np.uint8)
        sets.append((so, do, sizes))
    src.upload(), dst.upload()
    for rep in range(2):
        for so, do, sizes in sets:
            gpu.H.batched_d2d_memcpy([dst.ptr(o) for o in do], [src.ptr(o) for o in so], sizes, gpu.stream)
    gpu.sync()
    stats = _cache_stats()
    _cache_limits(4096, 256 << 20)
    assert stats["entries"] <= 3 and stats["evictions"] - before["evictions"] >= 7
    out = dst.download()
    for so, do, sizes in sets:
        for s_, d_, n in zip(so, do, sizes):
            assert np.array_equal(out[d_:d_ + n], src.host[s_:s_ + n])


def test_batched_copy_table_built_on_one_stream_used_on_another(gpu):
    # a miss uploads its table asynchronously on the calling stream; a hit from another stream
    # right behind it must wait for that upload
    import horovod_amd
    rng = np.random.default_rng(13)
    a, b = horovod_amd.Stream(), horovod_amd.Stream()
    n = 3000
    sizes = [int(x) for x in rng.integers(1, 9000, n)]
    src = Arena(sum(sizes) + 32 * n + 4096)
    so = [src.alloc(x, align=16) for x in sizes]
    for o, x in zip(so, sizes):
        src.host[o:o + x] = rng.integers(0, 256, x, dtype=np.uint8)
    src.upload()
    for rep in range(5):
        dst = Arena(src.capacity + 64 * rep, fill=0x5A)
        do = [dst.alloc(x, misalign=rep, align=16) for x in sizes]
        dst.upload()
        out_ptrs, in_ptrs = [dst.ptr(o) for o in do], [src.ptr(o) for o in so]
        gpu.H.batched_d2d_memcpy(out_ptrs, in_ptrs, sizes, a)   # miss: builds and uploads on a
        gpu.H.batched_d2d_memcpy(out_ptrs, in_ptrs, sizes, b)   # hit on b
        a.synchronize(), b.synchronize()
        out = dst.download()
        for s_, d_, x in zip(so, do, sizes):
            assert np.array_equal(out[d_:d_ + x], src.host[s_:s_ + x])
    a.destroy(), b.destroy()


def test_rejected_arguments(gpu):
    import horovod_amd
    L = horovod_amd.lib()
    with pytest.raises(horovod_amd.HvdHipError) as e:
        gpu.H.FusionPlan([1024], [1024], [4], F16, F32)  # only fp32 tensors in an fp16 buffer convert
    assert e.value.code == -2
    with pytest.raises(horovod_amd.HvdHipError):
        gpu.H.FusionPlan([1026], [1024], [4], F32)  # misaligned for its element size
    t = gpu.empty(64)
    plan = gpu.H.FusionPlan([t.data_ptr()], [t.data_ptr()], [4], U16)
    with pytest.raises(horovod_amd.HvdHipError) as e:
        plan.pack(t.data_ptr(), 0.5, gpu.stream)  # UINT16 cannot be scaled (collective_operations.cc:141-144)
    assert e.value.code == -2
    with pytest.raises(horovod_amd.HvdHipError):
        plan.pack(t.data_ptr() + 8, 1.0, gpu.stream)  # fusion buffer must be 16-byte aligned
    plan.destroy()


def _acquire(stream):
    import ctypes
    import horovod_amd
    ev = ctypes.c_void_p()
    horovod_amd.check(horovod_amd.lib().hvdhip_event_acquire(stream.handle, ctypes.byref(ev)), "hvdhip_event_acquire")
    return ev


def _event_done(ev):
    import ctypes
    import horovod_amd
    done = ctypes.c_int(-1)
    horovod_amd.check(horovod_amd.lib().hvdhip_event_query(ev, ctypes.byref(done)), "hvdhip_event_query")
    return done.value


@pytest.mark.parametrize("dtype,buffer_dtype,postscale", [(F32, F32, 1.0), (F32, F32, 0.5), (F16, F16, 0.25),
                                                          (F32, F16, 1.0), (U8, U8, 1.0)])
def test_unpack_that_records_its_completion_event(gpu, orc, dtype, buffer_dtype, postscale):
    """hvdhip_fusion_unpack_record = unpack followed by a record of the event (ops/gpu_operations.cc:82):
    once the event has completed the outputs are whole, for a host that waits on the event and
    for another stream that waits on it; the pooled event serves again afterwards."""
    import horovod_amd
    import torch
    L = horovod_amd.lib()
    rng = np.random.default_rng(11)
    es = SIZE_OF[dtype]
    counts = [int(c) for c in rng.integers(1, 400000, 37)] + [3, 0, 1 << 21]
    src, dst, offs, ooffs, vals = _build(gpu, rng, counts, dtype)
    plan = gpu.H.FusionPlan([src.ptr(o) for o in offs], [dst.ptr(o) for o in ooffs], counts, dtype, buffer_dtype)
    other = horovod_amd.Stream()
    copy = torch.zeros_like(dst.dev)
    try:
        fb = gpu.empty(plan.buffer_len + 64)
        cof = plan.offsets()
        bes = SIZE_OF[buffer_dtype]
        for turn, scale in enumerate((postscale, 1.0, postscale)):
            plan.pack(fb.data_ptr(), 1.0, gpu.stream)
            dst.dev.fill_(0x5A)
            torch.cuda.synchronize()
            ev = _acquire(gpu.stream)
            plan.unpack(fb.data_ptr(), scale, gpu.stream, event=ev)
            if turn == 1:
                # a second stream waits for the event and copies the outputs; only that stream is waited for
                horovod_amd.check(L.hvdhip_stream_wait_event(other.handle, ev), "hvdhip_stream_wait_event")
                horovod_amd.check(L.hvdhip_memcpy_async(copy.data_ptr(), dst.dev.data_ptr(), dst.dev.numel(), 3,
                                                        other.handle), "hvdhip_memcpy_async")
                other.synchronize()
                out = copy.cpu().numpy()
            else:
                horovod_amd.check(L.hvdhip_event_synchronize(ev), "hvdhip_event_synchronize")
                out = dst.dev.cpu().numpy()  # no wait for the stream itself
            assert _event_done(ev) == 1
            horovod_amd.check(L.hvdhip_event_release(gpu.stream.handle, ev), "hvdhip_event_release")
            buf = gpu.download(fb)
            for i, c in enumerate(counts):
                b = buf[cof[i]:cof[i] + c * bes]
                if buffer_dtype != dtype:
                    want = orc.scale_cast_f16_to_f32(b.view(np.uint16), scale)
                elif scale == 1.0:
                    want = b
                else:
                    want = orc.scale_buffer(b.view(NP_OF[dtype]) if dtype != F16 else b.view(np.uint16), scale, dtype)
                got = out[ooffs[i]:ooffs[i] + c * es]
                assert np.array_equal(got, want.view(np.uint8)), "turn %d tensor %d" % (turn, i)
    finally:
        gpu.sync()
        other.destroy()
        plan.destroy()


def test_unpack_record_without_payload_records_the_event(gpu):
    import horovod_amd
    L = horovod_amd.lib()
    plan = gpu.H.FusionPlan([], [], [], F32)
    ev = _acquire(gpu.stream)
    plan.unpack(0, 1.0, gpu.stream, event=ev)
    horovod_amd.check(L.hvdhip_event_synchronize(ev), "hvdhip_event_synchronize")
    assert _event_done(ev) == 1
    horovod_amd.check(L.hvdhip_event_release(gpu.stream.handle, ev), "hvdhip_event_release")
    assert L.hvdhip_fusion_unpack_record(plan.handle, None, 1.0, gpu.stream.handle, None) == -1  # event is NULL
    plan.destroy()


@pytest.mark.parametrize("nchunks", [1, 2, 7, 8, 9, 31, 32, 33, 63, 64, 65, 255, 256, 257, 511, 512, 513, 4095, 4096, 4097])
def test_table_sizes_around_the_group_boundaries(gpu, orc, nchunks):
    """Chunk tables are padded to a multiple of 32 entries and read through a mapping that permutes
    entries within groups of 32 (and chunks within runs per XCD, in groups of 512): chunk counts on
    both sides of every boundary, as one big tensor, as one-chunk tensors, and as a ragged mix, each
    packed with a prescale and unpacked with a postscale, every byte inside and outside checked."""
    per = 1024  # fp32 elements of a 4 KiB chunk
    _check_round_trip(gpu, orc, [nchunks * per - 3], F32, 0.5, 0.25, seed=nchunks)
    if nchunks <= 513:
        _check_round_trip(gpu, orc, [per] * nchunks, F32, 0.5, 1.0, seed=nchunks + 1)
        rng = np.random.default_rng(nchunks)
        counts, left = [], nchunks
        while left > 0:
            k = int(min(left, rng.integers(1, 6)))
            counts.append(k * per - int(rng.integers(0, per - 1)))
            left -= k
        _check_round_trip(gpu, orc, counts, F32, 1.0, 0.5, seed=nchunks + 2)
