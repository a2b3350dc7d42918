"""Every local rank's share of the reduce-scatter, played out on one device.

NCCLHierarchicalAllreduce::Execute (ops/nccl_operations.cc:255-430) packs, reduce-scatters the
buffer so that rank r ends up with the sum of everybody's share r at its own rank offset
(buffer_data_at_rank_offset), lets the last rank also reduce the elements that do not divide,
gathers the shares back into every buffer and unpacks.  Here the ranks are buffers on one GPU:
every rank packs its own tensors with the library, reduces its own range with
hvdhip_reduce_sum_k against the same range of the other ranks' buffers, and rank 0 collects
the other ranges with one batched copy before it unpacks.  The oracle does the same on the
host with the reference's CPU routines; peers are added in ascending rank order on both
sides (the order inside a real collective belongs to the communication library).
"""
import numpy as np
import pytest

from oracle_util import F16, F32, I32, NP_OF, SIZE_OF

pytestmark = pytest.mark.gpu


def _raw(v):
    return v.view(np.uint16) if v.dtype == np.float16 else v


def _values(rng, n, dtype):
    if dtype == I32:
        return rng.integers(-2 ** 31, 2 ** 31, n, dtype=np.int64).astype(np.int32)
    return (rng.standard_normal(n) * 1e-2).astype(NP_OF[dtype])


def _oracle_reduce(orc, buffers, ranges, dtype):
    """buffers: one typed array per rank (prescaled fusion buffers).  Returns rank 0's buffer after
    the reduce-scatter and the gather."""
    out = _raw(buffers[0]).copy()
    for r, (first, count) in enumerate(ranges):
        acc = _raw(buffers[r])[first:first + count].copy()
        for j in range(len(buffers)):
            if j != r:
                acc = orc.sum(_raw(buffers[j])[first:first + count], acc, dtype)
        out[first:first + count] = acc
    return out


def _device_reduce(gpu, bufs, ranges, dtype, es):
    """The same on the device; bufs are the ranks' device buffers (uint8 tensors)."""
    for r, (first, count) in enumerate(ranges):
        peers = [b.data_ptr() + first * es for j, b in enumerate(bufs) if j != r]
        if peers and count:
            gpu.H.reduce_sum_k(bufs[r].data_ptr() + first * es, peers, count, dtype, gpu.stream)
    # the gather, as far as rank 0 sees it: the other ranks' ranges arrive in its buffer
    moves = [(bufs[0].data_ptr() + f * es, bufs[r].data_ptr() + f * es, c * es)
             for r, (f, c) in enumerate(ranges) if r != 0 and c]
    if moves:
        gpu.H.batched_d2d_memcpy([m[0] for m in moves], [m[1] for m in moves], [m[2] for m in moves], gpu.stream)


@pytest.mark.parametrize("dtype", [F32, F16, I32])
@pytest.mark.parametrize("world", [2, 4, 8])
def test_fused_response_every_rank_reduces_its_share(gpu, orc, dtype, world):
    from horovod_amd import workloads as W
    rng = np.random.default_rng(100 + world)
    np_t, es = NP_OF[dtype], SIZE_OF[dtype]
    counts = [1, 777, 4096, 33, 250001, 5, 64 * 1024 + 3, 12]
    pre, post = (0.125, 3.0) if dtype != I32 else (1.0, 1.0)
    tensors = [[_values(rng, c, dtype) for c in counts] for _ in range(world)]
    d_t = [[gpu.upload(t) for t in rank] for rank in tensors]
    outs = [gpu.empty(c * es, fill=0x77) for c in counts]
    plans = [gpu.H.FusionPlan([t.data_ptr() for t in d_t[r]], [o.data_ptr() for o in outs], counts, dtype)
             for r in range(world)]
    try:
        blen = plans[0].buffer_len
        ranges = W.reduce_scatter_ranges(blen // es, world, fused=True)
        grown = ranges[-1][0] + ranges[-1][1]
        assert grown * es >= blen
        # the reference's fusion buffer is larger than any response; the dummy elements behind the
        # payload take part in the sums and are never unpacked
        bufs = [gpu.empty(grown * es + 64, fill=0) for _ in range(world)]
        for r in range(world):
            plans[r].pack(bufs[r].data_ptr(), pre, gpu.stream)
        _device_reduce(gpu, bufs, ranges, dtype, es)
        plans[0].unpack(bufs[0].data_ptr(), post, gpu.stream)
        got = [gpu.download(o, np.uint8) for o in outs]
        tail = gpu.download(bufs[0], np.uint8)[grown * es:]
        assert not tail.any(), "wrote behind the grown buffer"

        host = []
        for r in range(world):
            img, n = orc.pack([_raw(t) for t in tensors[r]], padded=True)
            assert n == blen
            buf = np.zeros(grown, np_t)
            buf.view(np.uint8)[:n] = img[:n]
            host.append(orc.scale_buffer(_raw(buf), pre, dtype).view(np_t) if pre != 1.0 else buf)
        red = _oracle_reduce(orc, host, ranges, dtype)
        red = orc.scale_buffer(red, post, dtype) if post != 1.0 else red
        want = [np.empty(c, _raw(np.empty(0, np_t)).dtype) for c in counts]
        orc.unpack(red.view(np.uint8), want, padded=True)
        for i in range(len(counts)):
            assert np.array_equal(got[i], want[i].view(np.uint8)), "tensor %d" % i

        if dtype == I32:
            # wrapping sums do not depend on the order: the shares together are the whole allreduce
            whole = _raw(host[0]).copy()
            for j in range(1, world):
                whole = orc.sum(_raw(host[j]), whole, dtype)
            assert np.array_equal(red, whole)
    finally:
        for p in plans:
            p.destroy()


@pytest.mark.parametrize("dtype", [F32, F16])
@pytest.mark.parametrize("n", [1003, 7, 8, 2 ** 20 + 5])
def test_single_tensor_last_rank_takes_the_rest(gpu, orc, dtype, n):
    """An unfused response is not grown (ops/nccl_operations.cc:262-270,289): n % local_size elements
    remain behind the shares and the last rank reduces them along with its own share."""
    from horovod_amd import workloads as W
    world = 8
    rng = np.random.default_rng(n)
    np_t, es = NP_OF[dtype], SIZE_OF[dtype]
    ranges = W.reduce_scatter_ranges(n, world, fused=False)
    assert sum(c for _, c in ranges) == n and ranges[-1][1] == n // world + n % world
    tensors = [_values(rng, n, dtype) for _ in range(world)]
    d_t = [gpu.upload(t) for t in tensors]
    outs = [gpu.empty(n * es + 16, fill=0x55) for _ in range(world)]
    for r in range(world):  # prescale, out of place into the output, which then serves as the buffer
        gpu.H.scale_buffer(d_t[r].data_ptr(), outs[r].data_ptr(), n, 0.125, dtype, gpu.stream)
    _device_reduce(gpu, outs, ranges, dtype, es)
    gpu.H.scale_buffer(outs[0].data_ptr(), outs[0].data_ptr(), n, 0.5, dtype, gpu.stream)
    got = gpu.download(outs[0], np.uint8)
    assert np.all(got[n * es:] == 0x55)
    host = [orc.scale_buffer(_raw(t), 0.125, dtype) for t in tensors]
    want = orc.scale_buffer(_oracle_reduce(orc, host, ranges, dtype), 0.5, dtype)
    assert np.array_equal(got[:n * es], want.view(np.uint8))
