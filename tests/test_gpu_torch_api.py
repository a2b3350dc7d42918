"""The allreduce surface of horovod.torch in front of the HIP path.

The first half restates the reference's own tests (test/parallel/test_torch.py:152-445,
607-705 and 1340-1400) for a simulated world: same inputs (integers in [-100, 100) in 17,
17x17 and 17x17x17 tensors, every rank holding the same values), same expectations.  The
second half gives every rank its own values and checks against the CPU oracle."""
import itertools
import warnings

import numpy as np
import pytest
import torch

from oracle_util import F16, F32, F64

pytestmark = pytest.mark.gpu

DTYPES = [torch.int32, torch.int64, torch.float32, torch.float64, torch.float16]
INT_TYPES = [torch.int32, torch.int64]
DIMS = [1, 2, 3]


@pytest.fixture()
def hvd(gpu):
    import horovod_amd.torch as hvd
    yield hvd
    hvd.shutdown()
    gpu.H.set_fp16_scale_mode(gpu.H.FP16_SCALE_FP32_FACTOR)


def _tensor(dtype, dim, seed=1234):
    torch.manual_seed(seed)
    return torch.FloatTensor(*([17] * dim)).random_(-100, 100).cuda().type(dtype)


@pytest.mark.parametrize("size", [1, 2, 3, 8])
def test_horovod_allreduce(hvd, size):
    """test_torch.py:152-183: the sum over ranks holding equal tensors is tensor * size."""
    hvd.init(size=size)
    for dtype, dim in itertools.product(DTYPES, DIMS):
        tensor = _tensor(dtype, dim)
        summed = hvd.allreduce(tensor, average=False)
        assert torch.equal(summed, tensor * size), (dtype, dim)
        assert summed.data_ptr() != tensor.data_ptr()


@pytest.mark.parametrize("size", [1, 2, 4])
def test_horovod_allreduce_average(hvd, size):
    """test_torch.py:185-216: Average gives the tensor back (exactly, for a power-of-two size)."""
    hvd.init(size=size)
    for dtype, dim in itertools.product(DTYPES, DIMS):
        tensor = _tensor(dtype, dim)
        averaged = hvd.allreduce(tensor, average=True)
        assert torch.equal(averaged, tensor), (dtype, dim)
        assert torch.equal(hvd.allreduce(tensor), tensor)  # Average is the default op
        assert torch.equal(hvd.allreduce(tensor, op=hvd.Average), tensor)


def test_horovod_allreduce_average_three_ranks_within_threshold(hvd):
    hvd.init(size=3)
    for dtype in (torch.float32, torch.float64, torch.float16):
        tensor = _tensor(dtype, 2)
        assert torch.allclose(hvd.allreduce(tensor, average=True), tensor, 1e-3 if dtype == torch.float16 else 1e-6)


@pytest.mark.parametrize("size", [1, 2])
def test_horovod_allreduce_inplace_and_async_fused(hvd, size):
    """test_torch.py:218-297: in place; many requests in flight are fused into few responses."""
    hvd.init(size=size)
    for dtype, dim in itertools.product(DTYPES, DIMS):
        tensor = _tensor(dtype, dim)
        want = tensor * size
        hvd.allreduce_(tensor, average=False)
        assert torch.equal(tensor, want)
    import horovod_amd.torch.mpi_ops as ops
    before = ops._engine.responses
    tests = []
    for dtype, dim in itertools.product(DTYPES, DIMS):
        tensor = _tensor(dtype, dim)
        tests.append((tensor * size, hvd.allreduce_async(tensor, average=False)))
    polled = [hvd.poll(h) for _, h in tests]
    assert all(isinstance(p, bool) for p in polled)
    for want, handle in tests:
        assert torch.equal(hvd.synchronize(handle), want)
    # 15 requests of 5 dtypes: one fused response per dtype
    assert ops._engine.responses - before == len(DTYPES)


def _expected_scaled(tensor, factor, dtype, half_factor_mode):
    """The expectation of test_torch.py:363-375 / :418-431: integers scale in float64; device
    half tensors in half arithmetic with the factor rounded to half, host half tensors in
    float32 with the float32 factor."""
    if dtype in INT_TYPES:
        return (torch.tensor(factor, dtype=torch.float64) * tensor.cpu().type(torch.float64))
    if dtype == torch.float16 and not half_factor_mode:
        return torch.tensor(factor, dtype=torch.float32) * tensor.cpu().type(torch.float32)
    return torch.tensor(factor, dtype=torch.float64).type(dtype) * tensor.cpu()


@pytest.mark.parametrize("half_factor_mode", [False, True])
@pytest.mark.parametrize("size", [1, 2])
def test_horovod_allreduce_prescale(hvd, gpu, size, half_factor_mode):
    """test_torch.py:339-388."""
    hvd.init(size=size)
    if half_factor_mode:
        gpu.H.set_fp16_scale_mode(gpu.H.FP16_SCALE_HALF_FACTOR)
    for dtype, dim in itertools.product(DTYPES, DIMS):
        np.random.seed(1234)
        factor = np.random.uniform()
        tensor = _tensor(dtype, dim)
        summed = hvd.allreduce(tensor, average=False, prescale_factor=factor)
        multiplied = _expected_scaled(tensor, factor, dtype, half_factor_mode).type(dtype) * size
        assert torch.equal(summed.cpu(), multiplied), (dtype, dim)


@pytest.mark.parametrize("size", [2, 4])
def test_inplace_allreduce_with_prescale_on_a_single_tensor(hvd, size):
    """An in-place request travels alone (no fusion buffer): the other ranks' buffers are made from
    the same tensor and must see it before rank 0 scales it in place."""
    hvd.init(size=size)
    torch.manual_seed(7)
    base = torch.FloatTensor(17, 17).random_(-100, 100).cuda()
    for fn in ("allreduce_", "allreduce_async_"):
        t = base.clone()
        r = getattr(hvd, fn)(t, op=hvd.Sum, prescale_factor=0.5)
        if fn.endswith("async_"):
            r = hvd.synchronize(r)
        assert r.data_ptr() == t.data_ptr()
        assert torch.equal(t.cpu(), (base * 0.5 * size).cpu()), fn


@pytest.mark.parametrize("half_factor_mode", [False, True])
@pytest.mark.parametrize("size", [1, 2])
def test_horovod_allreduce_postscale(hvd, gpu, size, half_factor_mode):
    """test_torch.py:390-445."""
    hvd.init(size=size)
    if half_factor_mode:
        gpu.H.set_fp16_scale_mode(gpu.H.FP16_SCALE_HALF_FACTOR)
    for dtype, dim in itertools.product(DTYPES, DIMS):
        np.random.seed(1234)
        factor = np.random.uniform()
        tensor = _tensor(dtype, dim)
        summed = hvd.allreduce(tensor, average=False, postscale_factor=factor)
        multiplied = _expected_scaled(tensor * size, factor, dtype, half_factor_mode).type(dtype)
        assert torch.equal(summed.cpu(), multiplied), (dtype, dim)


@pytest.mark.parametrize("size", [1, 2, 4])
def test_horovod_grouped_allreduce(hvd, size):
    """test_torch.py:607-705: sum, average and in place, five tensors per group."""
    hvd.init(size=size)
    import horovod_amd.torch.mpi_ops as ops
    for dtype, dim in itertools.product(DTYPES, DIMS):
        torch.manual_seed(1234)
        tensors = [torch.FloatTensor(*([17] * dim)).random_(-100, 100).cuda().type(dtype) for _ in range(5)]
        before = ops._engine.responses
        summed = hvd.grouped_allreduce(tensors, average=False)
        assert ops._engine.responses - before == 1  # the group travels as one fused response
        assert all(torch.equal(s, t * size) for s, t in zip(summed, tensors))
        averaged = hvd.grouped_allreduce(tensors, average=True)
        assert all(torch.equal(a, t) for a, t in zip(averaged, tensors))
        want = [t * size for t in tensors]
        hvd.grouped_allreduce_(tensors, average=False)
        assert all(torch.equal(t, w) for t, w in zip(tensors, want))


def test_horovod_allreduce_grad(hvd):
    """test_torch.py:547-605: the gradient of a sum over ranks is ones * size; of an average, ones."""
    hvd.init(size=4)
    for dtype, dim in itertools.product([torch.float32, torch.float64, torch.float16], DIMS):
        tensor = _tensor(dtype, dim)
        tensor.requires_grad_()
        summed = hvd.allreduce(tensor, average=False)
        summed.backward(torch.ones([17] * dim, device="cuda", dtype=dtype))
        assert torch.equal(tensor.grad, torch.ones([17] * dim, device="cuda", dtype=dtype) * 4)
        tensor.grad = None
        hvd.allreduce(tensor, average=True).backward(torch.ones([17] * dim, device="cuda", dtype=dtype))
        assert torch.equal(tensor.grad, torch.ones([17] * dim, device="cuda", dtype=dtype))


def test_errors_of_the_front_end(hvd):
    with pytest.raises(ValueError, match="not been initialized"):
        hvd.size()
    hvd.init(size=2)
    t = torch.ones(8, device="cuda")
    with pytest.raises(ValueError, match="supersedes average"):
        hvd.allreduce(t, average=True, op=hvd.Sum)
    with pytest.raises(ValueError, match="contiguous"):
        hvd.allreduce_async_(torch.ones(4, 4, device="cuda").t())
    with pytest.raises(ValueError, match="not supported"):
        hvd.allreduce_async_(torch.ones(4))
    with pytest.raises(ValueError, match="not supported"):
        hvd.allreduce_async_(torch.ones(4, device="cuda", dtype=torch.complex64))
    # test_torch.py:1340-1370: one name, two requests in flight
    h = hvd.allreduce_async(t, name="duplicate_name")
    with pytest.raises(hvd.HorovodInternalError, match="same name"):
        hvd.allreduce_async(t, name="duplicate_name")
    hvd.synchronize(h)
    hvd.synchronize(hvd.allreduce_async(t, name="duplicate_name"))  # free again once synchronised
    with pytest.raises(ValueError, match="Adasum"):
        hvd.allreduce(torch.ones(4, device="cuda", dtype=torch.int32), op=hvd.Adasum)
    with pytest.raises(ValueError, match="handle"):
        hvd.poll(12345)
    with warnings.catch_warnings(record=True) as w:
        warnings.simplefilter("always")
        hvd.allreduce(t, average=False)
    assert any(issubclass(x.category, DeprecationWarning) for x in w)
    hvd.shutdown()
    hvd.init(size=6, local_size=2)
    with pytest.raises(NotImplementedError, match="power of 2"):
        hvd.allreduce(t, op=hvd.Adasum)


# ---- every rank with values of its own, against the oracle --------------------------

def _peer_values(rank, name, tensor):
    g = torch.Generator(device="cuda")
    g.manual_seed(1000 * rank + sum(name.encode()) % 997)
    if tensor.dtype.is_floating_point:
        return torch.randn(tensor.shape, generator=g, device="cuda", dtype=torch.float32).type(tensor.dtype)
    return torch.randint(-1000, 1000, tensor.shape, generator=g, device="cuda").type(tensor.dtype)


def _np(t):
    t = t.detach().cpu()
    return t.view(torch.int16).numpy().view(np.uint16) if t.dtype == torch.float16 else t.numpy()


@pytest.mark.parametrize("dtype,code", [(torch.float32, F32), (torch.float16, F16), (torch.float64, F64)])
def test_sum_of_distinct_ranks_with_both_scale_factors(hvd, orc, dtype, code):
    size = 8
    hvd.init(size=size, peer_source=_peer_values)
    torch.manual_seed(7)
    shapes = [(5,), (300, 7), (1,), (64, 64, 3), (17,)]
    tensors = [torch.randn(s, device="cuda").type(dtype) for s in shapes]
    names = ["grad.%d" % i for i in range(len(tensors))]
    pre, post = 0.125, 1.0 / 3.0
    handles = [hvd.allreduce_async(t, op=hvd.Sum, name=n, prescale_factor=pre, postscale_factor=post)
               for t, n in zip(tensors, names)]
    outs = [hvd.synchronize(h) for h in handles]
    for t, n, out in zip(tensors, names, outs):
        acc = orc.scale_buffer(_np(t).reshape(-1), pre, code)
        for rank in range(1, size):
            peer = orc.scale_buffer(_np(_peer_values(rank, "allreduce." + n, t)).reshape(-1), pre, code)
            acc = orc.sum(peer, acc, code)
        want = orc.scale_buffer(acc, post, code)
        assert np.array_equal(_np(out).reshape(-1).view(np.uint8), want.view(np.uint8)), n


def test_fp16_compression_rides_on_pack_and_unpack(hvd, orc):
    """hvd.allreduce(..., compression=hvd.Compression.fp16) on float32: the reference casts,
    scales and sums in half and casts back (compression.py:46-64); here the two casts happen
    in the pack and unpack kernels with the same roundings and no half tensor exists."""
    size = 4
    hvd.init(size=size, peer_source=_peer_values)
    torch.manual_seed(9)
    tensors = [torch.randn(s, device="cuda") * 1e-3 for s in [(1000,), (33, 5), (1,)]]
    outs = hvd.grouped_allreduce(tensors, op=hvd.Average, name="g", compression=hvd.Compression.fp16,
                                 prescale_factor=0.5, postscale_factor=2.0)
    for i, (t, out) in enumerate(zip(tensors, outs)):
        assert out.dtype == torch.float32
        name = "grouped_allreduce.g_%dof%d" % (i + 1, len(tensors))
        acc = orc.scale_cast_f32_to_f16(_np(t).reshape(-1), 0.5, cast_first=True)
        for rank in range(1, size):
            peer = orc.scale_cast_f32_to_f16(_np(_peer_values(rank, name, t)).reshape(-1), 0.5, cast_first=True)
            acc = orc.float16_sum(peer, acc)
        want = orc.scale_cast_f16_to_f32(acc, 2.0 / size)
        assert np.array_equal(_np(out).reshape(-1).view(np.uint32), want.view(np.uint32))
    # the unfused route through the compressor's own casts gives the same values
    for t, out in zip(tensors, outs):
        h, ctx = hvd.Compression.fp16.compress(t)
        assert h.dtype == torch.float16 and hvd.Compression.fp16.decompress(h, ctx).dtype == torch.float32


@pytest.mark.parametrize("size,local_size", [(2, 1), (4, 1), (4, 2)])
@pytest.mark.parametrize("dtype,code", [(torch.float32, F32), (torch.float16, F16)])
def test_adasum_tree_matches_pairwise_oracle(hvd, orc, size, local_size, dtype, code):
    hvd.init(size=size, local_size=local_size, peer_source=_peer_values)
    torch.manual_seed(11)
    tensors = [torch.randn(s, device="cuda").type(dtype) for s in [(4099,), (7, 3), (20000,)]]
    outs = hvd.grouped_allreduce(tensors, op=hvd.Adasum, name="a")
    for i, (t, out) in enumerate(zip(tensors, outs)):
        name = "grouped_allreduce.a_%dof%d" % (i + 1, len(tensors))
        ranks = [_np(t).reshape(-1)] + [_np(_peer_values(r, name, t)).reshape(-1) for r in range(1, size)]
        nodes = []
        for node in range(size // local_size):
            acc = ranks[node * local_size]
            for r in ranks[node * local_size + 1:(node + 1) * local_size]:
                acc = orc.sum(r, acc, code)
            nodes.append(acc)
        d = 1
        while d < len(nodes):
            for j in range(0, len(nodes), 2 * d):
                nodes[j] = orc.adasum_pairwise(nodes[j], nodes[j + d], [t.numel()], code)[0]
            d *= 2
        want = orc.scale_buffer(nodes[0], 1.0 / local_size, code) if local_size > 1 else nodes[0]
        got = _np(out).reshape(-1)
        if dtype == torch.float16:
            assert np.array_equal(got, want)
        else:
            ulp = np.abs(got.view(np.int32).astype(np.int64) - want.view(np.int32).astype(np.int64))
            assert ulp.max() <= 2 * (size // local_size - 1), ulp.max()  # <= 1 ulp per level that feeds the next


def test_requests_with_mixed_dtypes_and_factors_fuse_by_class(hvd):
    hvd.init(size=2)
    import horovod_amd.torch.mpi_ops as ops
    a = [torch.ones(100, device="cuda") * i for i in range(4)]
    b = [torch.ones(50, device="cuda", dtype=torch.float16) * i for i in range(3)]
    handles = []
    for i in range(4):
        handles.append(hvd.allreduce_async(a[i], op=hvd.Sum))
        if i < 3:
            handles.append(hvd.allreduce_async(b[i], op=hvd.Sum))
    handles.append(hvd.allreduce_async(a[1], op=hvd.Sum, prescale_factor=0.5))
    before = ops._engine.responses
    outs = [hvd.synchronize(h) for h in handles]
    assert ops._engine.responses - before == 3  # fp32, fp16, and fp32 with another prescale
    assert torch.equal(outs[2], a[1] * 2) and torch.equal(outs[3], b[1] * 2) and torch.equal(outs[-1], a[1])


def test_small_fusion_threshold_splits_responses_and_two_streams_alternate(hvd):
    hvd.init(size=2, fusion_threshold=4096, num_streams=2)
    import horovod_amd.torch.mpi_ops as ops
    ts = [torch.full((600,), float(i), device="cuda") for i in range(6)]  # 2,400 bytes each: one per response
    hs = [hvd.allreduce_async(t, op=hvd.Sum) for t in ts]
    outs = [hvd.synchronize(h) for h in hs]
    assert ops._engine.responses == 6
    for i, o in enumerate(outs):
        assert torch.equal(o, ts[i] * 2)


_FUZZ_TYPES = [(torch.uint8, 0), (torch.int8, 1), (torch.int32, 4), (torch.int64, 5), (torch.float16, 6),
               (torch.float32, 7), (torch.float64, 8)]


def _fuzz_values(gen, n, dtype, rank):
    if dtype.is_floating_point:
        return (torch.randn(n, generator=gen, device="cuda") * 3).type(dtype)
    hi = 6 if dtype in (torch.uint8, torch.int8) else 1000
    lo = 0 if dtype == torch.uint8 else -hi
    return torch.randint(lo, hi, (n,), generator=gen, device="cuda").type(dtype)


@pytest.mark.parametrize("seed", range(12))
def test_fuzz_against_the_oracle(hvd, orc, seed):
    """Random worlds, dtypes, sizes (zero included), element-aligned-only addresses, factors,
    ops, in place and out of place, all in flight together: every output equals
    postscale * (sum over ranks in rank order of prescale * x_rank) as the oracle computes it."""
    rng = np.random.default_rng(100 + seed)
    size = int(rng.choice([1, 2, 3, 5, 8]))
    store = {}

    def peer_source(rank, name, tensor):
        return store[name][rank]

    hvd.init(size=size, peer_source=peer_source, fusion_threshold=int(rng.choice([1 << 12, 1 << 16, 64 << 20])),
             num_streams=int(rng.choice([1, 2])))
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    factors = [1.0, 0.5, 0.125, 1.0 / 3.0, 2.5]
    jobs = []
    for i in range(int(rng.integers(1, 14))):
        dtype, code = _FUZZ_TYPES[int(rng.integers(0, len(_FUZZ_TYPES)))]
        n = int(rng.choice([0, 1, 3, 17, 255, 1024, 1025, 4099, 20000]))
        shift = int(rng.integers(0, 4))
        ranks = []
        for r in range(size):
            base = _fuzz_values(gen, n + 4, dtype, r)
            ranks.append(base[shift:shift + n])
        name = "fuzz.%d" % i
        store["allreduce." + name] = ranks
        average = bool(rng.integers(0, 2)) and dtype.is_floating_point
        pre = float(rng.choice(factors))
        post = float(rng.choice(factors))
        if not dtype.is_floating_point and dtype != torch.int64 and dtype != torch.int32:
            pre = post = 1.0 if rng.integers(0, 2) else 0.5  # keep 8-bit results inside the type
        inplace = bool(rng.integers(0, 2))
        want = orc.scale_buffer(_np(ranks[0]), pre, code) if n else _np(ranks[0])
        for r in range(1, size):
            if n:
                want = orc.sum(orc.scale_buffer(_np(ranks[r]), pre, code), want, code)
        if n:
            want = orc.scale_buffer(want, post / size if average else post, code)
        op = hvd.Average if average else hvd.Sum
        fn = hvd.allreduce_async_ if inplace else hvd.allreduce_async
        handle = fn(ranks[0], name=name, op=op, prescale_factor=pre, postscale_factor=post)
        jobs.append((name, handle, want, n))
    for name, handle, want, n in jobs:
        out = hvd.synchronize(handle)
        assert out.numel() == n
        if n:
            assert np.array_equal(_np(out).reshape(-1).view(np.uint8), np.ascontiguousarray(want).view(np.uint8)), name


def test_adasum_responses_on_alternating_streams_do_not_share_state(hvd, orc):
    """Equal-shaped Adasum responses of one cycle run on different streams at the same time;
    each stream slot keeps Adasum partial sums of its own."""
    hvd.init(size=2, peer_source=_peer_values, fusion_threshold=1 << 20, num_streams=2)
    torch.manual_seed(21)
    tensors = [torch.randn(200000, device="cuda") for _ in range(6)]  # 800 KB each: one response per tensor
    names = ["t%d" % i for i in range(6)]
    handles = [hvd.allreduce_async(t, name=n, op=hvd.Adasum) for t, n in zip(tensors, names)]
    outs = [hvd.synchronize(h) for h in handles]
    import horovod_amd.torch.mpi_ops as ops
    assert ops._engine.responses == 6
    for t, n, out in zip(tensors, names, outs):
        peer = _np(_peer_values(1, "allreduce." + n, t))
        want = orc.adasum_pairwise(_np(t), peer, [t.numel()], F32)[0]
        ulp = np.abs(_np(out).view(np.int32).astype(np.int64) - want.view(np.int32).astype(np.int64))
        assert ulp.max() <= 1, n


def _adasum_reference_operation(a, b):
    """test/parallel/test_adasum_tensorflow.py:28-43, in float64."""
    anormsq, bnormsq = np.inner(a.ravel(), a.ravel()), np.inner(b.ravel(), b.ravel())
    dot = np.dot(a.ravel(), b.ravel())
    acoeff = 1.0 - dot / anormsq * 0.5 if anormsq != 0 else 1.0
    bcoeff = 1.0 - dot / bnormsq * 0.5 if bnormsq != 0 else 1.0
    return acoeff * a + bcoeff * b


def _reference_tree_reduction(tensors):
    """test_adasum_tensorflow.py:48-59: neighbours first, then the pairs' results."""
    level = list(tensors)
    while len(level) > 1:
        level = [_adasum_reference_operation(level[2 * i], level[2 * i + 1]) for i in range(len(level) // 2)]
    return level[0]


@pytest.mark.parametrize("size,local_size", [(2, 1), (4, 1), (8, 1), (8, 2), (4, 4)])
def test_adasum_against_the_reference_tests_numpy_tree(hvd, size, local_size):
    """test_adasum_tensorflow.py:103-176 (CPU and GPU-NCCL variants): two 2x2 tensors of uniform
    [0, 1) values per rank, each reduced on its own; expected = the numpy tree over the nodes'
    sums, divided by local_size; fp16, fp32 and fp64, compared with the tolerances of
    assertAllCloseAccordingToType (1e-3 for half, 1e-6 otherwise)."""
    rng = np.random.default_rng(17)
    rank_tensors = [[rng.random((2, 2)), rng.random((2, 2))] for _ in range(size)]
    table = {}

    def peer(rank, name, tensor):
        return table[(rank, name)]

    hvd.init(size=size, local_size=local_size, peer_source=peer)
    nodes = size // local_size
    for dtype, tol in [(torch.float16, 1e-3), (torch.float32, 1e-6), (torch.float64, 1e-6)]:
        for which in range(2):
            name = "ref.%s.%d" % (str(dtype).split(".")[1], which)
            cast = [torch.from_numpy(rank_tensors[r][which]).cuda().type(dtype) for r in range(size)]
            for r in range(1, size):
                table[(r, "allreduce." + name)] = cast[r]
            got = hvd.allreduce(cast[0], op=hvd.Adasum, name=name)
            # the expectation starts from the values as cast, like the tensors the ranks pass
            held = [c.double().cpu().numpy() for c in cast]
            sums = [sum(held[n * local_size:(n + 1) * local_size]) for n in range(nodes)]
            want = _reference_tree_reduction(sums) / local_size
            assert got.dtype == dtype
            assert np.allclose(got.double().cpu().numpy(), want, rtol=tol, atol=tol), (dtype, size, local_size)


def test_broadcast_in_the_simulated_world(hvd):
    """What a training script does before its first step (broadcast_parameters,
    broadcast_optimizer_state from rank 0) is the identity here; another root's value comes from
    peer_source."""
    def peer(rank, name, tensor):
        return torch.full_like(tensor, float(rank))

    hvd.init(size=4, peer_source=peer)
    model = torch.nn.Linear(3, 2).cuda()
    before = {k: v.clone() for k, v in model.state_dict().items()}
    hvd.broadcast_parameters(model.state_dict(), root_rank=0)
    hvd.broadcast_parameters(list(model.named_parameters()), root_rank=0)
    opt = torch.optim.SGD(model.parameters(), lr=0.1, momentum=0.9)
    hvd.broadcast_optimizer_state(opt, root_rank=0)
    assert hvd.broadcast_object({"epoch": 3}, root_rank=0) == {"epoch": 3}
    for k, v in model.state_dict().items():
        assert torch.equal(v, before[k])
    t = torch.zeros(5, device="cuda")
    out = hvd.broadcast(t, root_rank=2, name="b")
    assert torch.equal(out, torch.full_like(t, 2.0)) and torch.equal(t, torch.zeros_like(t))
    h = hvd.broadcast_async_(t, root_rank=3, name="c")
    assert hvd.poll(h) and hvd.synchronize(h) is t and torch.equal(t, torch.full_like(t, 3.0))
    with pytest.raises(ValueError, match="root rank"):
        hvd.broadcast_(t, root_rank=4)
    with pytest.raises(NotImplementedError):
        hvd.broadcast_optimizer_state(opt, root_rank=1)
