"""hvd.allgather in front of the batched fusion-buffer copies: the reference's own allgather tests
(test/parallel/test_torch.py:780-1000) restated for a simulated world in which rank r holds a
tensor filled with r, plus byte-for-byte checks with random contents."""
import itertools

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DTYPES = [torch.uint8, torch.int8, torch.int16, torch.int32, torch.int64, torch.float32, torch.float64,
          torch.float16]
SIZES = [17, 32, 81, 12, 15, 23, 22]


@pytest.fixture()
def hvd(gpu):
    import horovod_amd.torch as hvd
    yield hvd
    hvd.shutdown()


def _filled_like_rank(sizes=None):
    def source(rank, name, tensor):
        rows = tensor.shape[0] if sizes is None else sizes[rank]
        return torch.ones((rows,) + tuple(tensor.shape[1:]), device="cuda").mul_(rank).type(tensor.dtype)
    return source


@pytest.mark.parametrize("size", [1, 2, 5])
def test_horovod_allgather(hvd, size):
    """test_torch.py:780-808."""
    hvd.init(size=size, peer_source=_filled_like_rank())
    for dtype, dim in itertools.product(DTYPES, [1, 2, 3]):
        tensor = torch.zeros([17] * dim, device="cuda").type(dtype)  # this process is rank 0
        gathered = hvd.allgather(tensor)
        assert list(gathered.shape) == [17 * size] + [17] * (dim - 1)
        assert gathered.dtype == dtype
        for i in range(size):
            rank_tensor = gathered[i * 17:(i + 1) * 17].float()
            assert rank_tensor.min() == i and rank_tensor.max() == i


@pytest.mark.parametrize("size", [2, 7])
def test_horovod_allgather_variable_size(hvd, size):
    """test_torch.py:810-849: first dimensions differ between ranks."""
    sizes = SIZES[:size]
    hvd.init(size=size, peer_source=_filled_like_rank(sizes))
    for dtype, dim in itertools.product(DTYPES, [1, 2, 3]):
        tensor = torch.zeros([sizes[0]] + [17] * (dim - 1), device="cuda").type(dtype)
        gathered = hvd.allgather(tensor)
        assert list(gathered.shape) == [sum(sizes)] + [17] * (dim - 1)
        for i in range(size):
            rank_tensor = gathered[sum(sizes[:i]):sum(sizes[:i + 1])].float()
            assert list(rank_tensor.shape) == [sizes[i]] + [17] * (dim - 1)
            assert rank_tensor.min() == i and rank_tensor.max() == i


def test_horovod_allgather_async_fused(hvd):
    """test_torch.py:851-890: many requests in flight travel as few fused responses, one per dtype."""
    size = 3
    hvd.init(size=size, peer_source=_filled_like_rank())
    import horovod_amd.torch.mpi_ops as ops
    tests = []
    for dtype, dim in itertools.product(DTYPES, [1, 2, 3]):
        tensor = torch.zeros([17] * dim, device="cuda").type(dtype)
        tests.append((hvd.allgather_async(tensor), [17] * dim))
    before = ops._engine.responses
    assert all(isinstance(hvd.poll(h), bool) for h, _ in tests)
    for handle, shape in tests:
        gathered = hvd.synchronize(handle)
        for i in range(size):
            rank_tensor = gathered[i * 17:(i + 1) * 17].float()
            assert list(rank_tensor.shape) == shape
            assert rank_tensor.min() == i and rank_tensor.max() == i
    assert ops._engine.responses - before == len(DTYPES)


def test_horovod_allgather_grad(hvd):
    """test_torch.py:957-995: the gradient is this rank's rows of the averaged upstream gradient."""
    size = 4
    sizes = [3, 2, 7, 4]
    hvd.init(size=size, peer_source=_filled_like_rank(sizes))
    for dtype, dim in itertools.product([torch.float32, torch.float64, torch.float16], [1, 2, 3]):
        tensor = torch.zeros([sizes[0]] + [17] * (dim - 1), device="cuda").type(dtype)
        tensor.requires_grad_()
        grad_ys = torch.cat([torch.ones([s] + [17] * (dim - 1), device="cuda").type(dtype) * r
                             for r, s in enumerate(sizes)], dim=0)
        gathered = hvd.allgather(tensor)
        # every rank feeds the same upstream gradient, so their average is that gradient
        hvd.shutdown()
        hvd.init(size=size)
        gathered.backward(grad_ys)
        expected = np.zeros([sizes[0]] + [17] * (dim - 1))  # rank 0's rows of grad_ys are 0
        assert np.linalg.norm(expected - tensor.grad.float().cpu().numpy()) < 1e-8
        hvd.shutdown()
        hvd.init(size=size, peer_source=_filled_like_rank(sizes))


def test_allgather_bytes_with_random_contents_and_mixed_requests(hvd):
    """Random values, ragged first dimensions (a rank may contribute nothing), element-aligned-only
    addresses, allgathers and allreduces queued together: every output is the concatenation."""
    size = 4
    store = {}

    def source(rank, name, tensor):
        return store[name][rank]

    hvd.init(size=size, peer_source=source, fusion_threshold=1 << 16)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(5)
    rng = np.random.default_rng(5)
    jobs = []
    for i in range(12):
        dtype = DTYPES[int(rng.integers(0, len(DTYPES)))]
        rest = tuple(int(x) for x in rng.integers(1, 6, int(rng.integers(0, 3))))
        parts = []
        for r in range(size):
            rows = int(rng.choice([0, 1, 3, 40, 300]))
            if r == 0:
                rows = max(rows, 1)
            n = rows * int(np.prod(rest)) if rest else rows
            base = (torch.randn(n + 3, generator=gen, device="cuda") * 50).type(dtype)
            shift = int(rng.integers(0, 3))
            parts.append(base[shift:shift + n].view((rows,) + rest))
        name = "ag.%d" % i
        store["allgather." + name] = parts
        jobs.append((hvd.allgather_async(parts[0], name=name), torch.cat(parts, dim=0)))
        if i % 3 == 0:
            t = torch.ones(100, device="cuda") * i
            store["allreduce.mix.%d" % i] = [t] * size
            jobs.append((hvd.allreduce_async(t, name="mix.%d" % i, op=hvd.Sum), t * size))
    for handle, want in jobs:
        got = hvd.synchronize(handle)
        assert got.shape == want.shape and got.dtype == want.dtype
        assert torch.equal(got.view(torch.uint8) if got.numel() else got, want.view(torch.uint8) if want.numel() else want)


def test_allgather_errors(hvd):
    hvd.init(size=2, peer_source=lambda rank, name, t: torch.zeros(3, 5, device="cuda"))
    with pytest.raises(hvd.HorovodInternalError, match="first dimension"):
        hvd.allgather(torch.zeros(3, 4, device="cuda"))  # test_torch.py:892-911: ranks disagree beyond dim 0
    with pytest.raises(hvd.HorovodInternalError, match="rank-zero"):
        hvd.allgather(torch.tensor(1.0, device="cuda"))
    hvd.shutdown()
    hvd.init(size=2)
    t = torch.zeros(4, device="cuda")
    h = hvd.allgather_async(t, name="dup")
    with pytest.raises(hvd.HorovodInternalError, match="same name"):
        hvd.allgather_async(t, name="dup")  # test_torch.py:936-955
    assert hvd.synchronize(h).shape == (8,)
