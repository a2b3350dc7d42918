"""DistributedOptimizer over the HIP path (the caller of horovod/torch/optimizer.py:173-206):
gradients of a small model in a simulated world whose other ranks contribute seeded
gradients; the combined gradient is checked against a float64 restatement."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture()
def hvd(gpu):
    import horovod_amd.torch as hvd
    yield hvd
    hvd.shutdown()


def _peer_grad(rank, name, tensor):
    g = torch.Generator(device="cuda")
    g.manual_seed(31 * rank + len(name))
    return torch.randn(tensor.shape, generator=g, device="cuda", dtype=tensor.dtype) * 0.01


def _model():
    torch.manual_seed(3)
    return torch.nn.Sequential(torch.nn.Linear(20, 30), torch.nn.ReLU(), torch.nn.Linear(30, 5)).cuda()


def _local_grads(model):
    torch.manual_seed(4)
    x = torch.randn(16, 20, device="cuda")
    model.zero_grad()
    model(x).pow(2).sum().backward()
    return {n: p.grad.detach().clone() for n, p in model.named_parameters()}


def _expected(hvd_name, local, size, op_average=True):
    total = local.double()
    for rank in range(1, size):
        total = total + _peer_grad(rank, hvd_name, local).double()
    return total / size if op_average else total


@pytest.mark.parametrize("predivide", [1.0, 2.0])
@pytest.mark.parametrize("groups", [None, 2])
def test_average_of_gradients(hvd, predivide, groups):
    size = 4
    hvd.init(size=size, peer_source=_peer_grad)
    model = _model()
    want = _local_grads(model)
    opt = hvd.DistributedOptimizer(torch.optim.SGD(model.parameters(), lr=0.1),
                                   named_parameters=model.named_parameters(),
                                   gradient_predivide_factor=predivide, groups=groups)
    assert isinstance(opt, torch.optim.SGD)
    model.zero_grad()
    torch.manual_seed(4)
    model(torch.randn(16, 20, device="cuda")).pow(2).sum().backward()
    assert opt._handles, "the hooks enqueued nothing during backward"
    with pytest.raises(AssertionError, match="zero_grad"):
        opt.zero_grad()
    before = {n: p.detach().clone() for n, p in model.named_parameters()}
    opt.synchronize()
    names = list(dict(model.named_parameters()))
    for i, (n, p) in enumerate(model.named_parameters()):
        if groups is None:
            wire_name = "allreduce." + n
            exp = _expected(wire_name, want[n], size)
            assert torch.allclose(p.grad.double(), exp, rtol=1e-5, atol=1e-7), n
        else:
            assert p.grad.shape == want[n].shape and torch.isfinite(p.grad).all()
    with opt.skip_synchronize():
        opt.step()
    for n, p in model.named_parameters():
        assert torch.allclose(p, before[n] - 0.1 * p.grad)
    opt.zero_grad()


def test_grouped_gradients_match_ungrouped_semantics(hvd):
    """With every rank holding equal gradients the grouped and the per-parameter route agree."""
    size = 2
    hvd.init(size=size)
    model = _model()
    want = _local_grads(model)
    opt = hvd.DistributedOptimizer(torch.optim.SGD(model.parameters(), lr=0.1),
                                   named_parameters=model.named_parameters(), groups=[list(model.parameters())[:2]])
    model.zero_grad()
    torch.manual_seed(4)
    model(torch.randn(16, 20, device="cuda")).pow(2).sum().backward()
    opt.step()
    for n, p in model.named_parameters():
        assert torch.equal(p.grad, want[n]), n  # average of equal values, power-of-two size: exact


def test_backward_passes_per_step_and_sum(hvd):
    size = 2
    hvd.init(size=size)
    model = _model()
    g1 = _local_grads(model)
    opt = hvd.DistributedOptimizer(torch.optim.SGD(model.parameters(), lr=0.1),
                                   named_parameters=model.named_parameters(), backward_passes_per_step=2,
                                   op=hvd.Sum)
    model.zero_grad()
    for _ in range(2):
        torch.manual_seed(4)
        model(torch.randn(16, 20, device="cuda")).pow(2).sum().backward()
        if _ == 0:
            assert all(h[0] is None for h in opt._handles.values())  # nothing sent after the first pass
    opt.synchronize()
    for n, p in model.named_parameters():
        assert torch.allclose(p.grad, 2 * size * g1[n], rtol=1e-6), n
    with pytest.warns(UserWarning, match="skip_synchronize"):
        opt.step()


def test_fp16_compression_reduces_in_place_without_half_tensors(hvd):
    size = 2
    hvd.init(size=size)
    model = _model()
    want = _local_grads(model)
    opt = hvd.DistributedOptimizer(torch.optim.SGD(model.parameters(), lr=0.1),
                                   named_parameters=model.named_parameters(), compression=hvd.Compression.fp16)
    model.zero_grad()
    torch.manual_seed(4)
    model(torch.randn(16, 20, device="cuda")).pow(2).sum().backward()
    ptrs = {n: p.grad.data_ptr() for n, p in model.named_parameters()}
    opt.synchronize()
    for n, p in model.named_parameters():
        assert p.grad.dtype == torch.float32 and p.grad.data_ptr() == ptrs[n]
        # equal ranks, power-of-two size: the value is the gradient rounded to half
        assert torch.equal(p.grad, want[n].half().float()), n


def test_argument_checks(hvd):
    hvd.init(size=2)
    model = _model()
    sgd = torch.optim.SGD(model.parameters(), lr=0.1)
    with pytest.raises(ValueError, match="op != Average"):
        hvd.DistributedOptimizer(sgd, gradient_predivide_factor=2.0, op=hvd.Sum)
    with pytest.raises(ValueError, match="unique"):
        hvd.DistributedOptimizer(sgd, named_parameters=[("a", p) for p in model.parameters()])
    with pytest.raises(ValueError, match="not named"):
        hvd.DistributedOptimizer(sgd, named_parameters=list(model.named_parameters())[:1])


def test_adasum_optimizer_combines_deltas(hvd, orc):
    """optimizer.py:333-503: each rank steps locally, the deltas are combined with Adasum and
    added to the value before the step."""
    from oracle_util import F32
    size = 2
    lr = 0.1

    def peer_delta(rank, name, tensor):
        g = torch.Generator(device="cuda")
        g.manual_seed(77 + len(name))
        return torch.randn(tensor.shape, generator=g, device="cuda") * 0.01

    hvd.init(size=size, peer_source=peer_delta)
    model = _model()
    grads = _local_grads(model)
    before = {n: p.detach().clone() for n, p in model.named_parameters()}
    opt = hvd.DistributedOptimizer(torch.optim.SGD(model.parameters(), lr=lr),
                                   named_parameters=model.named_parameters(), op=hvd.Adasum)
    assert isinstance(opt, torch.optim.SGD) and hasattr(opt, "_starting_models")
    model.zero_grad()
    torch.manual_seed(4)
    model(torch.randn(16, 20, device="cuda")).pow(2).sum().backward()
    assert len(opt._handles) == 4
    with pytest.raises(AssertionError, match="not supported"):
        with opt.skip_synchronize():
            pass
    opt.step()
    for n, p in model.named_parameters():
        local = (-lr * grads[n]).cpu().numpy().reshape(-1)
        peer = peer_delta(1, "allreduce." + n, p).cpu().numpy().reshape(-1)
        combined = orc.adasum_pairwise(local, peer, [local.size], F32)[0]
        want = before[n].cpu().numpy().reshape(-1) + combined
        assert np.allclose(p.detach().cpu().numpy().reshape(-1), want, rtol=1e-6, atol=1e-8), n
    opt.zero_grad()


@pytest.mark.parametrize("sparse_as_dense", [False, True])
def test_sparse_gradients_travel_by_allgather(hvd, sparse_as_dense):
    """An embedding with sparse=True: indices and values are allgathered (optimizer.py:215-217,
    mpi_ops.py:515-535), or the gradient is densified first when sparse_as_dense is set."""
    size = 2
    hvd.init(size=size)
    torch.manual_seed(8)
    emb = torch.nn.Embedding(50, 8, sparse=True).cuda()
    idx = torch.tensor([1, 7, 7, 33], device="cuda")
    emb(idx).sum().backward()
    local = emb.weight.grad.to_dense().clone()
    emb.weight.grad = None
    opt = hvd.DistributedOptimizer(torch.optim.SGD(emb.parameters(), lr=0.5), named_parameters=emb.named_parameters(),
                                   sparse_as_dense=sparse_as_dense)
    before = emb.weight.detach().clone()
    emb(idx).sum().backward()
    assert emb.weight.grad.is_sparse
    opt.step()
    # every rank holds the same gradient: the average is that gradient
    assert torch.allclose(emb.weight.grad.to_dense(), local)
    assert torch.allclose(emb.weight, before - 0.5 * local)
