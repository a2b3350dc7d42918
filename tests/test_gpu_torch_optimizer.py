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


def test_force_allreduce_on_parameters_without_gradient(hvd):
    """test/parallel/test_torch.py:1791-1858: a branch of the model that this rank's loss does
    not reach still takes part in step(): the rank contributes zeros (optimizer.py:174-181)."""
    size = 2

    def peer(rank, name, tensor):
        return torch.full_like(tensor, 0.5)

    hvd.init(size=size, peer_source=peer)

    class Net(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.fc1 = torch.nn.Linear(10, 6)
            self.fc2 = torch.nn.Linear(6, 4)
            self.fc3 = torch.nn.Linear(4, 4)

        def forward(self, x):
            h = torch.relu(self.fc1(x))
            a = self.fc2(h)
            return a, self.fc3(torch.relu(a))

    for cls, kwargs in [(torch.optim.SGD, dict(lr=0.2, momentum=0.9, weight_decay=0.1)), (torch.optim.Adam, dict(lr=0.2)),
                        (torch.optim.RMSprop, dict(lr=0.2, centered=True)), (torch.optim.Adagrad, dict(lr=0.2))]:
        torch.manual_seed(5)
        model = Net().cuda()
        opt = hvd.DistributedOptimizer(cls(model.parameters(), **kwargs), named_parameters=model.named_parameters())
        assert isinstance(opt, cls)
        first, _ = model(torch.randn(8, 10, device="cuda"))
        opt.zero_grad()
        first.pow(2).sum().backward()  # fc3 gets no gradient here
        assert model.fc3.weight.grad is None
        opt.synchronize()
        # zeros from this rank and 0.5 from the other, averaged
        assert torch.equal(model.fc3.weight.grad, torch.full_like(model.fc3.weight, 0.25)), cls.__name__
        assert torch.equal(model.fc3.bias.grad, torch.full_like(model.fc3.bias, 0.25)), cls.__name__
        with opt.skip_synchronize():
            opt.step()
        assert all(torch.isfinite(p).all() for p in model.parameters())


def test_dynamic_requires_grad(hvd):
    """test/parallel/test_torch.py:1961-2009: two optimizers whose parameters are switched off and
    on between steps; only the trained half gets (non-zero) gradients and only its optimizer steps."""
    hvd.init(size=2)
    torch.manual_seed(6)
    gen = torch.nn.Conv2d(1, 10, 1).cuda()
    disc = torch.nn.Conv2d(10, 1, 1).cuda()
    inp = torch.rand([1, 1, 20, 20], device="cuda")
    gen_opt = hvd.DistributedOptimizer(torch.optim.SGD(gen.parameters(), lr=0.1), named_parameters=gen.named_parameters())
    disc_opt = hvd.DistributedOptimizer(torch.optim.SGD(disc.parameters(), lr=0.1), named_parameters=disc.named_parameters())

    def train_step(train_generator=False, train_discriminator=False):
        for p in gen.parameters():
            p.requires_grad_(train_generator)
        for p in disc.parameters():
            p.requires_grad_(train_discriminator)
        gen_opt.zero_grad()
        disc_opt.zero_grad()
        disc(gen(inp)).sum().backward()
        for p in gen.parameters():
            assert train_generator == (p.grad is not None and bool(p.grad.abs().max() != 0))
        for p in disc.parameters():
            assert train_discriminator == (p.grad is not None and bool(p.grad.abs().max() != 0))
        if train_generator:
            gen_opt.step()
        if train_discriminator:
            disc_opt.step()

    for _ in range(3):
        train_step(train_generator=True)
        train_step(train_discriminator=True)


def test_gradient_clipping_between_synchronize_and_step(hvd):
    """test/parallel/test_torch.py:2011-2041."""
    hvd.init(size=2)
    model = torch.nn.Linear(1, 1).cuda()
    with torch.no_grad():
        model.weight.fill_(0.5)
        model.bias.zero_()
    opt = hvd.DistributedOptimizer(torch.optim.SGD(model.parameters(), lr=0.1), named_parameters=model.named_parameters())
    x = torch.ones(1, 1, device="cuda")
    loss = torch.nn.functional.mse_loss(model(x), torch.ones(1, 1, device="cuda"))
    opt.zero_grad()
    loss.backward()
    opt.synchronize()
    prior = model.weight.grad.item()
    assert prior == pytest.approx(-1.0)  # d/dw (0.5 - 1)^2 = -1 on both ranks, averaged
    torch.nn.utils.clip_grad_norm_(model.parameters(), 0.1)
    clipped = model.weight.grad.item()
    assert abs(prior) > abs(clipped)
    with opt.skip_synchronize():
        opt.step()
    assert model.weight.item() == pytest.approx(0.5 - 0.1 * clipped)


def test_no_named_parameters(hvd):
    """test/parallel/test_torch.py:2076-2100, 2375-2392: generated names."""
    hvd.init(size=2)
    torch.manual_seed(7)
    model = torch.nn.Sequential(torch.nn.Conv2d(1, 20, 1), torch.nn.Conv2d(20, 1, 1)).cuda()
    opt = hvd.DistributedOptimizer(torch.optim.SGD(model.parameters(), lr=0.1))
    want = None
    for _ in range(2):  # the second pass reuses the names of the first
        opt.zero_grad()
        model(torch.ones([1, 1, 30, 30], device="cuda")).sum().backward()
        local = [p.grad.clone() for p in model.parameters()]
        opt.synchronize()
        for p, g in zip(model.parameters(), local):
            assert torch.equal(p.grad, g)  # equal ranks: the average is the gradient
        with opt.skip_synchronize():
            opt.step()


def test_joined_rank_contributes_zeros_to_a_fused_response(hvd):
    """test/parallel/test_torch.py:2126-2192 ("two tensors to test fusion"): a rank that has
    joined takes part with zero-filled tensors, so the average over all ranks is the sum of
    the others divided by size()."""
    size = 3

    def peer(rank, name, tensor):  # rank 2 has joined
        return torch.zeros_like(tensor) if rank == 2 else torch.ones_like(tensor) * (rank + 1)

    hvd.init(size=size, peer_source=peer)
    a = torch.ones(5, 3, device="cuda")
    b = torch.ones(7, device="cuda")
    ha = hvd.allreduce_async(a, name="join.a")
    hb = hvd.allreduce_async(b, name="join.b")
    ra, rb = hvd.synchronize(ha), hvd.synchronize(hb)
    assert torch.allclose(ra, torch.full_like(a, (1 + 2 + 0) / 3))
    assert torch.allclose(rb, torch.full_like(b, (1 + 2 + 0) / 3))


@pytest.mark.parametrize("opt_cls,kwargs", [(torch.optim.SGD, dict(lr=0.05, momentum=0.9)), (torch.optim.Adam, dict(lr=0.01))])
@pytest.mark.parametrize("compression", ["none", "fp16"])
def test_training_loop_equals_the_single_process_loop(hvd, opt_cls, kwargs, compression):
    """Twenty steps with every rank holding equal gradients (what the reference's tests create by
    seeding all ranks alike): the average over a power-of-two world is exact, so the distributed
    run must follow the plain optimizer bit for bit -- with fp16 compression, the plain optimizer
    fed gradients rounded to half.  Exercises hook -> fuse -> pack -> reduce -> unpack -> step
    over many steps with the cached plans and changing values."""
    hvd.init(size=4)
    ref_model, model = _model(), _model()
    ref_opt = opt_cls(ref_model.parameters(), **kwargs)
    comp = hvd.Compression.fp16 if compression == "fp16" else hvd.Compression.none
    opt = hvd.DistributedOptimizer(opt_cls(model.parameters(), **kwargs), named_parameters=model.named_parameters(),
                                   compression=comp)
    torch.manual_seed(11)
    for step in range(20):
        x = torch.randn(16, 20, device="cuda")
        ref_opt.zero_grad()
        ref_model(x).pow(2).mean().backward()
        if compression == "fp16":
            for p in ref_model.parameters():
                p.grad = p.grad.half().float()
        ref_opt.step()
        opt.zero_grad()
        model(x).pow(2).mean().backward()
        opt.step()
        for (n, p), q in zip(model.named_parameters(), ref_model.parameters()):
            assert torch.equal(p, q), (step, n)
