"""Host-only logic of the horovod.torch-shaped front end (no GPU needed)."""
import warnings

import pytest
import torch


def test_average_argument_compatibility():
    """horovod/common/util.py:214-232."""
    from horovod_amd.torch import mpi_ops as ops
    assert ops.handle_average_backwards_compatibility(None, None) == ops.Average
    assert ops.handle_average_backwards_compatibility(ops.Adasum, None) == ops.Adasum
    with warnings.catch_warnings(record=True) as w:
        warnings.simplefilter("always")
        assert ops.handle_average_backwards_compatibility(None, True) == ops.Average
        assert ops.handle_average_backwards_compatibility(None, False) == ops.Sum
    assert len(w) == 2 and all(issubclass(x.category, DeprecationWarning) for x in w)
    with pytest.raises(ValueError):
        ops.handle_average_backwards_compatibility(ops.Sum, True)
    assert (ops.Average, ops.Sum, ops.Adasum) == (0, 1, 2)  # common/operations.h:35-40


def test_power_of_two_check():
    from horovod_amd.torch.mpi_ops import num_rank_is_power_2
    assert [n for n in range(0, 20) if num_rank_is_power_2(n)] == [1, 2, 4, 8, 16]


def test_compressors_on_their_own_behave_like_the_reference():
    """horovod/torch/compression.py:33-64."""
    from horovod_amd.torch import Compression
    x = torch.tensor([1.0, 2.5, -3.25, 1e-8])
    same, ctx = Compression.none.compress(x)
    assert same is x and ctx is None and Compression.none.decompress(same, ctx) is x
    h, ctx = Compression.fp16.compress(x)
    assert h.dtype == torch.float16 and ctx == torch.float32
    back = Compression.fp16.decompress(h, ctx)
    assert back.dtype == torch.float32 and torch.equal(back, x.half().float())
    i = torch.arange(5)
    hi, ctx = Compression.fp16.compress(i)
    assert hi is i and Compression.fp16.decompress(hi, ctx) is i  # integers are left alone
    assert not Compression.fp16.fuses_into_packing(x)  # host tensors take the plain casts


def test_uninitialised_and_gpu_less_use_fails_loudly():
    import horovod_amd.torch as hvd
    if hvd.is_initialized():
        pytest.skip("engine running")
    with pytest.raises(ValueError, match="not been initialized"):
        hvd.rank()
    with pytest.raises(ValueError, match="not been initialized"):
        hvd.allreduce(torch.ones(3))
    if not torch.cuda.is_available():
        with pytest.raises(RuntimeError, match="no host path"):
            hvd.init()
