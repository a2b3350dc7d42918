"""``import horovod_amd.torch as hvd``: the allreduce surface of ``horovod.torch`` in front of
the MI355X gradient path (see mpi_ops.py, optimizer.py and engine.py)."""
from .compression import Compression  # noqa: F401
from .engine import HorovodInternalError  # noqa: F401
from .mpi_ops import (  # noqa: F401
    Adasum, Average, Sum, allgather, allgather_async, allreduce, allreduce_, allreduce_async, allreduce_async_,
    broadcast, broadcast_, broadcast_async, broadcast_async_, broadcast_object, broadcast_optimizer_state,
    broadcast_parameters, cross_rank, cross_size,
    cuda_built, grouped_allreduce, grouped_allreduce_, grouped_allreduce_async, grouped_allreduce_async_, init,
    is_homogeneous, is_initialized, local_rank, local_size, nccl_built, poll, rank, rocm_built, shutdown, size,
    sparse_allreduce_async, synchronize,
)
from .optimizer import DistributedOptimizer  # noqa: F401
