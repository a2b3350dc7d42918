"""The allreduce entry points of horovod/torch/mpi_ops.py, in front of the HIP path.

Names, arguments, defaults and error behaviour follow the reference
(horovod/torch/mpi_ops.py:98-520): ``allreduce``, ``allreduce_``, ``allreduce_async``,
``allreduce_async_``, the ``grouped_`` family, ``poll`` and ``synchronize``; ``Average``,
``Sum`` and ``Adasum``; the deprecated ``average=`` argument.  What this layer decides is the
pair of scale factors that reaches the kernels:

* ``Average`` becomes ``Sum`` with ``postscale_factor / size()``, as EnqueueTensorAllreduces
  does in non-ROCm builds (common/operations.cc:1394-1398).  The reference's ROCm build
  cannot do that (it has no scale kernels: ops/hip_operations.cc:150-153) and divides in the
  framework instead (mpi_ops.py:100-105, mpi_ops_v2.cc:69-77,118-120); with the kernels of
  this library the division rides on the unpack.
* ``Adasum`` on the GPU averages over the ranks of a node the same way, ``postscale_factor /
  local_size()`` (common/operations.cc:1403-1408), and needs a power-of-two number of nodes.

``init()`` here describes a simulated world (see engine.py); there is no launcher and no
communicator in this package.
"""
import os
import warnings

import torch

from .compression import Compression
from .engine import ADASUM, SUM, Engine, Entry, HorovodInternalError, Request, TORCH_TO_HVD

# ReduceOp values handed out by horovod_reduce_op_*(), common/operations.h:35-40
Average = 0
Sum = 1
Adasum = 2

_engine = None
_handle_map = {}
_next_handle = [0]
_noname = [0]


def init(size=1, local_size=1, peer_source=None, fusion_threshold=None, num_streams=None):
    """Starts the engine for a simulated world of ``size`` ranks (this process is rank 0).

    peer_source(rank, name, tensor) returns what rank 1..size-1 passes under that name; None
    means every rank holds the same values.  fusion_threshold and num_streams default to
    HOROVOD_FUSION_THRESHOLD (bytes, 64 MiB) and HOROVOD_NUM_NCCL_STREAMS, the knobs of
    common/operations.cc:419-441,475-481; without the variable there are two stream slots (the
    reference has one): consecutive fused responses then overlap each other's start-up and drain."""
    global _engine
    if _engine is not None:
        return
    if not torch.cuda.is_available():
        raise RuntimeError("horovod_amd.torch needs a GPU: every operation runs in libhvdhip.so, "
                           "there is no host path")
    if fusion_threshold is None:
        fusion_threshold = int(os.environ.get("HOROVOD_FUSION_THRESHOLD", 64 << 20))
    if num_streams is None:
        num_streams = int(os.environ.get("HOROVOD_NUM_NCCL_STREAMS", 2))
    batch = os.environ.get("HOROVOD_BATCH_D2D_MEMCOPIES", "1") != "0"
    _engine = Engine(size, local_size, peer_source, fusion_threshold, num_streams, batch)


def shutdown():
    global _engine
    if _engine is not None:
        _engine.shutdown()
        _engine = None
    _handle_map.clear()


def is_initialized():
    return _engine is not None


def _state():
    if _engine is None:
        # common/operations.cc:858-864
        raise ValueError("Horovod has not been initialized; use hvd.init().")
    return _engine


def size():
    return _state().size


def local_size():
    return _state().local_size


def cross_size():
    return _state().size // _state().local_size


def rank():
    _state()
    return 0


def local_rank():
    _state()
    return 0


def cross_rank():
    _state()
    return 0


def is_homogeneous():
    _state()
    return True


def rocm_built():
    return True


def nccl_built():
    return True  # the collective position is taken by RCCL in a real deployment


def cuda_built():
    return False


def num_rank_is_power_2(num_rank):
    return num_rank != 0 and (num_rank & (num_rank - 1)) == 0


def handle_average_backwards_compatibility(op, average):
    """horovod/common/util.py:214-232."""
    if op is not None:
        if average is not None:
            raise ValueError('The op parameter supersedes average. Please provide only one of them.')
        return op
    if average is not None:
        warnings.warn('Parameter `average` has been replaced with `op` and will be removed in v0.21.0',
                      DeprecationWarning)
        return Average if average else Sum
    return Average


def _check(tensor):
    if tensor.dtype not in TORCH_TO_HVD:
        raise ValueError('Tensor type %s is not supported.' % tensor.type())
    if not tensor.is_contiguous():
        raise ValueError('Tensor is required to be contiguous.')
    if not tensor.is_cuda:
        raise ValueError('Tensor type %s is not supported: this build only has the GPU path.' % tensor.type())


def _factors(op, prescale_factor, postscale_factor, dtype):
    """Average / Adasum -> (ReduceOp for the op layer, prescale, postscale)."""
    eng = _state()
    if op == Average:
        return SUM, prescale_factor, postscale_factor / eng.size
    if op == Adasum:
        if dtype not in (torch.float16, torch.float32, torch.float64):
            # ops/adasum/adasum.h:118-139
            raise ValueError('Unsupported data type in Adasum: %s' % dtype)
        if not num_rank_is_power_2(eng.size // eng.local_size):
            raise NotImplementedError('Running GPU Adasum with non-power of 2 nodes is not supported yet.')
        return ADASUM, prescale_factor, postscale_factor / eng.local_size
    if op == Sum:
        return SUM, prescale_factor, postscale_factor
    raise ValueError('Unknown reduction op %r' % (op,))


def _name(name, kind):
    if name is not None:
        return '%s.%s' % (kind, name)
    _noname[0] += 1
    return '%s.noname.%d' % (kind, _noname[0])  # GetOpName, horovod/torch/mpi_ops_v2.cc:55-62


def _submit(tensors, outputs, names, op, prescale_factor, postscale_factor, wire_dtype, grouped=False):
    eng = _state()
    if not tensors:
        raise ValueError('No tensors to reduce.')
    for t in tensors:
        _check(t)
    first = tensors[0]
    for t, o in zip(tensors, outputs):
        if t.dtype != first.dtype or t.device != first.device:
            raise ValueError('Tensors of one grouped allreduce must share dtype and device.')
        if o.shape != t.shape or o.dtype != t.dtype or o.device != t.device or not o.is_contiguous():
            raise ValueError('Output must be a contiguous tensor of the shape, dtype and device of the input.')
    red, pre, post = _factors(op, prescale_factor, postscale_factor,
                              torch.float16 if wire_dtype is not None else first.dtype)
    tdt = TORCH_TO_HVD[first.dtype]
    wire = tdt if wire_dtype is None else TORCH_TO_HVD[wire_dtype]
    req = Request([Entry(n, t, o) for n, t, o in zip(names, tensors, outputs)], red, pre, post, 1, tdt, wire,
                  first.device.index)
    req.grouped = grouped
    try:
        eng.enqueue(req)
    except RuntimeError as e:
        raise e if isinstance(e, HorovodInternalError) else HorovodInternalError(e)
    handle = _next_handle[0] = _next_handle[0] + 1
    _handle_map[handle] = req
    return handle


def _allreduce_async(tensor, output, name, op, prescale_factor, postscale_factor, wire_dtype=None):
    return _submit([tensor], [output], [_name(name, 'allreduce')], op, prescale_factor, postscale_factor, wire_dtype)


def _grouped_allreduce_async(tensors, outputs, name, op, prescale_factor, postscale_factor, wire_dtype=None):
    base = _name(name, 'grouped_allreduce')
    n = len(tensors)
    names = ['%s_%dof%d' % (base, i + 1, n) for i in range(n)]  # horovod/torch/mpi_ops_v2.cc:207
    return _submit(list(tensors), list(outputs), names, op, prescale_factor, postscale_factor, wire_dtype,
                   grouped=True)


def allreduce_async(tensor, average=None, name=None, op=None, prescale_factor=1.0, postscale_factor=1.0):
    """Asynchronous allreduce into a new tensor; returns a handle for poll() / synchronize()."""
    op = handle_average_backwards_compatibility(op, average)
    output = tensor.new(tensor.shape)
    return _allreduce_async(tensor, output, name, op, prescale_factor, postscale_factor)


def allreduce_async_(tensor, average=None, name=None, op=None, prescale_factor=1.0, postscale_factor=1.0):
    """Asynchronous in-place allreduce."""
    op = handle_average_backwards_compatibility(op, average)
    return _allreduce_async(tensor, tensor, name, op, prescale_factor, postscale_factor)


def _fused_fp16(compression, tensor):
    return compression is Compression.fp16 and Compression.fp16.fuses_into_packing(tensor)


class HorovodAllreduce(torch.autograd.Function):
    """Differentiable allreduce: the gradient of an allreduce is the allreduce of the gradient."""

    @staticmethod
    def forward(ctx, tensor, average, name, op, prescale_factor, postscale_factor, wire_dtype):
        ctx.args = (average, op, prescale_factor, postscale_factor, wire_dtype)
        red = handle_average_backwards_compatibility(op, average)
        tensor = tensor.contiguous()
        output = tensor.new(tensor.shape)
        return synchronize(_allreduce_async(tensor, output, name, red, prescale_factor, postscale_factor, wire_dtype))

    @staticmethod
    def backward(ctx, grad_output):
        average, op, pre, post, wire_dtype = ctx.args
        return (HorovodAllreduce.apply(grad_output, average, None, op, pre, post, wire_dtype),
                None, None, None, None, None, None)


def allreduce(tensor, average=None, name=None, compression=Compression.none, op=None,
              prescale_factor=1.0, postscale_factor=1.0):
    """Allreduce into a new tensor; differentiable.  With Compression.fp16 on a float32 device
    tensor the cast each way happens inside the pack and unpack kernels."""
    if _fused_fp16(compression, tensor):
        return HorovodAllreduce.apply(tensor, average, name, op, prescale_factor, postscale_factor, torch.float16)
    tensor_compressed, ctx = compression.compress(tensor)
    summed = HorovodAllreduce.apply(tensor_compressed, average, name, op, prescale_factor, postscale_factor, None)
    return compression.decompress(summed, ctx)


def allreduce_(tensor, average=None, name=None, op=None, prescale_factor=1.0, postscale_factor=1.0):
    """In-place allreduce."""
    return synchronize(allreduce_async_(tensor, average, name, op, prescale_factor, postscale_factor))


def grouped_allreduce_async(tensors, average=None, name=None, op=None, prescale_factor=1.0, postscale_factor=1.0):
    op = handle_average_backwards_compatibility(op, average)
    outputs = [t.new(t.shape) for t in tensors]
    return _grouped_allreduce_async(tensors, outputs, name, op, prescale_factor, postscale_factor)


def grouped_allreduce_async_(tensors, average=None, name=None, op=None, prescale_factor=1.0, postscale_factor=1.0):
    op = handle_average_backwards_compatibility(op, average)
    return _grouped_allreduce_async(tensors, tensors, name, op, prescale_factor, postscale_factor)


class HorovodGroupedAllreduce(torch.autograd.Function):
    @staticmethod
    def forward(ctx, average, name, op, prescale_factor, postscale_factor, wire_dtype, *tensors):
        ctx.args = (average, op, prescale_factor, postscale_factor, wire_dtype)
        red = handle_average_backwards_compatibility(op, average)
        tensors = [t.contiguous() for t in tensors]
        outputs = [t.new(t.shape) for t in tensors]
        out = synchronize(_grouped_allreduce_async(tensors, outputs, name, red, prescale_factor, postscale_factor,
                                                   wire_dtype))
        return tuple(out)

    @staticmethod
    def backward(ctx, *grad_output):
        average, op, pre, post, wire_dtype = ctx.args
        reduced = HorovodGroupedAllreduce.apply(average, None, op, pre, post, wire_dtype, *grad_output)
        return (None, None, None, None, None, None, *reduced)


def grouped_allreduce(tensors, average=None, name=None, compression=Compression.none, op=None,
                      prescale_factor=1.0, postscale_factor=1.0):
    if tensors and all(_fused_fp16(compression, t) for t in tensors):
        return list(HorovodGroupedAllreduce.apply(average, name, op, prescale_factor, postscale_factor,
                                                  torch.float16, *tensors))
    compressed, ctxs = zip(*[compression.compress(t) for t in tensors])
    summed = HorovodGroupedAllreduce.apply(average, name, op, prescale_factor, postscale_factor, None, *compressed)
    return [compression.decompress(t, c) for t, c in zip(summed, ctxs)]


def grouped_allreduce_(tensors, average=None, name=None, op=None, prescale_factor=1.0, postscale_factor=1.0):
    return synchronize(grouped_allreduce_async_(tensors, average, name, op, prescale_factor, postscale_factor))


def allgather_async(tensor, name=None):
    """Asynchronously concatenates the tensor with the same-named tensor of every other rank along
    the first dimension, which may differ between ranks (horovod/torch/mpi_ops.py:553-571)."""
    eng = _state()
    _check(tensor)
    output = tensor.new()
    req = Request([Entry(_name(name, 'allgather'), tensor, output)], SUM, 1.0, 1.0, 1, TORCH_TO_HVD[tensor.dtype],
                  TORCH_TO_HVD[tensor.dtype], tensor.device.index, kind="allgather")
    req.grouped = False
    try:
        eng.enqueue(req)
    except RuntimeError as e:
        raise e if isinstance(e, HorovodInternalError) else HorovodInternalError(e)
    handle = _next_handle[0] = _next_handle[0] + 1
    _handle_map[handle] = req
    return handle


class HorovodAllgather(torch.autograd.Function):
    """The gradient of an allgather is this rank's rows of the averaged gradient
    (horovod/torch/mpi_ops.py:574-592)."""

    @staticmethod
    def forward(ctx, tensor, name):
        ctx.dim = tensor.shape[0] if tensor.dim() else 0
        return synchronize(allgather_async(tensor.contiguous(), name))

    @staticmethod
    def backward(ctx, grad_output):
        grad_reduced = allreduce(grad_output.contiguous(), op=Average)
        return grad_reduced.narrow(0, 0, ctx.dim), None  # this process is rank 0: its rows come first


def allgather(tensor, name=None):
    """Concatenation over ranks along the first dimension; differentiable."""
    return HorovodAllgather.apply(tensor, name)


def sparse_allreduce_async(tensor, name, op):
    """A sparse gradient travels as two allgathers, of its indices (transposed, so that entries
    concatenate along the first dimension) and of its values; duplicate indices stay uncoalesced
    and add up when the result is used (horovod/torch/mpi_ops.py:515-535).  Returns a callable
    that waits and builds the combined sparse tensor."""
    t = tensor
    indices_handle = allgather_async(t._indices().transpose(0, 1).contiguous(), name='%s.indices' % name)
    values_handle = allgather_async(t._values().contiguous(), name='%s.values' % name)

    def handle():
        values = synchronize(values_handle)
        indices = synchronize(indices_handle)
        if op == Average:
            values = values / size()
        if indices.dim() == 0 or values.dim() == 0:
            return t.new().resize_as_(t)
        return torch.sparse_coo_tensor(indices.transpose(0, 1), values, t.size(), device=t.device)

    return handle


class _Broadcast:
    """A broadcast in the simulated world: nothing travels, the value is already in place."""

    def __init__(self, output):
        self.output = output


def broadcast_async_(tensor, root_rank, name=None):
    """In-place broadcast from root_rank (horovod/torch/mpi_ops.py:645-690).  This process is rank 0
    of the simulated world: with root 0 the tensor already holds the root's value; another
    root's value comes from peer_source.  No kernel of the library is involved (in the
    reference a broadcast has no fusion buffer either, ops/nccl_operations.cc:444-480)."""
    eng = _state()
    if not 0 <= root_rank < eng.size:
        raise ValueError('Invalid root rank %d for a world of %d ranks.' % (root_rank, eng.size))
    if root_rank != 0 and eng.peer_source is not None:
        value = eng.peer_source(root_rank, _name(name, 'broadcast'), tensor)
        if value.shape != tensor.shape or value.dtype != tensor.dtype:
            raise HorovodInternalError('Mismatched broadcast tensor shapes or types for %r.' % name)
        with torch.no_grad():
            tensor.copy_(value)
    handle = _next_handle[0] = _next_handle[0] + 1
    _handle_map[handle] = _Broadcast(tensor)
    return handle


def broadcast_async(tensor, root_rank, name=None):
    return broadcast_async_(tensor.clone(), root_rank, name)


def broadcast_(tensor, root_rank, name=None):
    return synchronize(broadcast_async_(tensor, root_rank, name))


def broadcast(tensor, root_rank, name=None):
    return synchronize(broadcast_async(tensor, root_rank, name))


def broadcast_parameters(params, root_rank):
    """horovod/torch/functions.py:28-59: a dict (state_dict), or a list of parameters or of
    (name, parameter) pairs."""
    if isinstance(params, dict):
        params = sorted(params.items())
    elif isinstance(params, list):
        params = [p if isinstance(p, tuple) else (None, p) for p in params]
    else:
        raise ValueError('invalid params of type: %s' % type(params))
    for handle in [broadcast_async_(p, root_rank, name) for name, p in params if isinstance(p, torch.Tensor)]:
        synchronize(handle)


def broadcast_optimizer_state(optimizer, root_rank):
    """horovod/torch/functions.py:62-187.  The simulated ranks hold no optimizer, so only rank 0,
    this process, can be the root, and then its state is already the state of the world."""
    if root_rank != 0:
        raise NotImplementedError('only rank 0 holds an optimizer in the simulated world')
    _state()


def broadcast_object(obj, root_rank=0, name=None):
    """horovod/torch/functions.py:190-230."""
    if root_rank != 0:
        raise NotImplementedError('only rank 0 holds Python objects in the simulated world')
    _state()
    return obj


def poll(handle):
    """True once the operation behind the handle has completed on the GPU; does not block."""
    if handle not in _handle_map:
        raise ValueError('Did not find a handle produced by an async operation.')  # mpi_ops.py poll()
    if isinstance(_handle_map[handle], _Broadcast):
        return True
    return _state().poll(_handle_map[handle])


def synchronize(handle):
    """Waits for the operation and returns its output (a list for grouped operations)."""
    if handle not in _handle_map:
        return None
    req = _handle_map.pop(handle)
    if isinstance(req, _Broadcast):
        return req.output
    _state().wait(req)
    outs = [e.output for e in req.entries]
    return outs if req.grouped else outs[0]
