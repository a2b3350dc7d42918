"""``DistributedOptimizer``: the caller that turns a backward pass into allreduce requests.

Follows horovod/torch/optimizer.py:34-330 for dense gradients: every parameter's gradient
is handed to ``allreduce_async_`` as soon as it has been accumulated
``backward_passes_per_step`` times, with

    op == Average:  prescale = 1 / gradient_predivide_factor, postscale = gradient_predivide_factor
                    (optimizer.py:190-198; the op layer divides postscale by size())
    otherwise:      both factors 1

``synchronize()`` waits for all of them before ``step()`` applies the update.  Parameters
listed in ``groups`` go out as one grouped request when the last gradient of the group
arrives (optimizer.py:208-213,236-247).  With ``op=Adasum`` in a world of more than one rank
the factory returns the delta-based variant (optimizer.py:333-503) instead.

Two things differ from the reference on purpose.  The ROCm refusal of
``gradient_predivide_factor`` (optimizer.py:570-572) is gone, because the scale kernels it
was waiting for exist here.  And ``Compression.fp16`` on float32 gradients allocates
nothing: the request carries the gradient itself with float16 as the dtype of the fusion
buffer, and the pack and unpack kernels do the two casts.
"""
import warnings
from contextlib import contextmanager

import torch

from . import mpi_ops
from .compression import Compression
from .mpi_ops import Adasum, Average


def _checked_names(param_groups, named_parameters):
    """(name, parameter) for every parameter: the caller's list, validated like
    optimizer.py:41-66, or generated names."""
    if named_parameters is not None:
        named_parameters = list(named_parameters)
    else:
        named_parameters = [('allreduce.noname.%d.%d' % (i, j), v)
                            for i, group in enumerate(param_groups)
                            for j, v in enumerate(group['params'])]
    if any(not isinstance(p, tuple) for p in named_parameters):
        raise ValueError('named_parameters should be a sequence of tuples (name, parameter), '
                         'usually produced by model.named_parameters().')
    names = [k for k, _ in named_parameters]
    dups = sorted({k for k in names if names.count(k) > 1})
    if dups:
        raise ValueError('Parameter names in named_parameters must be unique. '
                         'Found duplicates: %s' % ', '.join(dups))
    all_ids = {id(v) for group in param_groups for v in group['params']}
    unnamed = all_ids - {id(v) for _, v in named_parameters}
    if unnamed:
        raise ValueError('named_parameters was specified, but one or more model parameters were not '
                         'named. Python object ids: %s' % ', '.join(str(i) for i in unnamed))
    return named_parameters


class _DistributedOptimizer(torch.optim.Optimizer):
    def __init__(self, params, named_parameters, compression, backward_passes_per_step=1, op=Average,
                 gradient_predivide_factor=1.0, groups=None, sparse_as_dense=False):
        super(self.__class__, self).__init__(params)
        self._compression = compression
        named_parameters = _checked_names(self.param_groups, named_parameters)
        self._parameter_names = {v: k for k, v in sorted(named_parameters)}
        self.backward_passes_per_step = backward_passes_per_step
        self._allreduce_delay = {v: backward_passes_per_step for _, v in sorted(named_parameters)}
        self.op = op
        self.gradient_predivide_factor = gradient_predivide_factor
        self.sparse_as_dense = sparse_as_dense
        self._handles = {}
        self._hooks = []
        self._requires_update = set()
        self._synchronized = False
        self._should_synchronize = True
        if groups is not None:
            if not (isinstance(groups, list) or groups > 0):
                raise ValueError('groups should be a non-negative integer or a list of list of torch.Tensor.')
            if isinstance(groups, list):
                seen = set()
                for members in groups:
                    for p in members:
                        if not isinstance(p, torch.Tensor):
                            raise ValueError('groups must consist of torch.Tensor.')
                        if id(p) in seen:
                            raise ValueError('A parameter can only appear once in groups.')
                        seen.add(id(p))
        self._groups = groups
        self._p_to_group = {}
        self._group_counts = {}
        if mpi_ops.size() > 1:
            self._register_hooks()

    def set_backward_passes_per_step(self, passes):
        self.backward_passes_per_step = passes
        for p in self._allreduce_delay:
            self._allreduce_delay[p] = passes

    def _register_hooks(self):
        if self._groups is not None:
            ps = [p for group in self.param_groups for p in group['params'] if p.requires_grad]
            if isinstance(self._groups, list):
                have = {id(p) for p in ps}
                listed = [tuple(p for p in members if id(p) in have) for members in self._groups]
                grouped = {id(p) for members in listed for p in members}
                self._groups = [m for m in listed if m] + [(p,) for p in ps if id(p) not in grouped]
            else:  # that many runs of consecutive parameters, sizes as even as possible (optimizer.py:143-157)
                k = min(self._groups, max(len(ps), 1))
                step, extra = divmod(len(ps), k)
                runs, at = [], 0
                for i in range(k):
                    n = step + (1 if i < extra else 0)
                    runs.append(tuple(ps[at:at + n]))
                    at += n
                self._groups = [r for r in runs if r]
            for members in self._groups:
                for p in members:
                    self._p_to_group[p] = members
                self._group_counts[members] = 0
        for group in self.param_groups:
            for p in group['params']:
                if p.requires_grad:
                    self._requires_update.add(p)
                    self._hooks.append(p.register_post_accumulate_grad_hook(self._make_hook(p)))

    def _factors(self):
        if self.op == Average:
            return 1.0 / self.gradient_predivide_factor, self.gradient_predivide_factor
        return 1.0, 1.0

    def _allreduce_grad_async(self, p):
        if p.grad is None:
            # another rank may have computed it (dynamic graphs): contribute zeros, optimizer.py:174-181
            p.grad = p.data.new(p.size()).zero_()
        name = self._parameter_names.get(p)
        tensor = p.grad
        if tensor.is_sparse:
            if not self.sparse_as_dense:
                # indices and values by allgather, optimizer.py:215-217
                return mpi_ops.sparse_allreduce_async(tensor, name=name, op=self.op), None
            tensor = tensor.to_dense()
        pre, post = self._factors()
        if self._compression is Compression.fp16 and Compression.fp16.fuses_into_packing(tensor):
            handle = mpi_ops._allreduce_async(tensor, tensor, name, self.op, pre, post, wire_dtype=torch.float16)
            return handle, None
        compressed, ctx = self._compression.compress(tensor)
        handle = mpi_ops.allreduce_async_(compressed, name=name, op=self.op, prescale_factor=pre,
                                          postscale_factor=post)
        return handle, ctx

    def _grouped_allreduce_grad_async(self, ps):
        name = self._parameter_names.get(ps[0])
        grads = [p.grad for p in ps]
        if self._compression is Compression.fp16 and all(Compression.fp16.fuses_into_packing(g) for g in grads):
            handle = mpi_ops._grouped_allreduce_async(grads, grads, name, self.op, 1.0, 1.0, wire_dtype=torch.float16)
            return handle, [None] * len(ps)
        compressed, ctxs = zip(*[self._compression.compress(g) for g in grads])
        return mpi_ops.grouped_allreduce_async_(list(compressed), name=name, op=self.op), ctxs

    def _make_hook(self, p):
        def hook(*ignore):
            if p in self._handles and self._handles[p][0] is not None and self._allreduce_delay[p] <= 0:
                raise AssertionError(
                    "Gradients were computed more than backward_passes_per_step times before call to step(). "
                    "Increase backward_passes_per_step to accumulate gradients locally.")
            assert not p.grad.requires_grad
            assert self._allreduce_delay[p] > 0
            handle, ctx = None, None
            self._allreduce_delay[p] -= 1
            if self._allreduce_delay[p] == 0:
                if self._groups is not None:
                    members = self._p_to_group[p]
                    self._group_counts[members] += 1
                    if self._group_counts[members] == len(members):
                        self._handles[members] = self._grouped_allreduce_grad_async(members)
                        for gp in members:
                            self._handles.pop(gp, None)
                        self._group_counts[members] = 0
                        return
                else:
                    handle, ctx = self._allreduce_grad_async(p)
            self._handles[p] = (handle, ctx)
        return hook

    def _finish(self, p, output, ctx):
        self._allreduce_delay[p] = self.backward_passes_per_step
        if ctx is None and not output.is_sparse and not p.grad.is_sparse and output.data_ptr() == p.grad.data_ptr():
            return  # reduced in place
        result = output if ctx is None else self._compression.decompress(output, ctx)
        if p.grad.is_sparse:
            p.grad.zero_().add_(result if result.is_sparse else result.to_sparse())
        else:
            p.grad.set_(result)

    def synchronize(self):
        done = set()
        for x in self._handles:
            done.update(x) if isinstance(x, tuple) else done.add(x)
        for p in self._requires_update - done:
            self._handles[p] = self._allreduce_grad_async(p)
        for p, (handle, ctx) in list(self._handles.items()):
            if handle is None:
                self._handles[p] = self._allreduce_grad_async(p)
        for p, (handle, ctx) in self._handles.items():
            if isinstance(p, tuple):
                outputs = mpi_ops.synchronize(handle)
                for gp, output, gctx in zip(p, outputs, ctx):
                    self._finish(gp, output, gctx)
                if self._groups is not None:
                    self._group_counts[p] = 0
            else:
                # a sparse gradient's handle is a function that waits and assembles the result
                output = handle() if callable(handle) else mpi_ops.synchronize(handle)
                if self._groups is not None:
                    self._group_counts[self._p_to_group[p]] = 0
                self._finish(p, output, ctx)
        self._handles.clear()
        self._synchronized = True

    @contextmanager
    def skip_synchronize(self):
        """``optimizer.synchronize()``, then ``with optimizer.skip_synchronize(): optimizer.step()``
        (for gradient clipping between the two)."""
        self._should_synchronize = False
        try:
            yield
        finally:
            self._should_synchronize = True

    def step(self, closure=None):
        if self._should_synchronize:
            if self._synchronized:
                warnings.warn("optimizer.step() called without optimizer.skip_synchronize() context after "
                              "optimizer.synchronize(). This can cause training slowdown. You may want to "
                              "consider using optimizer.skip_synchronize() context if you use "
                              "optimizer.synchronize() in your code.")
            self.synchronize()
        self._synchronized = False
        return super(self.__class__, self).step(closure)

    def zero_grad(self, *args, **kwargs):
        if self._handles:
            raise AssertionError("optimizer.zero_grad() was called after loss.backward() but before "
                                 "optimizer.step() or optimizer.synchronize(). This is prohibited as it can "
                                 "cause a race condition.")
        return super(self.__class__, self).zero_grad(*args, **kwargs)

    def load_state_dict(self, *args, **kwargs):
        self._handles = {}
        self._synchronized = False
        self._should_synchronize = True
        for p in self._allreduce_delay:
            self._allreduce_delay[p] = self.backward_passes_per_step
        super(self.__class__, self).load_state_dict(*args, **kwargs)


class _DistributedAdasumOptimizer(torch.optim.Optimizer):
    """Adasum combines parameter *updates*, not gradients (horovod/torch/optimizer.py:333-503).

    When a parameter's gradient is complete the wrapped optimizer steps on that parameter
    alone; the difference to the value before the step (the delta) replaces the parameter's
    data and goes out as an in-place ``allreduce_async_(op=Adasum)``.  ``step()`` waits for the
    combined deltas and sets every parameter to its value before the local step plus the
    combined delta."""

    def __init__(self, params, named_parameters, compression, backward_passes_per_step=1):
        super(self.__class__, self).__init__(params)
        self._compression = compression
        named_parameters = _checked_names(self.param_groups, named_parameters)
        self._parameter_names = {v: k for k, v in sorted(named_parameters)}
        self.backward_passes_per_step = backward_passes_per_step
        self._allreduce_delay = {v: backward_passes_per_step for _, v in sorted(named_parameters)}
        self._handles = {}
        self._hooks = []
        self._requires_update = set()
        self._starting_models = {p: torch.zeros_like(p, requires_grad=False) for _, p in named_parameters}
        for group in self.param_groups:
            for p in group['params']:
                if p.requires_grad:
                    p.grad = p.data.new(p.size()).zero_()
                    self._requires_update.add(p)
                    self._hooks.append(p.register_post_accumulate_grad_hook(self._make_hook(p)))

    def set_backward_passes_per_step(self, passes):
        self.backward_passes_per_step = passes
        for p in self._allreduce_delay:
            self._allreduce_delay[p] = passes

    def _allreduce_grad_async(self, p):
        start = self._starting_models[p]
        kept = [group['params'] for group in self.param_groups]
        try:
            for group in self.param_groups:  # the wrapped optimizer steps on p alone
                group['params'] = [p] if any(p is v for v in group['params']) else []
            start.data.copy_(p)
            super(self.__class__, self).step()
            p.data.sub_(start)  # p now holds the delta of the local step
        finally:
            for group, params in zip(self.param_groups, kept):
                group['params'] = params
        compressed, ctx = self._compression.compress(p)
        handle = mpi_ops.allreduce_async_(compressed.data, name=self._parameter_names.get(p), op=Adasum)
        return handle, ctx

    def _make_hook(self, p):
        def hook(*ignore):
            if p in self._handles and self._handles[p][0] is not None and self._allreduce_delay[p] <= 0:
                raise AssertionError(
                    "Gradients were computed more than backward_passes_per_step times before call to step(). "
                    "Increase backward_passes_per_step to accumulate gradients locally.")
            assert not p.grad.requires_grad
            assert self._allreduce_delay[p] > 0
            handle, ctx = None, None
            self._allreduce_delay[p] -= 1
            if self._allreduce_delay[p] == 0:
                handle, ctx = self._allreduce_grad_async(p)
            self._handles[p] = (handle, ctx)
        return hook

    def synchronize(self):
        pass

    @contextmanager
    def skip_synchronize(self):
        raise AssertionError("Skipping synchronization is not supported when using Adasum optimizer.")
        yield  # pragma: no cover

    def step(self, closure=None):
        loss = closure() if closure is not None else None
        for p in self._requires_update - set(self._handles):
            self._handles[p] = self._allreduce_grad_async(p)
        for p, (handle, ctx) in list(self._handles.items()):
            if handle is None:  # step() before the last of backward_passes_per_step passes
                handle, ctx = self._handles[p] = self._allreduce_grad_async(p)
            delta = self._compression.decompress(mpi_ops.synchronize(handle), ctx)
            start = self._starting_models[p]
            start.data.add_(delta.data)
            p.data.copy_(start)
            self._allreduce_delay[p] = self.backward_passes_per_step
        self._handles.clear()
        return loss

    def zero_grad(self, *args, **kwargs):
        if self._handles:
            raise AssertionError("optimizer.zero_grad() was called after loss.backward() but before "
                                 "optimizer.step() or optimizer.synchronize(). This is prohibited as it can "
                                 "cause a race condition.")
        return super(self.__class__, self).zero_grad(*args, **kwargs)


def DistributedOptimizer(optimizer, named_parameters=None, compression=Compression.none,
                         backward_passes_per_step=1, op=Average, gradient_predivide_factor=1.0,
                         num_groups=0, groups=None, sparse_as_dense=False):
    """Wraps ``optimizer`` so that gradients are combined across ranks before ``step()``.

    Arguments as in horovod/torch/optimizer.py:506-597.  The returned object is an instance
    of a class derived from the optimizer's own class."""
    if gradient_predivide_factor != 1.0 and op != Average:
        raise ValueError('gradient_predivide_factor not supported with op != Average')
    if num_groups != 0:
        warnings.warn('Parameter `num_groups` has been replaced by `groups` and will be removed in v0.23.0.',
                      DeprecationWarning)
        if groups is None:
            groups = num_groups
    if op != Adasum or mpi_ops.size() == 1:
        cls = type(optimizer.__class__.__name__, (optimizer.__class__,), dict(_DistributedOptimizer.__dict__))
        return cls(optimizer.param_groups, named_parameters, compression, backward_passes_per_step, op,
                   gradient_predivide_factor, groups, sparse_as_dense)
    cls = type(optimizer.__class__.__name__, (optimizer.__class__,), dict(_DistributedAdasumOptimizer.__dict__))
    return cls(optimizer.param_groups, named_parameters, compression, backward_passes_per_step)
