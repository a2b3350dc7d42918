"""What sits between ``allreduce_async_()`` and the kernels, for one process and one GPU.

In the reference a background thread negotiates which tensors are ready on every rank,
fuses the responses (Controller::FuseResponses, common/controller.cc:793-866) and runs the
allreduce op on each fused response (NCCLAllreduce::Execute, ops/nccl_operations.cc:156-214;
AdasumGpuAllreduceOp, ops/adasum_gpu_operations.cc:64-310).  Here there is nothing to
negotiate: a cycle takes every request enqueued since the last one, fuses them with the same
rule (through the C++ adapter) and queues, for every fused response,

    wait for the framework's ready events -> pack (prescale, optional fp16 narrowing)
    -> combine with the other ranks' buffers -> unpack (postscale, widening) -> completion event

on one of the engine's streams through the C ABI of libhvdhip.so.  Nothing here computes.

One GPU cannot hold a real communicator, so the *world* is simulated: ``size`` ranks of which
this process is rank 0.  What ranks 1..size-1 contribute comes from ``peer_source(rank, name,
tensor)``; by default every rank holds the same values, which is what the reference's own
tests arrange by seeding all ranks alike (test/parallel/test_torch.py:251-445).  The peers'
tensors go through the same pack kernel into buffers of their own, as they would on their own
GPU, and the collective is the local reduce-sum (or the Adasum tree) over those resident buffers.
"""
import ctypes
from ctypes import c_int, c_int64, c_void_p

import torch

from .. import host as H
from .._lib import adapter_lib, check, dtype_size, lib

SUM = 1      # ReduceOp values, common/operations.h:35-40
ADASUM = 2
PACK_CAST_THEN_SCALE = 1

TORCH_TO_HVD = {
    torch.uint8: 0, torch.int8: 1, torch.int16: 3, torch.int32: 4, torch.int64: 5,
    torch.float16: 6, torch.float32: 7, torch.float64: 8, torch.bool: 9,
}
_ADASUM_DTYPES = (6, 7, 8)


class HorovodInternalError(RuntimeError):
    """An error of the op layer surfacing in the caller (horovod/common/exceptions.py:18-23)."""


class Entry:
    __slots__ = ("name", "tensor", "output", "count", "parts")

    def __init__(self, name, tensor, output):
        self.name, self.tensor, self.output, self.count = name, tensor, output, tensor.numel()
        self.parts = None  # allgather: what every rank contributes, rank 0 first


class Request:
    def __init__(self, entries, op, prescale, postscale, divisor, tensor_dtype, wire_dtype, device,
                 kind="allreduce"):
        self.kind = kind
        self.entries = entries
        self.op, self.prescale, self.postscale, self.divisor = op, float(prescale), float(postscale), divisor
        self.tensor_dtype, self.wire_dtype, self.device = tensor_dtype, wire_dtype, device
        self.producer = None     # the framework stream that was current at enqueue
        self.markers = []        # one Marker per fused response that carries one of the entries
        self.keepalive = []      # peer tensors in flight
        self.submitted = False
        self.error = None

    def key(self):
        return (self.kind, self.op, self.device, self.tensor_dtype, self.wire_dtype, self.prescale, self.postscale)


class Marker:
    """Completion event of one fused response, shared by the requests it carried
    (ops/gpu_operations.cc:50-56 records one per response)."""
    __slots__ = ("stream", "event", "refs")

    def __init__(self, stream, event, refs):
        self.stream, self.event, self.refs = stream, event, refs


class Engine:
    def __init__(self, size=1, local_size=1, peer_source=None, fusion_threshold=64 << 20, num_streams=1,
                 batch_d2d_memcopies=True, max_plans=128):
        if size < 1 or local_size < 1 or size % local_size:
            raise ValueError("size must be a positive multiple of local_size")
        self.size, self.local_size, self.peer_source = size, local_size, peer_source
        self.fusion_threshold = int(fusion_threshold)
        self.batch_d2d_memcopies = bool(batch_d2d_memcopies)
        self.streams = [H.Stream() for _ in range(max(1, num_streams))]
        self.slot = 0
        self.queue = []
        self.inflight = {}       # tensor name -> request, until synchronised
        self.buffers = {}        # (slot, rank) -> torch uint8 tensor
        self.plans = {}          # insertion-ordered: least recently used first
        self.adasum_plans = {}
        self.max_plans = max_plans
        self.cycles = 0
        self.responses = 0       # fused responses executed so far
        self.ready = {}          # framework stream -> event recorded at the start of the current cycle

    # ---- queueing -------------------------------------------------------

    def enqueue(self, request):
        for e in request.entries:
            if e.name in self.inflight:
                # common/tensor_queue.cc:27-31
                raise HorovodInternalError(
                    "Requested to allreduce a tensor with the same name as another tensor that is "
                    "currently being processed.  If you want to request another tensor, use a different "
                    "tensor name.")
        for e in request.entries:
            self.inflight[e.name] = request
        # The reference records a ready event per request on the framework's stream
        # (RecordReadyEvent, horovod/torch/ready_event.cc).  A cycle here runs on the caller's own
        # thread, after every enqueue it serves, so one event per producing stream and cycle, recorded
        # when the cycle starts, orders the same work and costs one record instead of one per tensor.
        if request.kind == "allgather":
            self._prepare_allgather(request)
        request.producer = torch.cuda.current_stream()
        self.queue.append(request)

    def _prepare_allgather(self, request):
        """Collects what every rank passes (first dimensions may differ, the rest may not:
        AllgatherOp::AllocateOutput, ops/collective_operations.cc:150-198) and allocates the
        output, here, before the cycle's ready event, so that its memory is ordered like any
        other tensor of the framework."""
        for e in request.entries:
            if e.tensor.dim() == 0:
                self.inflight.pop(e.name, None)
                # common/controller.cc:575-579
                raise HorovodInternalError("Rank zero tried to allgather a rank-zero tensor.")
            parts = [e.tensor]
            for rank in range(1, self.size):
                t = e.tensor if self.peer_source is None else self.peer_source(rank, e.name, e.tensor)
                if (not isinstance(t, torch.Tensor) or not t.is_cuda or t.dtype != e.tensor.dtype
                        or t.dim() != e.tensor.dim() or t.shape[1:] != e.tensor.shape[1:] or not t.is_contiguous()):
                    self.inflight.pop(e.name, None)
                    raise HorovodInternalError(
                        "Mismatched allgather tensor shapes: ranks may differ in the first dimension only "
                        "(tensor %r)." % e.name)
                parts.append(t)
            e.parts = parts
            e.output.resize_((sum(t.shape[0] for t in parts),) + tuple(e.tensor.shape[1:]))

    def run_cycle(self):
        """Fuses and queues everything enqueued so far (one pass of RunLoopOnce,
        common/operations.cc:593-717, with every request already agreed upon)."""
        pending, self.queue = self.queue, []
        if not pending:
            return
        self.cycles += 1
        self.ready = {}
        for r in pending:
            if r.producer not in self.ready:
                ev = torch.cuda.Event()
                ev.record(r.producer)
                self.ready[r.producer] = ev
        flat = [(r, e) for r in pending for e in r.entries]
        n = len(flat)
        pad = (lambda b: 16 * ((b + 15) // 16)) if self.batch_d2d_memcopies else (lambda b: b)
        sizes = (c_int64 * n)(*[
            e.output.numel() * dtype_size(r.tensor_dtype) if r.kind == "allgather"  # no padding on that path
            else pad(e.count * dtype_size(r.wire_dtype)) for r, e in flat])
        classes = {}
        keys = (c_int * n)(*[classes.setdefault(r.key(), len(classes)) for r, _ in flat])
        group_of = (c_int * n)()
        ngroups = adapter_lib().hvd_adapter_fuse_keyed(sizes, keys, n, self.fusion_threshold, 0, group_of)
        groups = [[] for _ in range(ngroups)]
        for i in range(n):
            groups[group_of[i]].append(flat[i])
        for g in groups:
            try:
                if g[0][0].kind == "allgather":
                    self._execute_allgather(g)
                else:
                    self._execute(g)
            except Exception as exc:  # surfaces in synchronize(), like a Status passed to the callback
                for r, _ in g:
                    r.error = exc
        for r in pending:
            r.submitted = True

    # ---- resources ------------------------------------------------------

    def _buffer(self, slot, rank, nbytes):
        t = self.buffers.get((slot, rank))
        if t is None or t.numel() < nbytes:
            if t is not None:
                self.streams[slot].synchronize()  # queued kernels may still use the smaller buffer
            t = torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device="cuda")
            self.buffers[(slot, rank)] = t
        return t.data_ptr()

    def _plan(self, tensors, outputs, counts, tensor_dtype, wire_dtype):
        key = (tuple(tensors), tuple(outputs), tuple(counts), tensor_dtype, wire_dtype)
        plan = self.plans.pop(key, None)
        if plan is None:
            if len(self.plans) >= self.max_plans:
                self.plans.pop(next(iter(self.plans))).destroy()
            plan = H.FusionPlan(tensors, outputs, counts, tensor_dtype, wire_dtype)
        self.plans[key] = plan
        return plan

    def _adasum_plan(self, slot, layer_counts, dtype):
        # an Adasum plan owns the partial sums of the combine in flight: one per stream slot
        key = (slot, tuple(layer_counts), dtype)
        plan = self.adasum_plans.get(key)
        if plan is None:
            if len(self.adasum_plans) >= self.max_plans:
                self.adasum_plans.pop(next(iter(self.adasum_plans))).destroy()
            plan = self.adasum_plans[key] = H.AdasumPlan(layer_counts, dtype)
        return plan

    def _peer_tensor(self, rank, request, entry):
        if self.peer_source is None:
            return entry.tensor
        t = self.peer_source(rank, entry.name, entry.tensor)
        if (not isinstance(t, torch.Tensor) or not t.is_cuda or t.dtype != entry.tensor.dtype
                or t.numel() != entry.count or not t.is_contiguous()):
            raise ValueError("peer_source must return a contiguous device tensor of the shape and dtype of %r"
                             % entry.name)
        request.keepalive.append(t)
        return t

    # ---- one fused response --------------------------------------------

    def _execute(self, group):
        first = group[0][0]
        tdt, wire = first.tensor_dtype, first.wire_dtype
        es = dtype_size(wire)
        slot, s, requests = self._begin(group)
        counts = [e.count for _, e in group]
        fused = len(group) > 1 or wire != tdt
        flags = PACK_CAST_THEN_SCALE if wire != tdt else 0

        # the other ranks' tensors (framework stream), then this response's stream waits for them
        peers = [[self._peer_tensor(rank, r, e) for r, e in group] for rank in range(1, self.size)]
        if self.peer_source is not None and peers:
            made = torch.cuda.Event()
            made.record()
            check(lib().hvdhip_stream_wait_event(s.handle, c_void_p(made.cuda_event)), "hvdhip_stream_wait_event")
            first.keepalive.append(made)

        if fused:
            plan = self._plan([e.tensor.data_ptr() for _, e in group], [e.output.data_ptr() for _, e in group],
                              counts, tdt, wire)
            nbytes = plan.buffer_len
        else:
            nbytes = group[0][1].count * es

        # The other ranks' buffers first: with peer_source=None they are made from this rank's own
        # tensors, which an in-place request (output is tensor) overwrites below.
        peer_bufs = []
        for rank, tensors in enumerate(peers, start=1):
            pb = self._buffer(slot, rank, nbytes)
            if fused:
                ptrs = [t.data_ptr() for t in tensors]
                self._plan(ptrs, ptrs, counts, tdt, wire).pack(pb, first.prescale, s, flags)
            else:
                self._scale_or_copy(tensors[0].data_ptr(), pb, counts[0], first.prescale, tdt, s)
            peer_bufs.append(pb)

        if fused:
            result = self._buffer(slot, 0, nbytes)
            plan.pack(result, first.prescale, s, flags)
            offsets = plan.offsets() + [nbytes]
            layer_counts = [(offsets[i + 1] - offsets[i]) // es for i in range(len(group))]  # pad bytes are zero
        else:
            e = group[0][1]
            result = e.output.data_ptr()
            self._scale_or_copy(e.tensor.data_ptr(), result, e.count, first.prescale, tdt, s)
            layer_counts = [e.count]
        nelem = nbytes // es

        if nelem and peer_bufs:
            if first.op == ADASUM:
                self._adasum(slot, result, peer_bufs, nelem, layer_counts, wire, s)
            else:
                self._sum(result, peer_bufs, nelem, wire, s)

        if fused:
            plan.unpack(result, first.postscale, s)
        elif first.postscale != 1.0 and nelem:
            H.scale_buffer(result, result, nelem, first.postscale, tdt, s)

        self._finish(s, requests)

    def _begin(self, group):
        """Picks the stream slot of a fused response and makes it wait for the framework."""
        self.responses += 1
        slot, self.slot = self.slot, (self.slot + 1) % len(self.streams)
        s = self.streams[slot]
        requests = []
        for r, _ in group:
            if r not in requests:
                requests.append(r)
        for producer in {r.producer for r in requests}:
            check(lib().hvdhip_stream_wait_event(s.handle, c_void_p(self.ready[producer].cuda_event)),
                  "hvdhip_stream_wait_event")
        return slot, s, requests

    def _finish(self, s, requests):
        ev = c_void_p()  # completion marker from the event pool
        check(lib().hvdhip_event_acquire(s.handle, ctypes.byref(ev)), "hvdhip_event_acquire")
        check(lib().hvdhip_event_record(ev, s.handle), "hvdhip_event_record")
        marker = Marker(s, ev, len(requests))
        for r in requests:
            r.markers.append(marker)

    def _execute_allgather(self, group):
        """The fusion-buffer side of a fused allgather (AllgatherOp::MemcpyInFusionBuffer /
        MemcpyOutFusionBuffer, ops/collective_operations.cc:234-288): rank r's entries lie back
        to back at displacement sum(recvcounts[:r]); entry e of rank r is copied out to row
        offset sum(first dimensions of ranks < r) of output e.  Every rank's slab is packed here
        (which stands in for the collective), each direction as one batched copy."""
        slot, s, requests = self._begin(group)
        es = dtype_size(group[0][0].tensor_dtype)
        recv = [sum(e.parts[rank].numel() for _, e in group) * es for rank in range(self.size)]
        total = sum(recv)
        buf = self._buffer(slot, 0, total)
        into_buf, from_src, nbytes, out_dst, from_buf = [], [], [], [], []
        written = [0] * len(group)
        at = 0
        for rank in range(self.size):
            for i, (_, e) in enumerate(group):
                part = e.parts[rank]
                n = part.numel() * es
                if n:
                    into_buf.append(buf + at)
                    from_src.append(part.data_ptr())
                    nbytes.append(n)
                    out_dst.append(e.output.data_ptr() + written[i])
                    from_buf.append(buf + at)
                written[i] += n
                at += n
        if nbytes:
            H.batched_d2d_memcpy(into_buf, from_src, nbytes, s)
            H.batched_d2d_memcpy(out_dst, from_buf, nbytes, s)
        self._finish(s, requests)

    @staticmethod
    def _scale_or_copy(src, dst, count, scale, dtype, s):
        """ops/nccl_operations.cc:176-186: an unfused tensor is scaled out of place into its
        output, or copied there when there is nothing to scale."""
        if count == 0:
            return
        if scale != 1.0:
            H.scale_buffer(src, dst, count, scale, dtype, s)
        elif src != dst:
            H.batched_d2d_memcpy([dst], [src], [count * dtype_size(dtype)], s)

    @staticmethod
    def _sum(result, peer_bufs, nelem, dtype, s):
        for i in range(0, len(peer_bufs), 16):
            H.reduce_sum_k(result, peer_bufs[i:i + 16], nelem, dtype, s)

    def _adasum(self, slot, result, peer_bufs, nelem, layer_counts, dtype, s):
        """Ranks of one node are summed (the reduce-scatter leg of
        ops/adasum_gpu_operations.cc:174-197), then the node results are combined pairwise at
        distances 1, 2, 4 ... like the levels of Adasum::FusedAllreduce (ops/adasum/adasum.h:194-340)."""
        bufs = [result] + peer_bufs
        L = self.local_size
        leaders = []
        for node in range(self.size // L):
            lead = bufs[node * L]
            if L > 1:
                self._sum(lead, bufs[node * L + 1:node * L + L], nelem, dtype, s)
            leaders.append(lead)
        plan = self._adasum_plan(slot, layer_counts, dtype)
        d = 1
        while d < len(leaders):
            for i in range(0, len(leaders), 2 * d):
                plan.combine(leaders[i], leaders[i + d], s)
            d *= 2

    # ---- completion -----------------------------------------------------

    def poll(self, request):
        if not request.submitted:
            self.run_cycle()
        if request.error is not None:
            return True
        for m in request.markers:
            done = c_int()
            check(lib().hvdhip_event_query(m.event, ctypes.byref(done)), "hvdhip_event_query")
            if not done.value:
                return False
        return True

    def wait(self, request):
        if not request.submitted:
            self.run_cycle()
        try:
            for m in request.markers:
                check(lib().hvdhip_event_synchronize(m.event), "hvdhip_event_synchronize")
        finally:
            for m in request.markers:
                m.refs -= 1
                if m.refs == 0:  # the last request of the response hands the event back to its pool
                    check(lib().hvdhip_event_release(m.stream.handle, m.event), "hvdhip_event_release")
            request.markers = []
            request.keepalive = []
            for e in request.entries:
                self.inflight.pop(e.name, None)
        if request.error is not None:
            raise HorovodInternalError(str(request.error)) from request.error

    def shutdown(self):
        for r in set(self.inflight.values()):
            try:
                self.wait(r)
            except HorovodInternalError:
                pass
        for plan in list(self.plans.values()) + list(self.adasum_plans.values()):
            plan.destroy()
        self.plans, self.adasum_plans = {}, {}
        for s in self.streams:
            s.destroy()
        self.streams, self.buffers = [], {}
