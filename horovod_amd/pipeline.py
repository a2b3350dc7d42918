"""The allreduce op sequence of the reference on one GPU, driven through the C ABI.

Mirrors NCCLAllreduce::Execute (ops/nccl_operations.cc:156-214) for a list of
gradient tensors: the tensors are grouped into fusion cycles by the greedy
planner, and every cycle runs

    fused (more than one entry):  scaled pack -> sum with the peer chunk(s) -> scaled unpack
    single entry:                 prescale tensor -> output (out of place), sum in place, postscale

with the inter-GPU collective replaced by the local reduce-sum against peer
buffers resident on the same device.  Cycles alternate over `num_streams`
streams, each with its own fusion buffer, as the reference rotates
current_nccl_stream after every op (ops/gpu_operations.cc:101-103).

This module only sequences calls; all arithmetic happens in libhvdhip.so.
"""
import ctypes

import torch

from . import host as H
from ._lib import check, dtype_size, lib
from .workloads import FUSION_THRESHOLD, fuse, reduce_scatter_share


class Cycle:
    def __init__(self, indices, plan, single):
        self.indices = indices
        self.plan = plan          # FusionPlan, or None for a single-entry response
        self.single = single      # (tensor_ptr, output_ptr, count) for a single-entry response
        self.buffer_elems = 0     # elements of the fusion buffer (padded) or of the single tensor
        self.payload_in = 0       # bytes read from tensors
        self.payload_buf = 0      # payload bytes in the buffer dtype
        self.payload_out = 0      # bytes written to outputs


class AllreducePipeline:
    """tensor_ptrs/output_ptrs/counts describe the gradients (device addresses).

    peers: list of callables or None; peer_ptr(cycle_index, peer) must return the
    device address of that peer's chunk for the cycle, `reduce_fraction` of the
    cycle's buffer long (1.0 = the whole buffer, 1/8 = one GPU's reduce-scatter
    share)."""

    def __init__(self, tensor_ptrs, output_ptrs, counts, tensor_dtype, buffer_dtype=None,
                 threshold=FUSION_THRESHOLD, num_streams=1, completion_events=None, streams=None,
                 buffers=None, array_entry_points=False, record_with_unpack=False):
        """completion_events: record a pooled event after every cycle and wait on those in
        synchronize(), as GPUOpContext::FinalizeGPUQueue does (about 2 us of stream time per
        event).  Default: on when cycles alternate over several streams, off for one stream,
        where synchronize() simply waits for the stream.

        streams: existing Stream objects to run on instead of creating num_streams new ones
        (they stay with the caller), so that several pipelines queue on the same streams.

        buffers: the fusion buffers of another pipeline on the same streams, one per stream slot, to
        share instead of allocating new ones (the reference keeps one fusion buffer per stream slot
        for every response that runs there, ops/gpu_operations.cc:122-124).

        array_entry_points: pack and unpack through hvdhip_batched_scaled_d2d_memcpy, the launcher
        that takes the copies as arrays with every call (ops/gpu_operations.cc:186-206), instead of
        explicit plans; same-dtype buffers only.

        record_with_unpack: a fused cycle's completion event goes out with its unpack
        (hvdhip_fusion_unpack_record) instead of as a record of its own behind it."""
        self.record_with_unpack = bool(record_with_unpack)
        self.tensor_dtype = int(tensor_dtype)
        self.buffer_dtype = int(tensor_dtype if buffer_dtype is None else buffer_dtype)
        ts, bs = dtype_size(self.tensor_dtype), dtype_size(self.buffer_dtype)
        self.bs = bs
        groups = fuse([c * bs for c in counts], threshold)
        self.cycles = []
        max_len = 0
        for g in groups:
            if len(g) > 1 or self.buffer_dtype != self.tensor_dtype:
                plan = H.FusionPlan([tensor_ptrs[i] for i in g], [output_ptrs[i] for i in g],
                                    [counts[i] for i in g], self.tensor_dtype, self.buffer_dtype)
                cyc = Cycle(g, plan, None)
                cyc.buffer_elems = plan.buffer_len // bs
                max_len = max(max_len, plan.buffer_len)
            else:
                i = g[0]
                cyc = Cycle(g, None, (tensor_ptrs[i], output_ptrs[i], counts[i]))
                cyc.buffer_elems = counts[i]
            n = sum(counts[i] for i in g)
            cyc.payload_in, cyc.payload_buf, cyc.payload_out = n * ts, n * bs, n * ts
            self.cycles.append(cyc)
        self.owns_streams = streams is None
        self.streams = [H.Stream() for _ in range(num_streams)] if streams is None else list(streams)
        num_streams = len(self.streams)
        self.completion_events = (num_streams > 1) if completion_events is None else bool(completion_events)
        self.pending = []  # (stream, event) recorded after each cycle
        # room for the dummy elements a reduce-scatter over up to 64 ranks may append (64 * 64 elements)
        need = max(max_len, 16) + 4096 * bs
        if buffers is not None:
            if len(buffers) != num_streams or any(b.numel() < need for b in buffers):
                raise ValueError("shared fusion buffers must be one per stream slot and large enough")
            self.buffers = list(buffers)
        else:
            self.buffers = [torch.zeros(need, dtype=torch.uint8, device="cuda") for _ in range(num_streams)]
        self.array_entry_points = bool(array_entry_points)
        if self.array_entry_points:
            if self.buffer_dtype != self.tensor_dtype:
                raise ValueError("the array-taking copies do not convert between dtypes")
            # the descriptor arrays as a C caller holds them, built once per (cycle, stream slot)
            for cyc in self.cycles:
                if cyc.plan is None:
                    continue
                offs = cyc.plan.offsets()
                cyc.arrays = []
                for slot in range(num_streams):
                    fb = self.buffers[slot].data_ptr()
                    in_buf = H._ptr_array([fb + o for o in offs])
                    tens = H._ptr_array([tensor_ptrs[i] for i in cyc.indices])
                    outs = H._ptr_array([output_ptrs[i] for i in cyc.indices])
                    sizes = H._size_array([counts[i] * bs for i in cyc.indices])
                    cyc.arrays.append((in_buf, tens, outs, sizes, len(cyc.indices)))
        torch.cuda.synchronize()

    def reduce_elems(self, cyc, fraction):
        """Elements of the chunk that is reduced: the whole buffer, or with fraction = 1 / world the
        share of rank 0 in the reference's reduce-scatter (ops/nccl_operations.cc:289-316)."""
        if fraction >= 1.0:
            return cyc.buffer_elems
        return reduce_scatter_share(cyc.buffer_elems, int(round(1.0 / fraction)), fused=cyc.plan is not None)

    def _copy_arrays(self, out, inp, sizes, n, scale, s):
        check(lib().hvdhip_batched_scaled_d2d_memcpy(out, inp, sizes, n, float(scale), self.tensor_dtype, s.handle),
              "hvdhip_batched_scaled_d2d_memcpy")

    def run(self, prescale, postscale, peer_ptr=None, num_peers=0, fraction=1.0, kway=True, flags=0, first_slot=0):
        """Queues every cycle; returns without synchronising.  Cycle i runs on stream slot
        (first_slot + i) % streams."""
        for ci, cyc in enumerate(self.cycles):
            slot = (first_slot + ci) % len(self.streams)
            s = self.streams[slot]
            if cyc.plan is not None:
                fb = self.buffers[slot].data_ptr()
                if self.array_entry_points:
                    in_buf, tens, _, sizes, n = cyc.arrays[slot]
                    self._copy_arrays(in_buf, tens, sizes, n, prescale, s)
                else:
                    cyc.plan.pack(fb, prescale, s, flags)
                res = fb
            else:
                t, o, n = cyc.single
                if prescale != 1.0:
                    H.scale_buffer(t, o, n, prescale, self.tensor_dtype, s)
                elif t != o:
                    H.batched_d2d_memcpy([o], [t], [n * self.bs], s)
                res = o
            if num_peers:
                n = self.reduce_elems(cyc, fraction)
                ptrs = [peer_ptr(ci, p) for p in range(num_peers)]
                if kway:
                    H.reduce_sum_k(res, ptrs, n, self.buffer_dtype, s)
                else:
                    for p in ptrs:
                        H.reduce_sum(res, p, n, self.buffer_dtype, s)
            if cyc.plan is not None and self.array_entry_points:
                in_buf, _, outs, sizes, n = cyc.arrays[slot]
                self._copy_arrays(outs, in_buf, sizes, n, postscale, s)
            elif cyc.plan is not None and self.completion_events and self.record_with_unpack:
                ev = ctypes.c_void_p()
                check(lib().hvdhip_event_acquire(s.handle, ctypes.byref(ev)), "hvdhip_event_acquire")
                cyc.plan.unpack(self.buffers[slot].data_ptr(), postscale, s, event=ev)
                self.pending.append((s, ev))
                continue
            elif cyc.plan is not None:
                cyc.plan.unpack(self.buffers[slot].data_ptr(), postscale, s)
            elif postscale != 1.0:
                t, o, n = cyc.single
                H.scale_buffer(o, o, n, postscale, self.tensor_dtype, s)
            # completion marker from the event pool (ops/gpu_operations.cc:50-56); the finalizer waits on it
            if self.completion_events:
                ev = ctypes.c_void_p()
                check(lib().hvdhip_event_acquire(s.handle, ctypes.byref(ev)), "hvdhip_event_acquire")
                check(lib().hvdhip_event_record(ev, s.handle), "hvdhip_event_record")
                self.pending.append((s, ev))

    def synchronize(self):
        """Waits for every cycle's completion event and returns the events to their pools
        (GPUContext::WaitForEvents, ops/cuda_operations.cc:102-148)."""
        for s, ev in self.pending:
            check(lib().hvdhip_event_synchronize(ev), "hvdhip_event_synchronize")
            check(lib().hvdhip_event_release(s.handle, ev), "hvdhip_event_release")
        self.pending = []
        for s in self.streams:
            s.synchronize()

    def algorithmic_bytes(self, num_peers=0, fraction=1.0, kway=True):
        """pack = P_in + P_buf, unpack = P_buf + P_out, reduce = (k+2)*C k-way or 3*C per peer."""
        total = 0
        for cyc in self.cycles:
            if cyc.plan is not None:
                total += cyc.payload_in + cyc.payload_buf + cyc.payload_buf + cyc.payload_out
            else:
                total += cyc.payload_in + cyc.payload_out  # prescale tensor -> output
            if num_peers:
                c = self.reduce_elems(cyc, fraction) * self.bs
                total += (num_peers + 2) * c if kway else 3 * c * num_peers
        return total

    def destroy(self):
        self.synchronize()
        for cyc in self.cycles:
            if cyc.plan is not None:
                cyc.plan.destroy()
        if self.owns_streams:
            for s in self.streams:
                s.destroy()
