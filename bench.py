#!/usr/bin/env python3
"""Throughput of the fusion-buffer hot path on one MI355X.

One "step" is one pass of the hot path over one batch of synthetic gradients.
The headline workload is the fusion stress configuration: 1,024 fp32 tensors
with element counts log-uniform in [256, 65536] (seed 3), values U(-1,1)
(seed 4), packed into a 64 MiB fusion buffer with prescale 0.125 and unpacked
again.  Inputs are resident in HBM before the timed region starts.

Prints ONE JSON line.  `value` is algorithmic GB/s of the whole step
(pack = P_in + P_buf, unpack = P_buf + P_out); `roofline` prices the dominant
kernel (the scaled pack) against the 8 TB/s HBM peak from its average launch
duration measured with HIP events on the stream it runs on; `cpu_baseline` is
the CPU oracle (a restatement of the reference's CPU path) timed on one host
core over the same workload; `extra` carries the other pipelines (ResNet-50
cycle with a peer reduce, BERT-large fp16-compressed with 7 peers, Adasum,
GPT-2 XL streamed on two streams).
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0

# HBM bytes per launch of the scaled pack kernel on the headline workload, from rocprofv3
# FETCH_SIZE and WRITE_SIZE runs of `bench.py --kernel-only`, each scaled by what the same
# counter reads for a plain 256 MiB copy (`bench.py --calibrate`): FETCH_SIZE x 1.9544,
# WRITE_SIZE x 1.0000.  The summary with the commands is profiles/pack_kernel_fusion_stress.txt.
PACK_TRAFFIC_BYTES_MEASURED = 93204449


# One step of the headline is the fusion stress workload as the baseline configuration states it:
# 200 repetitions of pack + unpack over the 1,024 tensors.
REPS = 200


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20,
                    help="timed steps; one step is the workload's %d repetitions of pack + unpack" % REPS)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-extra", action="store_true", help="only the headline workload")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--kernel-only", nargs="?", const="pack", default=None,
                    choices=["pack", "reduce", "adasum"],
                    help="only launch one kernel family (for rocprofv3 runs): the scaled pack of the headline "
                         "workload (default), the fp32 reduce-sum of a 64 MiB buffer with one peer, or the "
                         "Adasum combine of 2 x 2^25 fp32 in 64 layers")
    ap.add_argument("--calibrate", action="store_true",
                    help="only launch a plain 256 MiB device copy (scales rocprofv3 byte counters)")
    ap.add_argument("--streams", type=int, default=2,
                    help="stream slots the headline steps alternate over, each with a fusion buffer of its own "
                         "(HOROVOD_NUM_NCCL_STREAMS); default 2, the configuration this library is meant to run "
                         "in; the one-stream figure is reported beside it")
    ap.add_argument("--replicas", type=int, default=8,
                    help="independent copies of the workload that steps rotate over, so that the "
                         "bytes touched between two uses of one copy exceed the 256 MB Infinity Cache")
    return ap.parse_args()


def timed(fn, sync, steps, warmup):
    """Wall time of `steps` calls of fn bracketed by synchronisation on both sides."""
    import torch
    for _ in range(warmup):
        fn()
    sync()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    sync()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def event_timed(fn, stream, steps, warmup):
    """Average stream time per call of fn, from HIP events recorded on `stream`."""
    from horovod_amd import Timer
    for _ in range(warmup):
        fn()
    stream.synchronize()
    t = Timer()
    t.start(stream)
    for _ in range(steps):
        fn()
    t.stop(stream)
    ms = t.elapsed_ms()
    t.destroy()
    return ms / steps * 1e-3


class DeviceSet:
    """Gradient tensors carved out of one device allocation at 256-byte aligned offsets."""

    def __init__(self, counts, elem_size, fill):
        import torch
        self.counts = counts
        self.es = elem_size
        offs, cur = [], 0
        for c in counts:
            offs.append(cur)
            cur += (c * elem_size + 255) // 256 * 256
        self.offs = offs
        self.nbytes = max(cur, 256)
        self.dev = fill(self.nbytes)
        torch.cuda.synchronize()
        self.ptrs = [self.dev.data_ptr() + o for o in offs]


def stress_workload(replicas):
    """Returns counts, the host image of the tensors, and `replicas` (src, dst) device sets."""
    import torch
    from horovod_amd import workloads as W
    counts = W.stress_counts(seed=3)
    rng = np.random.default_rng(4)
    host = np.zeros(sum((c * 4 + 255) // 256 * 256 for c in counts), np.uint8)
    off = 0
    for c in counts:
        host[off:off + 4 * c] = rng.uniform(-1, 1, c).astype(np.float32).view(np.uint8)
        off += (c * 4 + 255) // 256 * 256
    sets = []
    for _ in range(replicas):
        src = DeviceSet(counts, 4, lambda n: torch.from_numpy(host).cuda())
        dst = DeviceSet(counts, 4, lambda n: torch.zeros(n, dtype=torch.uint8, device="cuda"))
        sets.append((src, dst))
    return counts, host, sets


def cpu_baseline_stress(counts, host, budget_s=12.0):
    """The reference CPU sequence (ops/gloo_operations.cc:118-170) on one core:
    memcpy pack, in-place ScaleBuffer(0.125), memcpy unpack."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle_util
    from ctypes import c_double, c_int, c_int64, c_void_p
    orc = oracle_util.Oracle()
    L = orc.lib
    offs, cur = [], 0
    for c in counts:
        offs.append(cur)
        cur += (c * 4 + 255) // 256 * 256
    out = np.zeros_like(host)
    n = len(counts)
    tptr = (c_void_p * n)(*[host.ctypes.data + o for o in offs])
    optr = (c_void_p * n)(*[out.ctypes.data + o for o in offs])
    nb = np.array([4 * c for c in counts], np.int64)
    payload = int(nb.sum())
    buf = np.zeros(payload + 64, np.uint8)
    reps, t0 = 0, time.perf_counter()
    while True:
        L.orc_pack(tptr, c_void_p(nb.ctypes.data), c_int(n), c_void_p(buf.ctypes.data))
        L.orc_scale_buffer(c_void_p(buf.ctypes.data), c_void_p(buf.ctypes.data), c_int64(payload // 4),
                           c_double(0.125), c_int(oracle_util.F32))
        L.orc_unpack(c_void_p(buf.ctypes.data), optr, c_void_p(nb.ctypes.data), c_int(n))
        reps += 1
        dt = time.perf_counter() - t0
        if dt > budget_s:
            break
    gbs = 4 * payload * reps / dt / 1e9
    return {"value": round(gbs, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": "%d repetitions of the same 1,024-tensor workload (memcpy pack, in-place ScaleBuffer 0.125, "
                      "memcpy unpack; 4P algorithmic bytes each) in %.1f s; host has %d cores"
                      % (reps, dt, os.cpu_count())}


def cpu_extras(budget_s=2.5):
    """The CPU oracle on one core over bounded samples of the other pipelines, in the same
    algorithmic bytes as the GPU figures: the whole ResNet-50 set, one 42-tensor BERT-large cycle
    (cast and scale fused into the copy, which flatters the CPU), the whole Adasum pair, one
    GPT-2 XL layer.  Buffers are preallocated and every oracle call works in place."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle_util
    from ctypes import c_double, c_int, c_int64, c_void_p
    from oracle_util import F16, F32
    from horovod_amd import workloads as W
    L = oracle_util.Oracle().lib
    rng = np.random.default_rng(0)
    out = {}

    def P(a, off=0):
        return c_void_p(a.ctypes.data + off)

    def ptrs(arrays):
        return (c_void_p * len(arrays))(*[a.ctypes.data for a in arrays])

    def run(name, fn, nbytes):
        fn()
        reps, t0 = 0, time.perf_counter()
        while True:
            fn()
            reps += 1
            dt = time.perf_counter() - t0
            if dt > budget_s:
                break
        out[name] = {"cpu_GB/s": round(nbytes * reps / dt / 1e9, 2), "cores": 1, "reps": reps}

    # ResNet-50: memcpy pack, ScaleBuffer 0.125 in place, sum with one peer, memcpy unpack (7P)
    counts = [W.numel(s) for s in W.resnet50_shapes()]
    ts = [(rng.standard_normal(c, dtype=np.float32) * np.float32(1e-3)) for c in counts]
    outs = [np.empty_like(t) for t in ts]
    n, k = sum(counts), len(counts)
    nb = np.array([4 * c for c in counts], np.int64)
    buf = np.zeros(n, np.float32)
    peer = rng.standard_normal(n, dtype=np.float32)
    tp, op = ptrs(ts), ptrs(outs)

    def resnet():
        L.orc_pack(tp, P(nb), c_int(k), P(buf))
        L.orc_scale_buffer(P(buf), P(buf), c_int64(n), c_double(0.125), c_int(F32))
        L.orc_sum(P(peer), P(buf), c_int64(n), c_int(F32))
        L.orc_unpack(P(buf), op, P(nb), c_int(k))

    run("resnet50_fp32_pack_scale_reduce_unpack", resnet, 7 * 4 * n)

    # BERT-large, one cycle of 42 tensors: fp32 -> fp16 with prescale, 7 peers on 1/8, fp16 -> fp32
    counts = [W.numel(s) for s in W.bert_large_shapes()][7:49]
    ts = [(rng.standard_normal(c, dtype=np.float32) * np.float32(1e-4)) for c in counts]
    outs = [np.empty_like(t) for t in ts]
    n = sum(counts)
    hbuf = np.zeros(n, np.uint16)
    peers = [rng.integers(0, 0x0400, n // 8, dtype=np.uint16) for _ in range(7)]

    def bert():
        off = 0
        for t, c in zip(ts, counts):
            L.orc_scale_cast_f32_to_f16_f16c(P(t), P(hbuf, 2 * off), c_int64(c), c_double(0.125))
            off += c
        for p in peers:
            L.orc_float16_sum(P(p), P(hbuf), c_int64(n // 8))
        off = 0
        for o, c in zip(outs, counts):
            L.orc_scale_cast_f16_to_f32_f16c(P(hbuf, 2 * off), P(o), c_int64(c), c_double(1.0))
            off += c

    run("bert_large_fp32_to_fp16_7peers_eighth_chunk", bert, 6 * n + 9 * 2 * (n // 8) + 6 * n)

    # Adasum: the whole pair, in place on a (values stay finite from repetition to repetition)
    n = 1 << 25
    lc = np.array(W.adasum_layer_counts(n, 64, seed=13), np.int32)
    a = rng.standard_normal(n, dtype=np.float32)
    b = rng.standard_normal(n, dtype=np.float32)
    nd, co = np.zeros(192), np.zeros(128)
    run("adasum_fp32_2x32M_64layers",
        lambda: L.orc_adasum_pairwise(P(a), P(b), c_int(F32), P(lc), c_int(64), P(nd), P(co)), 5 * n * 4)

    # GPT-2 XL: one transformer layer (12 fp16 tensors, 61.5 MB)
    counts = [W.numel(s) for s in W.gpt2_xl_shapes()][2:14]
    ts = [rng.integers(0, 0x3c00, c, dtype=np.uint16) for c in counts]
    outs = [np.empty_like(t) for t in ts]
    n, k = sum(counts), len(counts)
    nb = np.array([2 * c for c in counts], np.int64)
    hbuf = np.zeros(n, np.uint16)
    peer = rng.integers(0, 0x3c00, n, dtype=np.uint16)
    tp2, op2 = ptrs(ts), ptrs(outs)

    def gpt2():
        L.orc_pack(tp2, P(nb), c_int(k), P(hbuf))
        L.orc_scale_buffer(P(hbuf), P(hbuf), c_int64(n), c_double(0.125), c_int(F16))
        L.orc_float16_sum(P(peer), P(hbuf), c_int64(n))
        L.orc_unpack(P(hbuf), op2, P(nb), c_int(k))

    run("gpt2_xl_fp16_two_streams", gpt2, 7 * 2 * n)
    return out


def per_tensor_comparator(counts, src, dst, reps=20):
    """The fusion stress step through the C++ adapter's GPUAllreduce::Execute twice: with the
    offset-table kernels, and with one hipMemcpyAsync per tensor each way plus a whole-buffer
    ScaleBuffer (HOROVOD_BATCH_D2D_MEMCOPIES=0, what Horovod does on ROCm today,
    ops/gpu_operations.cc:209-222,230-235,327-332).  Both include the op's completion wait."""
    import ctypes
    import torch
    lib = ctypes.CDLL(os.path.join(ROOT, "horovod_amd", "lib", "libhvdhip_adapter.so"))
    lib.hvd_adapter_create.restype = ctypes.c_void_p
    lib.hvd_adapter_create.argtypes = [ctypes.c_int] * 4 + [ctypes.c_void_p]
    lib.hvd_adapter_destroy.argtypes = [ctypes.c_void_p]
    lib.hvd_adapter_allreduce.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                          ctypes.c_int, ctypes.c_int, ctypes.c_double, ctypes.c_double,
                                          ctypes.c_void_p, ctypes.c_int, ctypes.c_char_p, ctypes.c_size_t]
    n = len(counts)
    fb = torch.empty(64 << 20, dtype=torch.uint8, device="cuda")
    fbs = (ctypes.c_void_p * 1)(fb.data_ptr())
    tp = (ctypes.c_void_p * n)(*src.ptrs)
    op = (ctypes.c_void_p * n)(*dst.ptrs)
    cnt = (ctypes.c_int64 * n)(*counts)
    err = ctypes.create_string_buffer(512)
    out = {}
    for name, batch in (("offset_table_kernels_ms", 1), ("per_tensor_copies_ms", 0)):
        h = lib.hvd_adapter_create(1, batch, 0, 0, fbs)
        for _ in range(3):
            rc = lib.hvd_adapter_allreduce(h, tp, op, cnt, n, 7, 0.125, 1.0, None, 0, err, 512)
            if rc != 0:
                raise RuntimeError(err.value.decode())
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            lib.hvd_adapter_allreduce(h, tp, op, cnt, n, 7, 0.125, 1.0, None, 0, err, 512)
        torch.cuda.synchronize()
        out[name] = round((time.perf_counter() - t0) / reps * 1e3, 4)
        lib.hvd_adapter_destroy(h)
    out["speedup"] = round(out["per_tensor_copies_ms"] / out["offset_table_kernels_ms"], 1)
    return out


_PAIR = []


def stream_pair():
    """Two library streams created once, before any other, and shared by everything in this run
    that alternates over stream slots: streams that are created later, while others exist, can
    land on a hardware queue that is already in use and then overlap nothing."""
    if not _PAIR:
        from horovod_amd import Stream
        _PAIR.extend([Stream(), Stream()])
    return _PAIR


def extras(steps, warmup):
    """The other pipelines, each as algorithmic GB/s and fraction of the HBM peak."""
    import torch
    from horovod_amd import AdasumPlan, DTYPE, Stream, workloads as W
    from horovod_amd.pipeline import AllreducePipeline
    out = {}
    g = torch.Generator(device="cuda")

    def randn(nbytes, dtype, std, seed):
        g.manual_seed(seed)
        n = nbytes // torch.empty(0, dtype=dtype).element_size()
        return (torch.randn(n, generator=g, device="cuda", dtype=torch.float32) * std).to(dtype).view(torch.uint8)

    def run_pipeline(name, shapes, tdtype, bdtype, std, peers, fraction, streams, kway=True, steps_=steps,
                     replicas=1):
        tt = {DTYPE["float32"]: torch.float32, DTYPE["float16"]: torch.float16}
        es = 4 if tdtype == DTYPE["float32"] else 2
        counts = [W.numel(s) for s in shapes]
        reps = []
        shared = stream_pair()[:streams]  # every replica queues on the same stream(s)
        for r in range(replicas):
            src = DeviceSet(counts, es, lambda n: randn(n, tt[tdtype], std, 1 + r))
            dst = DeviceSet(counts, es, lambda n: torch.zeros(n, dtype=torch.uint8, device="cuda"))
            pipe = AllreducePipeline(src.ptrs, dst.ptrs, counts, tdtype, bdtype, streams=shared)
            bs = 4 if pipe.buffer_dtype == DTYPE["float32"] else 2
            max_elems = max(c.buffer_elems for c in pipe.cycles)
            peer_bufs = []
            for p in range(peers):
                nb = int(max_elems * fraction) * bs + 256
                peer_bufs.append(randn((nb + 255) // 256 * 256, tt[pipe.buffer_dtype], std, 100 + 16 * r + p))
            reps.append((src, dst, pipe, peer_bufs))
        torch.cuda.synchronize()
        turn = [0]

        def fn():
            i = turn[0] = (turn[0] + 1) % len(reps)
            _, _, pipe, peer_bufs = reps[i]
            pipe.run(0.125, 1.0, (lambda ci, p: peer_bufs[p].data_ptr()) if peers else None, peers, fraction, kway)

        def sync():
            for _, _, pipe, _ in reps:
                pipe.synchronize()

        sec = timed(fn, sync, steps_, max(2, warmup // 4))
        pipe = reps[0][2]
        ab = pipe.algorithmic_bytes(peers, fraction, kway)
        out[name] = {"GB/s": round(ab / sec / 1e9, 1), "frac_of_hbm_peak": round(ab / sec / 1e9 / HBM_PEAK_GBS, 4),
                     "ms": round(sec * 1e3, 4), "algorithmic_MB": round(ab / 1e6, 1), "cycles": len(pipe.cycles),
                     "streams": streams, "peers": peers, "reduce": "k-way" if kway else "per-peer",
                     "completion_event_per_cycle": pipe.completion_events,
                     "replicas_rotated": replicas}
        for _, _, pipe, _ in reps:
            pipe.destroy()
        del reps
        torch.cuda.empty_cache()

    F32, F16 = DTYPE["float32"], DTYPE["float16"]
    run_pipeline("resnet50_fp32_pack_scale_reduce_unpack", W.resnet50_shapes(), F32, F32, 1e-3, 1, 1.0, 1,
                 replicas=4)
    run_pipeline("resnet50_fp32_two_streams", W.resnet50_shapes(), F32, F32, 1e-3, 1, 1.0, 2, replicas=4)
    run_pipeline("bert_large_fp32_to_fp16_7peers_eighth_chunk", W.bert_large_shapes(), F32, F16, 1e-4, 7, 0.125, 1,
                 steps_=max(5, steps // 10))
    run_pipeline("bert_large_fp32_to_fp16_two_streams", W.bert_large_shapes(), F32, F16, 1e-4, 7, 0.125, 2,
                 steps_=max(5, steps // 10))
    run_pipeline("gpt2_xl_fp16_two_streams", W.gpt2_xl_shapes(), F16, F16, 1e-3, 1, 1.0, 2,
                 steps_=max(3, steps // 40))

    # Adasum combine: two fp32 vectors of 2^25 elements, 64 layers, per-layer correlation 0.3;
    # four independent pairs are rotated so that no pair is still cached when its turn comes again
    n = 1 << 25
    counts = W.adasum_layer_counts(n, 64, seed=13)
    pairs = []
    for r in range(4):
        g.manual_seed(14 + 2 * r)
        a = torch.randn(n, generator=g, device="cuda", dtype=torch.float32)
        g.manual_seed(15 + 2 * r)
        b = 0.3 * a + (1 - 0.09) ** 0.5 * torch.randn(n, generator=g, device="cuda", dtype=torch.float32)
        pairs.append((a, b))
    plan = AdasumPlan(counts, F32)
    s = stream_pair()[0]
    torch.cuda.synchronize()
    turn = [0]

    def combine():
        # the combine rewrites a; its cost does not depend on the values, which stay finite
        i = turn[0] = (turn[0] + 1) % len(pairs)
        plan.combine(pairs[i][0].data_ptr(), pairs[i][1].data_ptr(), s)

    sec = event_timed(combine, s, max(8, steps // 4), 4)
    ab = 5 * n * 4
    out["adasum_fp32_2x32M_64layers"] = {"GB/s": round(ab / sec / 1e9, 1),
                                         "frac_of_hbm_peak": round(ab / sec / 1e9 / HBM_PEAK_GBS, 4),
                                         "ms": round(sec * 1e3, 4), "algorithmic_MB": round(ab / 1e6, 1),
                                         "replicas_rotated": len(pairs)}
    plan.destroy()
    del pairs
    torch.cuda.empty_cache()

    # Allgather fusion buffer (ops/collective_operations.cc:234-288): 8 ranks, 128 entries per rank with
    # the stress workload's size mix.  This GPU packs its own slab at its displacement (the other
    # slabs arrive by the collective, which is not built) and unpacks one component per (entry, rank).
    # Each direction is one batched copy; 4 independent sets are rotated.
    import ctypes
    import horovod_amd
    world, es = 8, 4
    counts = W.stress_counts(seed=21, n=128)
    slab = es * sum(counts)
    sets = []
    for r in range(4):
        src = DeviceSet(counts, es, lambda n: randn(n, torch.float32, 1.0, 60 + r))
        fusion = torch.empty(world * slab, dtype=torch.uint8, device="cuda")
        outs = [torch.empty(world * c * es, dtype=torch.uint8, device="cuda") for c in counts]
        pack_dst, at = [], 3 * slab  # this rank's displacement (rank 3 of 8)
        for c in counts:
            pack_dst.append(fusion.data_ptr() + at)
            at += c * es
        un_dst, un_src, un_sz = [], [], []
        for rank in range(world):
            at = rank * slab
            for i, c in enumerate(counts):
                un_dst.append(outs[i].data_ptr() + rank * c * es)
                un_src.append(fusion.data_ptr() + at)
                un_sz.append(c * es)
                at += c * es
        # the descriptor arrays as the C caller holds them, built once
        VP, SZ = ctypes.c_void_p, ctypes.c_size_t
        pack_args = ((VP * len(counts))(*pack_dst), (VP * len(counts))(*src.ptrs),
                     (SZ * len(counts))(*[c * es for c in counts]), len(counts))
        un_args = ((VP * len(un_dst))(*un_dst), (VP * len(un_dst))(*un_src), (SZ * len(un_dst))(*un_sz), len(un_dst))
        sets.append((src, fusion, outs, pack_args, un_args))
    torch.cuda.synchronize()
    copy = horovod_amd.lib().hvdhip_batched_d2d_memcpy

    def gather_step():
        i = turn[0] = (turn[0] + 1) % len(sets)
        horovod_amd.check(copy(*sets[i][3], s.handle), "hvdhip_batched_d2d_memcpy")
        horovod_amd.check(copy(*sets[i][4], s.handle), "hvdhip_batched_d2d_memcpy")

    sec = event_timed(gather_step, s, max(8, steps // 4), 4)
    ab = 2 * slab + 2 * world * slab
    out["allgather_fusion_8ranks_pack_unpack"] = {
        "GB/s": round(ab / sec / 1e9, 1), "frac_of_hbm_peak": round(ab / sec / 1e9 / HBM_PEAK_GBS, 4),
        "ms": round(sec * 1e3, 4), "algorithmic_MB": round(ab / 1e6, 1), "entries": len(counts), "ranks": world,
        "copies_per_step": len(counts) * (world + 1), "streams": 1, "replicas_rotated": len(sets)}
    del sets
    return out


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU's share of the hot path: this build has no inter-GPU collectives, "
              "run it with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    import horovod_amd
    from horovod_amd import DTYPE, FusionPlan, Stream
    from horovod_amd import build as native
    native.ensure_built()  # loads what is built; builds only if nothing is
    horovod_amd.lib()  # fails loudly if the HIP library cannot be loaded

    stream = stream_pair()[0]
    F32 = DTYPE["float32"]
    if args.calibrate:
        from horovod_amd import host as H
        n = 256 << 20
        a = torch.zeros(n, dtype=torch.uint8, device="cuda")
        b = torch.empty(n, dtype=torch.uint8, device="cuda")
        torch.cuda.synchronize()
        for _ in range(args.warmup + args.steps):
            H.batched_d2d_memcpy([b.data_ptr()], [a.data_ptr()], [n], stream)
        stream.synchronize()
        return

    if args.kernel_only in ("reduce", "adasum"):
        from horovod_amd import AdasumPlan, host as H, workloads as W
        g = torch.Generator(device="cuda")
        g.manual_seed(7)
        n = (64 << 20) // 4 if args.kernel_only == "reduce" else 1 << 25
        pairs = [(torch.randn(n, generator=g, device="cuda"), torch.randn(n, generator=g, device="cuda"))
                 for _ in range(4)]
        plan = AdasumPlan(W.adasum_layer_counts(n, 64, seed=13), F32) if args.kernel_only == "adasum" else None
        torch.cuda.synchronize()
        for i in range(args.warmup + args.steps):
            a, b = pairs[i % 4]
            if plan is None:
                H.reduce_sum(a.data_ptr(), b.data_ptr(), n, F32, stream)
            else:
                plan.combine(a.data_ptr(), b.data_ptr(), stream)
        stream.synchronize()
        return

    counts, host, sets = stress_workload(max(1, args.replicas))
    plans = [FusionPlan(src.ptrs, dst.ptrs, counts, F32) for src, dst in sets]
    # One fusion buffer per stream slot, reused by every repetition: Horovod's FusionBufferManager keeps
    # one per (device, framework, stream slot) for the life of the job (ops/gpu_operations.cc:122-124).
    # The gradient tensors on either side of it rotate over the replicas.
    fbs = [torch.empty(plans[0].buffer_len, dtype=torch.uint8, device="cuda") for _ in range(2)]
    plan = plans[0]
    payload = 4 * sum(counts)
    torch.cuda.synchronize()
    turn = [0]

    def pack():
        i = turn[0] = (turn[0] + 1) % len(plans)
        plans[i].pack(fbs[0].data_ptr(), 0.125, stream)

    if args.streams not in (1, 2):
        print("bench.py alternates over one or two stream slots", file=sys.stderr)
        sys.exit(2)
    slots = stream_pair()[:args.streams]

    def step():
        for _ in range(REPS):
            i = turn[0] = (turn[0] + 1) % len(plans)
            plans[i].pack(fbs[i % len(slots)].data_ptr(), 0.125, slots[i % len(slots)])
            plans[i].unpack(fbs[i % len(slots)].data_ptr(), 1.0, slots[i % len(slots)])

    def sync_slots():
        for st in slots:
            st.synchronize()

    if args.kernel_only:
        for _ in range(args.warmup + args.steps):
            pack()
        stream.synchronize()
        return

    sec = timed(step, sync_slots, args.steps, args.warmup)
    value = REPS * 4 * payload / sec / 1e9

    ksec = event_timed(pack, stream, 200, 20)
    achieved = 2 * payload / ksec / 1e9
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": PACK_TRAFFIC_BYTES_MEASURED,
                "kernel": "xfer_k<Scale<float,float>, pack, write-through stores>", "launch_us": round(ksec * 1e6, 2),
                "timed": "launched back to back on one stream: tensors of another replica every launch, "
                         "the stream slot's one fusion buffer as the destination",
                "algorithmic_bytes_per_launch": 2 * payload, "workgroups": plan.num_chunks}

    result = {
        "metric": "achieved HBM GB/s (% of 8 TB/s) for fused pack+scale+reduce+unpack; Adasum GB/s",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(sec * 1e3, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "fusion stress: 1,024 fp32 tensors, log-uniform 256..65,536 elements (seed 3), "
                               "U(-1,1) (seed 4); pack with prescale 0.125 into the fusion buffer, unpack, 200 repetitions; "
                               "consecutive repetitions alternate over the stream slots, each slot with its own persistent "
                               "fusion buffer (as FusionBufferManager keeps them); the tensors rotate over the replicas",
                   "tensors": len(counts), "payload_bytes": payload, "buffer_len": plan.buffer_len,
                   "repetitions_per_step": REPS, "algorithmic_bytes_per_step": REPS * 4 * payload,
                   "replicas_rotated": len(plans),
                   "streams": len(slots)},
        "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4),
        "roofline": roofline,
    }
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline_stress(counts, host)
    other = None
    if not args.no_extra:
        # The same steps with the other stream count: all on one stream when the headline alternates over
        # several (every kernel then waits for its predecessor, the reference's default
        # HOROVOD_NUM_NCCL_STREAMS=1), or on two streams when the headline was asked to use one.
        try:
            alt = stream_pair()[:1 if len(slots) > 1 else 2]

            def step_alt():
                for _ in range(REPS):
                    i = turn[0] = (turn[0] + 1) % len(plans)
                    plans[i].pack(fbs[i % len(alt)].data_ptr(), 0.125, alt[i % len(alt)])
                    plans[i].unpack(fbs[i % len(alt)].data_ptr(), 1.0, alt[i % len(alt)])

            def sync_alt():
                for st in alt:
                    st.synchronize()

            sec2 = timed(step_alt, sync_alt, args.steps, args.warmup)
            other = {"GB/s": round(REPS * 4 * payload / sec2 / 1e9, 1),
                     "frac_of_hbm_peak": round(REPS * 4 * payload / sec2 / 1e9 / HBM_PEAK_GBS, 4),
                     "ms_per_step": round(sec2 * 1e3, 5), "streams": len(alt)}
        except Exception as e:  # pragma: no cover
            other = {"error": "%s: %s" % (type(e).__name__, e)}
    comparator = None
    if not args.no_extra:
        try:
            comparator = per_tensor_comparator(counts, sets[0][0], sets[0][1])
        except Exception as e:  # pragma: no cover
            comparator = {"error": "%s: %s" % (type(e).__name__, e)}
    for p in plans:
        p.destroy()
    del fbs, sets
    torch.cuda.empty_cache()
    if not args.no_extra:
        # the extra pipelines must never cost the headline line
        try:
            result["extra"] = extras(200, 20)
        except Exception as e:  # pragma: no cover
            result["extra"] = {"error": "%s: %s" % (type(e).__name__, e)}
        result["extra"]["fusion_stress_execute_vs_per_tensor_copies"] = comparator
        result["extra"]["fusion_stress_one_stream" if len(slots) > 1 else "fusion_stress_two_streams"] = other
        if not args.no_cpu and "error" not in result["extra"]:
            try:
                for name, v in cpu_extras().items():
                    result["extra"][name].update({"cpu_GB/s": v["cpu_GB/s"], "cpu_cores": 1,
                                                  "cpu_sample_reps": v["reps"]})
            except Exception as e:  # pragma: no cover
                result["extra"]["cpu_error"] = "%s: %s" % (type(e).__name__, e)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
