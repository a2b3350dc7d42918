#!/usr/bin/env python3
"""Throughput of the fusion-buffer hot path on one MI355X.

The headline workload is the pipeline the metric names, on the ResNet-50 configuration: 161 fp32
gradient tensors (25,557,032 elements, N(0, 1e-3)), fused by the reference's planner into two
cycles of at most 64 MiB; per cycle a pack with prescale 0.125 into the fusion buffer, the
reduce-sum of the buffer with one peer buffer resident on the same device, and the unpack
(postscale 1.0) -- the sequence of NCCLAllreduce::Execute (ops/nccl_operations.cc:156-214) with
the collective replaced by the local sum.  One "step" is REPS passes of that pipeline over
tensor sets that rotate so that no pass finds its inputs in the 256 MB Infinity Cache.  Inputs
are resident in HBM before the timed region starts; everything runs on one stream.

Prints ONE JSON line on stdout, small enough for a reader who keeps the last 8 KB: the contract's keys
in full, every other configuration as one row per pipeline and one row per kernel loop.  The same
results with the description of what each figure timed go to stderr as one line that begins with
"DETAIL ".  `value` is ALGORITHMIC GB/s of the whole step (pack = P_in + P_buf, reduce = (k+2) C,
unpack = P_buf + P_out; the bytes a pipeline must move with the fusion buffer materialised on both
sides of the collective) -- not an HBM counter: inside a cycle the fusion buffer is handed from
kernel to kernel through the Infinity Cache, so a pipeline's algorithmic rate can exceed what any
one of its kernels streams out of HBM (`value_kind` says so; `hbm_GB/s` is the counter-derived HBM
rate of the roofline kernel).  `ms_per_step` is the wall-clock mean of the K timed steps;
`ms_per_step_median_min_max` comes from a HIP event pair around each step on the pipeline's stream.
The HBM claim is `roofline`: the dominant kernel of the workload launched back to back on rotating
buffers, algorithmic bytes per launch over its launch time from HIP events on its stream (mean over
ten batches of launches, with median / min / max of the batches), against the 8 TB/s peak.
`roofline.traffic` (HBM bytes per launch) is measured in the same run: before it touches the GPU
itself the benchmark starts four rocprofv3 child runs (FETCH_SIZE and WRITE_SIZE over the headline's
kernel loops and over the calibration copies) and scales the counters; if that cannot be done
(no rocprofv3, the run is itself under a profiler, `--no-live-traffic`) the figure of the committed
profile stands in and `roofline.traffic_from` says so.
`cpu_baseline` is the CPU oracle (a restatement of the reference's CPU path) on one host core over
the same workload.  `extra` carries the other configurations: C1-C5 pipelines on one and two
streams, C1 and C5 once more through the C++ adapter's GPUAllreduce::Execute with its finalizer
threads, the allgather buffer's copies, the device's own 1 GiB copy rates, and one row per kernel
loop (an unpack's `in_pipeline_us` is its time right behind the reduce-sum that wrote its buffer).

`--kernel-only <config>` runs exactly the back-to-back kernel loops of one configuration and
nothing else, for rocprofv3 (the summaries under profiles/ come from these runs); `--calibrate`
launches two plain 256 MiB copies that are not the library's kernels, whose known byte counts scale
the profiler's FETCH_SIZE and WRITE_SIZE counters.
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

# One step of the headline = this many passes of the two-cycle ResNet-50 pipeline (a pass takes
# about 0.11 ms; a step of 50 passes keeps even a short run measuring the device, not the host's
# wake-up after the final synchronisation).
REPS = 50

# Independent copies of a configuration's buffers that launches rotate over.
ROTATE = 6

# HBM bytes per launch, per kernel of the --kernel-only loops, from rocprofv3 FETCH_SIZE and
# WRITE_SIZE runs (KiB per dispatch), each scaled by what the same counter reads for two plain
# 256 MiB device copies of known size that are not the library's own kernels
# (`bench.py --calibrate`).  The summaries with the commands are the files named here under
# profiles/; tests/test_host_logic.py re-derives every figure from them.  A default run measures the
# headline configuration's own figures again (live_traffic) and overwrites those entries.
TRAFFIC_BYTES_MEASURED = {
    "ag.pack": 138114304,
    "ag.pack_small": 12592616,
    "ag.unpack": 1097172458,
    "ag.unpack_small": 99925726,
    "c1.pack": 126061655,
    "c1.pack_rotating_destination": 126060918,
    "c1.reduce": 187599846,
    "c1.reduce+unpack": 313670934,
    "c1.unpack": 126053086,
    "c2.pack": 93545897,
    "c2.unpack": 92911342,
    "c3.pack": 196398853,
    "c3.reduce": 73234670,
    "c3.reduce_8MiB_apart": 73234301,
    "c3.unpack": 197359055,
    "c3.unpack_postscale4": 197372951,
    "c4.combine": 674533614,
    "c4h.combine": 337240035,
    "c5.pack": 123955137,
    "c5.reduce": 184445164,
    "c5.reduce+unpack": 308444437,
    "c5.reduce_single": 482447512,
    "c5.scale_single": 321694896,
    "c5.unpack": 123958579,
    "copy.library": 2164285318,
    "copy.runtime": 2147400151,
    "copy.torch": 2147400909,
}
# Kernel-trace duration (ns) of an unpack launched right behind the reduce-sum that wrote its buffer (the
# `<config>.reduce+unpack` loops), from the same summaries: what the unpack takes in a cycle, where its
# input comes out of the Infinity Cache.  HIP events cannot single it out without getting between the two
# kernels, so the figure is carried from the profile and pinned by the same test.
IN_PIPELINE_NS_MEASURED = {
    "c1.unpack": 18104.4,
    "c5.unpack": 18005.2,
}
TRAFFIC_PROFILE = {
    "c1": "profiles/c1_resnet50_fp32_kernels.txt",
    "c2": "profiles/c2_fusion_stress_kernels.txt",
    "c3": "profiles/c3_bert_large_fp16_kernels.txt",
    "c4": "profiles/c4_adasum_fp32_kernels.txt",
    "c5": "profiles/c5_gpt2_xl_fp16_kernels.txt",
    "copy": "profiles/device_copy_1GiB_three_ways.txt",
    "ag": "profiles/ag_allgather_kernels.txt",
}

CONFIGS = ("c1", "c2", "c3", "c4", "c5")
KERNEL_ONLY = CONFIGS + ("c4h", "copy", "ag")


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20,
                    help="timed steps; one step is %d passes of the ResNet-50 pipeline" % REPS)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-extra", action="store_true", help="only the headline workload")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baselines")
    ap.add_argument("--kernel-only", choices=KERNEL_ONLY, default=None,
                    help="only the back-to-back kernel loops of one configuration (for rocprofv3 runs): c1 ResNet-50 "
                         "fp32 cycle, c2 fusion stress, c3 BERT-large fp32->fp16 cycle with 7 peers on the 1/8 share, "
                         "c4 Adasum 2 x 2^25 fp32, c4h the same in fp16, c5 GPT-2 XL fp16 cycle and embedding, copy 1 GiB moved by the "
                         "library's kernel, by hipMemcpyAsync and by an elementwise kernel of torch, ag the allgather "
                         "fusion buffer's pack and unpack (8 ranks x 128 entries) at a 6 MB and at a 66 MB slab; "
                         "--steps launches per kernel after --warmup")
    ap.add_argument("--no-live-traffic", action="store_true",
                    help="take roofline.traffic from the committed profile instead of measuring it in this run with "
                         "rocprofv3 child processes")
    ap.add_argument("--calibrate", action="store_true",
                    help="only launch a plain 256 MiB device copy (scales rocprofv3 byte counters)")
    return ap.parse_args()


# ----------------------------------------------------------------------------------------------
# timing
# ----------------------------------------------------------------------------------------------

def timed(fn, sync, steps, warmup, stream=None):
    """Wall time of `steps` calls of fn bracketed by synchronisation on both sides.  With `stream`
    (everything fn queues goes onto that one stream) every call is bracketed by a HIP event pair on
    it as well, and the per-call stream times come back as a second value: (seconds per call,
    [seconds of each call] or None)."""
    import torch
    from horovod_amd import Timer
    for _ in range(warmup):
        fn()
    sync()
    torch.cuda.synchronize()
    timers = [Timer() for _ in range(steps)] if stream is not None else []
    t0 = time.perf_counter()
    for i in range(steps):
        if timers:
            timers[i].start(stream)
        fn()
        if timers:
            timers[i].stop(stream)
    sync()
    torch.cuda.synchronize()
    sec = (time.perf_counter() - t0) / steps
    each = [t.elapsed_ms() * 1e-3 for t in timers] or None
    for t in timers:
        t.destroy()
    return sec, each


def spread(values, scale=1.0, digits=4):
    """[median, min, max] of a list of times."""
    v = sorted(values)
    n = len(v)
    med = v[n // 2] if n % 2 else 0.5 * (v[n // 2 - 1] + v[n // 2])
    return [round(med * scale, digits), round(v[0] * scale, digits), round(v[-1] * scale, digits)]


def event_timed(fn, stream, steps, warmup, batches=10):
    """Stream time per call of fn from HIP events recorded on `stream`: the launches go out in
    `batches` runs, each bracketed by an event pair (an event per launch would put its own
    2-3 us between the kernels).  Returns (mean seconds per call over all batches,
    [mean seconds per call of each batch])."""
    from horovod_amd import Timer
    for _ in range(warmup):
        fn()
    stream.synchronize()
    batches = max(1, min(batches, steps))
    per = max(1, steps // batches)
    timers = [Timer() for _ in range(batches)]
    for t in timers:
        t.start(stream)
        for _ in range(per):
            fn()
        t.stop(stream)
    each = [t.elapsed_ms() * 1e-3 / per for t in timers]
    for t in timers:
        t.destroy()
    return sum(each) / len(each), each


def timed_batches(fn, sync, steps, warmup, batches=5):
    """Wall time per call of fn over `batches` runs, each bracketed by synchronisation (for pipelines
    that spread over two streams, where no single stream's events bracket a call).  Returns (mean
    seconds per call, [mean seconds per call of each batch])."""
    import torch
    for _ in range(warmup):
        fn()
    sync()
    torch.cuda.synchronize()
    batches = max(1, min(batches, steps))
    per = max(1, steps // batches)
    each = []
    for _ in range(batches):
        t0 = time.perf_counter()
        for _ in range(per):
            fn()
        sync()
        torch.cuda.synchronize()
        each.append((time.perf_counter() - t0) / per)
    return sum(each) / len(each), each


_PAIR = []


def stream_pair():
    """Two library streams created once, before any other, and shared by everything in this run:
    streams that are created later, while others exist, can land on a hardware queue that is
    already in use and then overlap nothing."""
    if not _PAIR:
        from horovod_amd import Stream
        _PAIR.extend([Stream(), Stream()])
    return _PAIR


# ----------------------------------------------------------------------------------------------
# device data
# ----------------------------------------------------------------------------------------------

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


_GEN = []


def randn_bytes(nbytes, dtype, std, seed):
    """nbytes of N(0, std) values of torch dtype `dtype`, as a uint8 device tensor."""
    import torch
    if not _GEN:
        _GEN.append(torch.Generator(device="cuda"))
    g = _GEN[0]
    g.manual_seed(seed)
    n = nbytes // torch.empty(0, dtype=dtype).element_size()
    return (torch.randn(n, generator=g, device="cuda", dtype=torch.float32) * std).to(dtype).view(torch.uint8)


def zeros_bytes(nbytes):
    import torch
    return torch.zeros(nbytes, dtype=torch.uint8, device="cuda")


def torch_dtype(dtype):
    import torch
    from horovod_amd import DTYPE
    return {DTYPE["float32"]: torch.float32, DTYPE["float16"]: torch.float16}[dtype]


# ----------------------------------------------------------------------------------------------
# kernel loops: every kernel family of a configuration, launched back to back on rotating buffers
# ----------------------------------------------------------------------------------------------

class Case:
    """One kernel at one grid.  fn() queues one launch on `stream` (the next rotating buffer set
    every call); alg = algorithmic bytes per launch; kernel = its name as a profiler prints it
    (template arguments: ..., 0 pack / 1 unpack, 0 non-temporal / 1 write-through stores).
    parts: for a call that launches several kernels, [(kernel, algorithmic bytes, algorithmic bytes read)] per
    kernel; reads: the algorithmic bytes read of a single-kernel call when that is not half of alg."""

    def __init__(self, key, kernel, fn, alg, what, workgroups=None, cleanup=None, parts=None, reads=None):
        self.key, self.kernel, self.fn, self.alg, self.what, self.workgroups = key, kernel, fn, alg, what, workgroups
        self.cleanup = cleanup  # destroys the plans behind fn (the closures hold the device memory)
        # per kernel of the call: (name, algorithmic bytes, of which read); a copy reads half of what it moves
        self.parts = parts or [(kernel, alg, alg // 2 if reads is None else reads)]


def cycle_cases(cfg, counts, tdtype, bdtype, std, peers, share_world, stream, pack_kernel, reduce_kernel,
                unpack_kernel, seed0, extra_postscale=None, pack_rotating=False):
    """Pack, reduce-sum and unpack of ONE fusion cycle, each launched back to back:
    pack reads another replica's tensors every launch and writes the slot's one fusion buffer (as the
    reference keeps one per stream slot); the reduce-sum and the unpack rotate over ROTATE buffers."""
    import torch
    from horovod_amd import FusionPlan, dtype_size, host as H, workloads as W
    ts, bs = dtype_size(tdtype), dtype_size(bdtype)
    tt, bt = torch_dtype(tdtype), torch_dtype(bdtype)
    sets = []
    for r in range(ROTATE):
        src = DeviceSet(counts, ts, lambda n: randn_bytes(n, tt, std, seed0 + r))
        dst = DeviceSet(counts, ts, zeros_bytes)
        sets.append((src, dst, FusionPlan(src.ptrs, dst.ptrs, counts, tdtype, bdtype)))
    plan0 = sets[0][2]
    blen = plan0.buffer_len
    nelem = blen // bs
    share = nelem if share_world == 1 else W.reduce_scatter_share(nelem, share_world)
    slack = 4096 * bs
    fb_pack = zeros_bytes(blen + slack)
    # The rotating fusion buffers and peer chunks lie back to back (256-byte aligned) in one allocation,
    # like the chunks of a staging buffer.  Buffers allocated one by one land wherever the driver finds
    # physical pages, and the same kernel then measures 4 % apart from process to process (the ResNet-50
    # reduce-sum: 29.5 or 30.8 us); and where they lie relative to each other matters to the memory
    # controllers: the 7-peer sum of an 8 MiB share takes 12.3-12.4 us with its eight chunks back to back
    # (8,135,424 bytes apart), 9 MiB or 8 MiB + 4 KiB apart, and 13.2-13.7 us with them exactly 8 or 16 MiB
    # (or 8 MiB + 16 or 64 KiB) apart.
    step = 256
    fb_bytes = (blen + slack + step - 1) // step * step
    peer_bytes = (share * bs + step - 1) // step * step
    arena = randn_bytes(ROTATE * (fb_bytes + peers * peer_bytes), bt, std, seed0 + 50)
    fbs = [arena[r * fb_bytes:(r + 1) * fb_bytes] for r in range(ROTATE)]
    at = ROTATE * fb_bytes
    peer_bufs = [[arena[at + (r * peers + p) * peer_bytes:at + (r * peers + p + 1) * peer_bytes] for p in range(peers)]
                 for r in range(ROTATE)]
    torch.cuda.synchronize()
    payload = sum(counts)
    turn = [0]

    def rot():
        turn[0] = (turn[0] + 1) % ROTATE
        return turn[0]

    def pack():
        sets[rot()][2].pack(fb_pack.data_ptr(), 0.125, stream)

    def pack_rotating_destination():
        i = rot()
        sets[i][2].pack(fbs[i].data_ptr(), 0.125, stream)

    def reduce():
        i = rot()
        H.reduce_sum_k(fbs[i].data_ptr(), [p.data_ptr() for p in peer_bufs[i]], share, bdtype, stream)

    def unpack():
        i = rot()
        sets[i][2].unpack(fbs[i].data_ptr(), 1.0, stream)

    def unpack_scaled():
        i = rot()
        sets[i][2].unpack(fbs[i].data_ptr(), extra_postscale, stream)

    def reduce_then_unpack():
        # the drop-in's order: the collective has just written the buffer (through the Infinity Cache)
        # when the unpack reads it
        i = rot()
        H.reduce_sum_k(fbs[i].data_ptr(), [p.data_ptr() for p in peer_bufs[i]], share, bdtype, stream)
        sets[i][2].unpack(fbs[i].data_ptr(), 1.0, stream)

    def cleanup():
        for _, _, plan in sets:
            plan.destroy()

    tile = 4096 // bs
    cases = [
        Case(cfg + ".pack", pack_kernel, pack, payload * (ts + bs),
             "pack with prescale 0.125 of %d tensors (%d payload bytes in, %d in the buffer); tensors of another replica "
             "every launch, the slot's one fusion buffer as destination" % (len(counts), payload * ts, payload * bs),
             plan0.num_chunks, cleanup, reads=payload * ts),
        Case(cfg + ".reduce", reduce_kernel, reduce, (peers + 2) * share * bs,
             "resident chunk of %d bytes += %d peer chunk(s) in one pass; %d (resident, peers) sets rotated"
             % (share * bs, peers, ROTATE), (share + tile - 1) // tile, reads=(peers + 1) * share * bs),
        Case(cfg + ".unpack", unpack_kernel, unpack, payload * (bs + ts),
             "unpack (postscale 1.0) of the same tensors; fusion buffer and outputs of another replica every launch",
             plan0.num_chunks, reads=payload * bs),
    ]
    if pack_rotating:
        cases.append(Case(cfg + ".pack_rotating_destination", pack_kernel, pack_rotating_destination, payload * (ts + bs),
                          "the same pack into a different fusion buffer every launch (%d rotated): what the pack takes when "
                          "its destination, like the unpack's, is not resident in the Infinity Cache" % ROTATE,
                          plan0.num_chunks, reads=payload * ts))
    if extra_postscale is not None:
        cases.append(Case(cfg + ".unpack_postscale%g" % extra_postscale, unpack_kernel, unpack_scaled, payload * (bs + ts),
                          "the same unpack with postscale %g" % extra_postscale, plan0.num_chunks, reads=payload * bs))
    if share_world == 1:
        cases.append(Case(cfg + ".reduce+unpack", reduce_kernel + " + " + unpack_kernel, reduce_then_unpack,
                          (peers + 2) * share * bs + payload * (bs + ts),
                          "the reduce-sum and, right behind it on the same buffer, the unpack: the unpack's input comes "
                          "out of the Infinity Cache as in a cycle (a kernel trace gives each kernel's own duration)",
                          None, None, [(reduce_kernel, (peers + 2) * share * bs, (peers + 1) * share * bs),
                                       (unpack_kernel, payload * (bs + ts), payload * bs)]))
    if peers >= 3:
        # The worst placement of a staging ring: the resident chunk and its peers exactly 8 MiB apart
        # (a 1/8 share of a 64 MiB buffer is 8 MiB), against the back-to-back placement above.
        gap = 8 << 20
        assert share * bs <= gap
        ring = randn_bytes(ROTATE * (peers + 1) * gap, bt, std, seed0 + 60)
        torch.cuda.synchronize()

        def reduce_pow2():
            i = rot()
            at = ring.data_ptr() + i * (peers + 1) * gap
            H.reduce_sum_k(at, [at + (p + 1) * gap for p in range(peers)], share, bdtype, stream)

        cases.append(Case(cfg + ".reduce_8MiB_apart", reduce_kernel, reduce_pow2, (peers + 2) * share * bs,
                          "the same sum with the resident chunk and the %d peer chunks exactly 8 MiB apart in one "
                          "allocation (the spacing of a power-of-two staging ring)" % peers, (share + tile - 1) // tile,
                          reads=(peers + 1) * share * bs))
    return cases


def build_cases(cfg):
    """The kernel loops of one configuration (all on the first stream of the pair)."""
    import torch
    from horovod_amd import AdasumPlan, DTYPE, FusionPlan, host as H, workloads as W
    F32, F16 = DTYPE["float32"], DTYPE["float16"]
    s = stream_pair()[0]
    if cfg == "c1":
        counts = [W.numel(x) for x in W.resnet50_shapes()]
        g0 = W.fuse([4 * c for c in counts])[0]
        return cycle_cases("c1", [counts[i] for i in g0], F32, F32, 1e-3, 1, 1, s,
                           "xfer_k<Scale<float, float>, 0, 1>", "reduce_k<float, 1, 1>",
                           "xfer_k<Copy<unsigned int>, 1, 0>", 1000, pack_rotating=True)
    if cfg == "c2":
        counts = W.stress_counts(seed=3)
        cases = cycle_cases("c2", counts, F32, F32, 1.0, 1, 1, s, "xfer_k<Scale<float, float>, 0, 1>",
                            "reduce_k<float, 1, 1>", "xfer_k<Copy<unsigned int>, 1, 0>", 2000)
        return [cases[0], cases[2]]  # the stress configuration has no reduce stage
    if cfg == "c3":
        counts = [W.numel(x) for x in W.bert_large_shapes()]
        g1 = W.fuse([2 * c for c in counts])[1]
        return cycle_cases("c3", [counts[i] for i in g1], F32, F16, 1e-4, 7, 8, s,
                           "xfer_k<PackF32F16, 0, 1>", "reduce_k<_Float16, 7, 1>",
                           "xfer_k<UnpackF16F32, 1, 0>", 3000, extra_postscale=4.0)
    if cfg == "c5":
        counts = [W.numel(x) for x in W.gpt2_xl_shapes()]
        groups = W.fuse([2 * c for c in counts])
        layer = next(g for g in groups if len(g) == 12)
        cases = cycle_cases("c5", [counts[i] for i in layer], F16, F16, 1e-3, 1, 1, s,
                            "xfer_k<ScaleHalf, 0, 1>", "reduce_k<_Float16, 1, 1>",
                            "xfer_k<Copy<unsigned short>, 1, 0>", 5000)
        # the 50257 x 1600 embedding exceeds the threshold and travels alone: prescale tensor -> output,
        # sum in place (ops/nccl_operations.cc:176-186)
        n = counts[0]
        emb = [(randn_bytes(2 * n, torch.float16, 1e-3, 5100 + r), zeros_bytes(2 * n),
                randn_bytes(2 * n, torch.float16, 1e-3, 5200 + r)) for r in range(3)]
        torch.cuda.synchronize()
        turn = [0]

        def scale():
            i = turn[0] = (turn[0] + 1) % len(emb)
            H.scale_buffer(emb[i][0].data_ptr(), emb[i][1].data_ptr(), n, 0.125, F16, s)

        def reduce_emb():
            i = turn[0] = (turn[0] + 1) % len(emb)
            H.reduce_sum(emb[i][1].data_ptr(), emb[i][2].data_ptr(), n, F16, s)

        cases += [
            Case("c5.scale_single", "contig_k<ScaleHalf, 0>", scale, 4 * n,
                 "the embedding (%d halves) scaled by 0.125 from tensor to output; 3 pairs rotated" % n,
                 (2 * n + 4095) // 4096),
            Case("c5.reduce_single", "reduce_k<_Float16, 1, 1>", reduce_emb, 6 * n,
                 "the embedding summed in place with one peer; 3 pairs rotated", (2 * n + 4095) // 4096, reads=4 * n),
        ]
        return cases
    if cfg in ("c4", "c4h"):
        n = 1 << 25
        dt, tdt, es = (F32, torch.float32, 4) if cfg == "c4" else (F16, torch.float16, 2)
        tname = "float" if cfg == "c4" else "_Float16"
        lc = W.adasum_layer_counts(n, 64, seed=13)
        g = torch.Generator(device="cuda")
        pairs = []
        for r in range(4):
            g.manual_seed(14 + 2 * r)
            a = torch.randn(n, generator=g, device="cuda", dtype=torch.float32)
            g.manual_seed(15 + 2 * r)
            b = 0.3 * a + (1 - 0.09) ** 0.5 * torch.randn(n, generator=g, device="cuda", dtype=torch.float32)
            pairs.append((a.to(tdt), b.to(tdt)))
        plan = AdasumPlan(lc, dt)
        torch.cuda.synchronize()
        turn = [0]

        def combine():
            # the combine rewrites a; its cost does not depend on the values, which stay finite
            i = turn[0] = (turn[0] + 1) % len(pairs)
            plan.combine(pairs[i][0].data_ptr(), pairs[i][1].data_ptr(), s)

        # the first pass keeps a alone in the Infinity Cache for the 2 x 128 MiB of fp32, both vectors for the 2 x 64 MiB of fp16
        k1, k2 = "dot_partials_k<%s, %d>" % (tname, 1 if cfg == "c4" else 2), "scaled_add_k<%s, true, 0>" % tname
        return [Case(cfg + ".combine", k1 + " + " + k2, combine, 5 * n * es,
                     "Adasum combine of two vectors of 2^25 elements in 64 layers: first pass 2 N s bytes (leaves what "
                     "pays in the Infinity Cache), second pass 3 N s bytes; 4 pairs rotated", None, plan.destroy,
                     parts=[(k1, 2 * n * es, 2 * n * es), (k2, 3 * n * es, 2 * n * es)])]
    if cfg == "ag":
        return allgather_cases(s)
    if cfg == "copy":
        # One GiB copied to another by the library's copy kernel, by the runtime's own device-to-device
        # hipMemcpyAsync and by an elementwise kernel of torch: what this device streams, whoever asks.
        import horovod_amd
        n = 1 << 30
        pairs = [(randn_bytes(n, torch.float32, 1.0, 90 + i), torch.empty(n, dtype=torch.uint8, device="cuda"))
                 for i in range(3)]
        torch.cuda.synchronize()
        turn = [0]

        def nxt():
            turn[0] = (turn[0] + 1) % len(pairs)
            return pairs[turn[0]]

        def library():
            src, dst = nxt()
            H.batched_d2d_memcpy([dst.data_ptr()], [src.data_ptr()], [n], s)

        memcpy = horovod_amd.lib().hvdhip_memcpy_async
        D2D = 3  # HVDHIP_MEMCPY_D2D

        def runtime():
            src, dst = nxt()
            horovod_amd.check(memcpy(dst.data_ptr(), src.data_ptr(), n, D2D, s.handle), "hvdhip_memcpy_async")

        ext = torch.cuda.ExternalStream(s.handle.value)

        def framework():
            src, dst = nxt()
            # an elementwise kernel of torch's own (Tensor.copy_ between buffers of one dtype is the
            # runtime's hipMemcpyAsync again)
            with torch.cuda.stream(ext):
                torch.mul(src.view(torch.float32), 1.0, out=dst.view(torch.float32))

        what = "1 GiB copied from one buffer to another; 3 (source, destination) pairs rotated"
        return [Case("copy.library", "xfer_k<Copy<unsigned char>, 2, 0>", library, 2 * n,
                     what + "; hvdhip_batched_d2d_memcpy with one entry", n // 4096),
                Case("copy.runtime", "__amd_rocclr_copyBuffer", runtime, 2 * n,
                     what + "; hipMemcpyAsync, device to device"),
                Case("copy.torch", "at::native::vectorized_elementwise_kernel<4, MulFunctor<float>>", framework, 2 * n,
                     what + "; torch.mul(x, 1.0, out=y) on fp32 views, on the same stream")]
    raise ValueError(cfg)


def measure_cases(cases, steps=100, warmup=10):
    """Roofline block per case, from HIP events on the stream the kernel is launched on."""
    s = stream_pair()[0]
    out = []
    for c in cases:
        sec, each = event_timed(c.fn, s, steps, warmup)
        gbs = c.alg / sec / 1e9
        out.append({"bound": "hbm", "kernel": c.kernel, "case": c.key, "launch_us": round(sec * 1e6, 2),
                    "launch_us_median_min_max": spread(each, 1e6, 2), "timed_batches": len(each),
                    "algorithmic_bytes_per_launch": c.alg, "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS,
                    "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
                    "traffic": TRAFFIC_BYTES_MEASURED.get(c.key), "workgroups": c.workgroups, "timed": c.what})
    for b in out:
        ns = IN_PIPELINE_NS_MEASURED.get(b["case"])
        if ns:
            b["in_pipeline_us"] = round(ns / 1e3, 2)
            b["in_pipeline_frac"] = round(b["algorithmic_bytes_per_launch"] / ns / HBM_PEAK_GBS, 4)
            b["in_pipeline_from"] = "kernel-trace duration behind the reduce-sum that wrote its buffer (%s.reduce+unpack in the profile)" % b["case"].split(".")[0]
    return out


def release(cases):
    """Destroys the plans of the cases and lets go of their device memory."""
    import torch
    torch.cuda.synchronize()
    for c in cases:
        if c.cleanup:
            c.cleanup()
        c.cleanup = c.fn = None
    torch.cuda.empty_cache()


# ----------------------------------------------------------------------------------------------
# whole pipelines
# ----------------------------------------------------------------------------------------------

class PipelineRun:
    """A configuration's whole pipeline over `replicas` rotating tensor sets.  All replicas queue on
    the same stream(s) and share the one fusion buffer of each stream slot."""

    def __init__(self, shapes, tdtype, bdtype, std, peers, fraction, streams, replicas, arrays=False,
                 completion_events=None, record_with_unpack=False, postscale=1.0):
        import torch
        self.postscale = postscale
        from horovod_amd import dtype_size, workloads as W
        from horovod_amd.pipeline import AllreducePipeline
        es = dtype_size(tdtype)
        self.counts = [W.numel(x) for x in shapes]
        self.peers, self.fraction = peers, fraction
        self.reps = []
        shared = stream_pair()[:streams]
        buffers = None
        for r in range(replicas):
            src = DeviceSet(self.counts, es, lambda n: randn_bytes(n, torch_dtype(tdtype), std, 1 + r))
            dst = DeviceSet(self.counts, es, zeros_bytes)
            pipe = AllreducePipeline(src.ptrs, dst.ptrs, self.counts, tdtype, bdtype, streams=shared, buffers=buffers,
                                     array_entry_points=arrays, completion_events=completion_events,
                                     record_with_unpack=record_with_unpack)
            buffers = pipe.buffers
            bs = dtype_size(pipe.buffer_dtype)
            # one buffer per peer, sized for the largest cycle's reduced chunk, serves every cycle
            need = max(pipe.reduce_elems(c, fraction) for c in pipe.cycles) * bs
            peer_bufs = [randn_bytes((need + 255) // 256 * 256, torch_dtype(pipe.buffer_dtype), std, 100 + 16 * r + p)
                         for p in range(peers)]
            self.reps.append((src, dst, pipe, peer_bufs))
        torch.cuda.synchronize()
        self.turn = 0
        self.pipe = self.reps[0][2]

    def one_pass(self):
        self.turn += 1
        _, _, pipe, peer_bufs = self.reps[self.turn % len(self.reps)]
        # a single-cycle configuration alternates its passes over the stream slots
        first_slot = self.turn if len(pipe.cycles) == 1 else 0
        pipe.run(0.125, self.postscale, (lambda ci, p: peer_bufs[p].data_ptr()) if self.peers else None, self.peers,
                 self.fraction, True, first_slot=first_slot)

    def sync(self):
        for _, _, pipe, _ in self.reps:
            pipe.synchronize()

    def algorithmic_bytes(self):
        return self.pipe.algorithmic_bytes(self.peers, self.fraction, True)

    def destroy(self):
        import torch
        for _, _, pipe, _ in self.reps:
            pipe.destroy()
        self.reps = []
        torch.cuda.empty_cache()


class AdapterRun:
    """The same pipelines through the C++ adapter: every fused response goes through
    GPUAllreduce::Execute (pack -> sum with the peer buffer -> unpack with the completion event bound to
    it -> FinalizeGPUQueue), which returns once the kernels are queued; finalizer threads, one per
    stream slot, wait for the events and call the entries' callbacks, and the stream slot rotates after
    every response (ops/gpu_operations.cc:50-103).  The calling thread plays Horovod's background thread."""

    def __init__(self, shapes, dtype, std, slots, replicas):
        import ctypes
        import torch
        from horovod_amd import dtype_size, workloads as W
        from horovod_amd._lib import adapter_lib
        lib = adapter_lib()
        VP = ctypes.c_void_p
        lib.hvd_adapter_create_ex.restype = VP
        lib.hvd_adapter_create_ex.argtypes = [ctypes.c_int] * 4 + [VP, ctypes.c_int]
        lib.hvd_adapter_destroy.argtypes = [VP]
        lib.hvd_adapter_prepare.argtypes = [VP, VP, VP, VP, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        lib.hvd_adapter_execute_prepared.argtypes = [VP, ctypes.c_int, ctypes.c_double, ctypes.c_double, VP, ctypes.c_int,
                                                     ctypes.c_char_p, ctypes.c_size_t]
        lib.hvd_adapter_wait_all.argtypes = [VP, ctypes.c_char_p, ctypes.c_size_t]
        lib.hvd_adapter_reset_tickets.argtypes = [VP]
        self.lib = lib
        es = dtype_size(dtype)
        self.es = es
        self.counts = [W.numel(x) for x in shapes]
        groups = W.fuse([c * es for c in self.counts])
        self.groups = groups
        need = max([sum((self.counts[i] * es + 15) // 16 * 16 for i in g) for g in groups if len(g) > 1] + [16]) + 4096 * es
        self.fbs = [zeros_bytes(need) for _ in range(slots)]
        self.h = lib.hvd_adapter_create_ex(slots, 1, 0, 0, (VP * slots)(*[b.data_ptr() for b in self.fbs]), slots)
        # the run's one pair of streams, created before any other (see stream_pair)
        lib.hvd_adapter_use_streams.argtypes = [VP, VP]
        lib.hvd_adapter_use_streams(self.h, (VP * slots)(*[st.handle.value for st in stream_pair()[:slots]]))
        self.err = ctypes.create_string_buffer(512)
        self.reps = []
        for r in range(replicas):
            src = DeviceSet(self.counts, es, lambda n: randn_bytes(n, torch_dtype(dtype), std, 1 + r))
            dst = DeviceSet(self.counts, es, zeros_bytes)
            # one peer buffer, sized for the largest response, serves every response of the replica
            largest = max(sum((self.counts[i] * es + 15) // 16 * 16 for i in g) for g in groups)
            peer = randn_bytes((largest + 255) // 256 * 256, torch_dtype(dtype), std, 100 + 16 * r)
            ids = []
            for g in groups:
                n = len(g)
                ids.append(lib.hvd_adapter_prepare(self.h, (VP * n)(*[src.ptrs[i] for i in g]),
                                                   (VP * n)(*[dst.ptrs[i] for i in g]),
                                                   (ctypes.c_int64 * n)(*[self.counts[i] for i in g]), n, dtype, -1))
            self.reps.append((src, dst, peer, ids, (VP * 1)(peer.data_ptr())))
        torch.cuda.synchronize()
        self.turn = 0

    def one_pass(self):
        self.turn += 1
        _, _, _, ids, peers = self.reps[self.turn % len(self.reps)]
        for i in ids:
            if self.lib.hvd_adapter_execute_prepared(self.h, i, 0.125, 1.0, peers, 1, self.err, 512) < 0:
                raise RuntimeError(self.err.value.decode())

    def sync(self):
        if self.lib.hvd_adapter_wait_all(self.h, self.err, 512) != 0:
            raise RuntimeError(self.err.value.decode())
        self.lib.hvd_adapter_reset_tickets(self.h)

    def algorithmic_bytes(self):
        # fused: pack 2P + reduce 3C (C = the padded buffer) + unpack 2P; single entry: scale 2P + reduce 3P
        total = 0
        for g in self.groups:
            payload = sum(self.counts[i] for i in g) * self.es
            if len(g) > 1:
                total += 4 * payload + 3 * sum((self.counts[i] * self.es + 15) // 16 * 16 for i in g)
            else:
                total += 5 * payload
        return total

    def destroy(self):
        import torch
        self.sync()
        self.lib.hvd_adapter_destroy(self.h)
        self.reps = []
        self.fbs = []
        torch.cuda.empty_cache()


def pipeline_figures(run, sec, streams, note=None):
    ab = run.algorithmic_bytes()
    d = {"algorithmic_GB/s": round(ab / sec / 1e9, 1), "algorithmic_frac_of_8TBps": round(ab / sec / 1e9 / HBM_PEAK_GBS, 4),
         "ms": round(sec * 1e3, 4), "algorithmic_MB": round(ab / 1e6, 1), "cycles": len(run.pipe.cycles),
         "streams": streams, "peers": run.peers, "reduce": "k-way" if run.peers else None,
         "completion_event_per_cycle": run.pipe.completion_events, "replicas_rotated": len(run.reps)}
    if note:
        d["note"] = note
    return d


# ----------------------------------------------------------------------------------------------
# CPU baselines: the oracle on one host core, same algorithmic bytes
# ----------------------------------------------------------------------------------------------

def _oracle():
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle_util
    return oracle_util, oracle_util.Oracle().lib


def cpu_baseline_resnet(budget_s=12.0):
    """The reference CPU sequence (ops/gloo_operations.cc:118-170) over the whole ResNet-50 set:
    memcpy pack, in-place ScaleBuffer(0.125), sum with one peer buffer, memcpy unpack (7P bytes)."""
    from ctypes import c_double, c_int, c_int64, c_void_p
    from horovod_amd import workloads as W
    ou, L = _oracle()
    rng = np.random.default_rng(1)
    counts = [W.numel(s) for s in W.resnet50_shapes()]
    ts = [(rng.standard_normal(c, dtype=np.float32) * np.float32(1e-3)) for c in counts]
    outs = [np.empty_like(t) for t in ts]
    n, k = sum(counts), len(counts)
    nb = np.array([4 * c for c in counts], np.int64)
    buf = np.zeros(n, np.float32)
    peer = np.random.default_rng(2).standard_normal(n, dtype=np.float32) * np.float32(1e-3)
    tp = (c_void_p * k)(*[t.ctypes.data for t in ts])
    op = (c_void_p * k)(*[t.ctypes.data for t in outs])
    P = lambda a: c_void_p(a.ctypes.data)  # noqa: E731

    def one():
        L.orc_pack(tp, P(nb), c_int(k), P(buf))
        L.orc_scale_buffer(P(buf), P(buf), c_int64(n), c_double(0.125), c_int(ou.F32))
        L.orc_sum(P(peer), P(buf), c_int64(n), c_int(ou.F32))
        L.orc_unpack(P(buf), op, P(nb), c_int(k))

    one()
    reps, t0 = 0, time.perf_counter()
    while True:
        one()
        reps += 1
        dt = time.perf_counter() - t0
        if dt > budget_s:
            break
    gbs = 7 * 4 * n * reps / dt / 1e9
    return {"value": round(gbs, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": "%d passes over the whole 161-tensor set (memcpy pack, in-place ScaleBuffer 0.125, sum with one "
                      "peer buffer, memcpy unpack; 7P bytes each) in %.1f s; host has %d cores" % (reps, dt, os.cpu_count())}


def cpu_extras(budget_s=2.5):
    """The CPU oracle on one core over the other configurations, whole sets, in the same algorithmic
    bytes as the GPU figures: the stress set, BERT-large in its 11 cycles (cast and scale fused into
    the copy, which flatters the CPU), the Adasum pair, GPT-2 XL in its 49 cycles."""
    from ctypes import c_double, c_int, c_int64, c_void_p
    from horovod_amd import workloads as W
    ou, L = _oracle()
    F16, F32 = ou.F16, ou.F32
    rng = np.random.default_rng(0)
    out = {}

    def P(a, off=0):
        return c_void_p(a.ctypes.data + off)

    def ptrs(arrays):
        return (c_void_p * len(arrays))(*[a.ctypes.data for a in arrays])

    def rep(block, c):
        """c values: the block, repeated as often as it takes."""
        if c <= block.size:
            return block[:c].copy()
        return np.concatenate([block] * (c // block.size) + [block[:c % block.size]])

    def run(name, fn, nbytes, sample):
        fn()
        reps, t0 = 0, time.perf_counter()
        while True:
            fn()
            reps += 1
            dt = time.perf_counter() - t0
            if dt > budget_s:
                break
        out[name] = {"cpu_GB/s": round(nbytes * reps / dt / 1e9, 2), "cpu_cores": 1, "cpu_sample": "%d x %s" % (reps, sample)}

    # fusion stress: memcpy pack, ScaleBuffer 0.125 in place, memcpy unpack (4P)
    counts = W.stress_counts(seed=3)
    ts = [rng.uniform(-1, 1, c).astype(np.float32) for c in counts]
    outs = [np.empty_like(t) for t in ts]
    n, k = sum(counts), len(counts)
    nb = np.array([4 * c for c in counts], np.int64)
    buf = np.zeros(n, np.float32)
    tp, op = ptrs(ts), ptrs(outs)

    def stress():
        L.orc_pack(tp, P(nb), c_int(k), P(buf))
        L.orc_scale_buffer(P(buf), P(buf), c_int64(n), c_double(0.125), c_int(F32))
        L.orc_unpack(P(buf), op, P(nb), c_int(k))

    run("c2_fusion_stress", stress, 4 * 4 * n, "the whole 1,024-tensor set")

    # BERT-large, the whole set in its 11 cycles: fp32 -> fp16 with prescale, 7 peers on 1/8, fp16 -> fp32
    counts = [W.numel(s) for s in W.bert_large_shapes()]
    groups = W.fuse([2 * c for c in counts])
    # (the tensors repeat one block of random values: the CPU's time does not depend on the values,
    # and drawing 336 M of them would take longer than the measurement)
    block = rng.standard_normal(1 << 24, dtype=np.float32) * np.float32(1e-4)
    ts = [rep(block, c) for c in counts]
    outs = [np.empty_like(t) for t in ts]
    sizes = [sum(counts[i] for i in g) for g in groups]
    shares = [W.reduce_scatter_share(n, 8) for n in sizes]
    hbuf = np.zeros(max(sizes) + 4096, np.uint16)
    peers = [[rng.integers(0, 0x0400, sh, dtype=np.uint16) for _ in range(7)] for sh in shares]

    def bert():
        for g, share, ps in zip(groups, shares, peers):
            off = 0
            for i in g:
                L.orc_scale_cast_f32_to_f16_f16c(P(ts[i]), P(hbuf, 2 * off), c_int64(counts[i]), c_double(0.125))
                off += counts[i]
            for p in ps:
                L.orc_float16_sum(P(p), P(hbuf), c_int64(share))
            off = 0
            for i in g:
                L.orc_scale_cast_f16_to_f32_f16c(P(hbuf, 2 * off), P(outs[i]), c_int64(counts[i]), c_double(1.0))
                off += counts[i]

    run("c3_bert_large_fp32_to_fp16_7peers_eighth_share", bert,
        sum(12 * n + 9 * 2 * sh for n, sh in zip(sizes, shares)), "the whole 397-tensor set in %d cycles" % len(groups))
    del ts, outs, peers, block

    # Adasum: the whole pair, in place on a (values stay finite from repetition to repetition)
    n = 1 << 25
    lc = np.array(W.adasum_layer_counts(n, 64, seed=13), np.int32)
    a = rng.standard_normal(n, dtype=np.float32)
    b = rng.standard_normal(n, dtype=np.float32)
    nd, co = np.zeros(192), np.zeros(128)
    run("c4_adasum_fp32_2x32M_64layers",
        lambda: L.orc_adasum_pairwise(P(a), P(b), c_int(F32), P(lc), c_int(64), P(nd), P(co)), 5 * n * 4,
        "the whole pair")

    # GPT-2 XL, the whole set: 48 fused cycles (memcpy pack, ScaleBuffer in place, sum with the peer buffer,
    # memcpy unpack: 7P) and the embedding by itself (scale from tensor to output, sum in place: 5P)
    counts = [W.numel(s) for s in W.gpt2_xl_shapes()]
    groups = W.fuse([2 * c for c in counts])
    block = rng.integers(0x0400, 0x3c00, 1 << 25, dtype=np.uint16)  # normal halves below 1, repeated
    ts = [rep(block, c) for c in counts]
    outs = [np.empty_like(t) for t in ts]
    sizes = [sum(counts[i] for i in g) for g in groups]
    peers = [rep(block[12345:], n) for n in sizes]
    hbuf = np.zeros(max(n for n, g in zip(sizes, groups) if len(g) > 1), np.uint16)
    args = []
    for g, n in zip(groups, sizes):
        nb = np.array([2 * counts[i] for i in g], np.int64)
        args.append((ptrs([ts[i] for i in g]), ptrs([outs[i] for i in g]), nb, len(g), n))

    def gpt2():
        for (tp2, op2, nb, k, n), g, peer in zip(args, groups, peers):
            if k == 1:
                L.orc_scale_buffer(P(ts[g[0]]), P(outs[g[0]]), c_int64(n), c_double(0.125), c_int(F16))
                L.orc_float16_sum(P(peer), P(outs[g[0]]), c_int64(n))
                continue
            L.orc_pack(tp2, P(nb), c_int(k), P(hbuf))
            L.orc_scale_buffer(P(hbuf), P(hbuf), c_int64(n), c_double(0.125), c_int(F16))
            L.orc_float16_sum(P(peer), P(hbuf), c_int64(n))
            L.orc_unpack(P(hbuf), op2, P(nb), c_int(k))

    run("c5_gpt2_xl_fp16_two_streams", gpt2, sum((7 if len(g) > 1 else 5) * 2 * n for g, n in zip(groups, sizes)),
        "the whole 580-tensor set in %d cycles" % len(groups))
    return out


# ----------------------------------------------------------------------------------------------
# extras
# ----------------------------------------------------------------------------------------------

def per_tensor_comparator(reps=20):
    """The fusion stress step through the C++ adapter's GPUAllreduce::Execute twice: with the
    offset-table kernels, and with one hipMemcpyAsync per tensor each way plus a whole-buffer
    ScaleBuffer (HOROVOD_BATCH_D2D_MEMCOPIES=0, what Horovod does on ROCm today,
    ops/gpu_operations.cc:209-222,230-235,327-332).  Both include the op's completion wait."""
    import ctypes
    import torch
    from horovod_amd import workloads as W
    counts = W.stress_counts(seed=3)
    src = DeviceSet(counts, 4, lambda n: randn_bytes(n, torch.float32, 1.0, 4))
    dst = DeviceSet(counts, 4, zeros_bytes)
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


def allgather_cases(s):
    """Allgather fusion buffer (ops/collective_operations.cc:234-288, GPU copies ops/gpu_operations.cc:350-363):
    8 ranks, 128 entries per rank.  This GPU packs its own slab at its displacement (the other slabs arrive
    by the collective, which is not built) and unpacks one component per (entry, rank): 1,024 copies.  Each
    direction is one batched copy through the descriptor-array entry point.  Two sizes: the stress
    workload's size mix as it is (a 6 MB slab: the pack is a launch floor) and eleven times that (a 66 MB
    slab, a 528 MB buffer: bandwidth-bound)."""
    import ctypes
    import torch
    import horovod_amd
    from horovod_amd import workloads as W
    world, es = 8, 4
    copy = horovod_amd.lib().hvdhip_batched_d2d_memcpy
    cases = []
    for tag, mult, rotate in (("_small", 1, 4), ("", 11, 3)):
        counts = [c * mult for c in W.stress_counts(seed=21, n=128)]
        slab = es * sum(counts)
        sets = []
        for r in range(rotate):
            src = DeviceSet(counts, es, lambda n: randn_bytes(n, torch.float32, 1.0, 60 + r))
            fusion = randn_bytes(world * slab, torch.float32, 1.0, 70 + r)
            out_set = DeviceSet([world * c for c in counts], es, zeros_bytes)
            pack_dst, at = [], 3 * slab  # this rank's displacement (rank 3 of 8)
            for c in counts:
                pack_dst.append(fusion.data_ptr() + at)
                at += c * es
            un_dst, un_src, un_sz = [], [], []
            for rank in range(world):
                at = rank * slab
                for i, c in enumerate(counts):
                    un_dst.append(out_set.ptrs[i] + rank * c * es)
                    un_src.append(fusion.data_ptr() + at)
                    un_sz.append(c * es)
                    at += c * es
            # the descriptor arrays as the C caller holds them, built once
            VP, SZ = ctypes.c_void_p, ctypes.c_size_t
            pack_args = ((VP * len(counts))(*pack_dst), (VP * len(counts))(*src.ptrs),
                         (SZ * len(counts))(*[c * es for c in counts]), len(counts))
            un_args = ((VP * len(un_dst))(*un_dst), (VP * len(un_dst))(*un_src), (SZ * len(un_dst))(*un_sz), len(un_dst))
            sets.append((src, fusion, out_set, pack_args, un_args))
        torch.cuda.synchronize()
        turn = [0]

        def pack(sets=sets, turn=turn):
            i = turn[0] = (turn[0] + 1) % len(sets)
            horovod_amd.check(copy(*sets[i][3], s.handle), "hvdhip_batched_d2d_memcpy")

        def unpack(sets=sets, turn=turn):
            i = turn[0] = (turn[0] + 1) % len(sets)
            horovod_amd.check(copy(*sets[i][4], s.handle), "hvdhip_batched_d2d_memcpy")

        chunks = lambda sizes: sum((z + 4095) // 4096 for z in sizes)  # noqa: E731
        cases += [
            Case("ag.pack" + tag, "xfer_k<Copy<unsigned char>, 2, 1>", pack, 2 * slab,
                 "this rank's %d entries (%d bytes) copied to its displacement in the allgather buffer; %d sets rotated"
                 % (len(counts), slab, rotate), chunks([c * es for c in counts])),
            Case("ag.unpack" + tag, "xfer_k<Copy<unsigned char>, 2, 0>", unpack, 2 * world * slab,
                 "%d components (entry x rank) copied out of the %d-byte buffer into the entries' outputs; %d sets rotated"
                 % (world * len(counts), world * slab, rotate), chunks(un_sz)),
        ]
    return cases


def allgather_extra():
    """The allgather fusion buffer's two copies as one step (pack + unpack), from their kernel loops."""
    import torch
    cases = build_cases("ag")
    blocks = measure_cases(cases, steps=60, warmup=6)
    release(cases)
    del cases
    torch.cuda.empty_cache()
    out = {}
    for tag, name in (("_small", "allgather_fusion_8ranks_128entries_6MB_slab"), ("", "allgather_fusion_8ranks_128entries_66MB_slab")):
        pk = next(b for b in blocks if b["case"] == "ag.pack" + tag)
        un = next(b for b in blocks if b["case"] == "ag.unpack" + tag)
        ab = pk["algorithmic_bytes_per_launch"] + un["algorithmic_bytes_per_launch"]
        sec = (pk["launch_us"] + un["launch_us"]) * 1e-6
        out[name] = {"algorithmic_GB/s": round(ab / sec / 1e9, 1), "algorithmic_frac_of_8TBps": round(ab / sec / 1e9 / HBM_PEAK_GBS, 4),
                     "ms": round(sec * 1e3, 4), "algorithmic_MB": round(ab / 1e6, 1), "streams": 1,
                     "kernels": [pk, un], "traffic_profile": TRAFFIC_PROFILE["ag"],
                     "note": "pack + unpack launch times added; each from its own back-to-back loop"}
    return out


def device_ceiling_extra(steps=20):
    """What this device streams, measured in the same run: one 1 GiB buffer copied to another by the
    library's copy kernel, by the runtime's own device-to-device hipMemcpyAsync, and by an elementwise
    kernel of torch, all on the same stream and timed with HIP events on it (the `copy` kernel loops).  The
    kernels above are to be read against these figures as well as against the nominal 8 TB/s."""
    import torch
    cases = build_cases("copy")
    blocks = measure_cases(cases, steps=steps, warmup=3)
    release(cases)
    del cases
    torch.cuda.empty_cache()
    return {"kernels": blocks, "traffic_profile": TRAFFIC_PROFILE["copy"]}


def adasum_split_extra(steps=30):
    """The Adasum configuration through hvdhip_adasum_dot_norms -> hvdhip_adasum_read (the host gets the 64
    triples; between ranks they would be summed here, adasum.h:380-382) -> coefficients on the host
    (adasum.h:397-404) -> hvdhip_adasum_set_coeffs -> hvdhip_adasum_scaled_add: what the combine costs once
    the sums have to leave the device, which is what more than one GPU needs."""
    import math
    import torch
    from horovod_amd import AdasumPlan, DTYPE, workloads as W
    s = stream_pair()[0]
    n = 1 << 25
    lc = W.adasum_layer_counts(n, 64, seed=13)
    g = torch.Generator(device="cuda")
    pairs = []
    for r in range(4):
        g.manual_seed(14 + 2 * r)
        a = torch.randn(n, generator=g, device="cuda", dtype=torch.float32)
        g.manual_seed(15 + 2 * r)
        b = 0.3 * a + (1 - 0.09) ** 0.5 * torch.randn(n, generator=g, device="cuda", dtype=torch.float32)
        pairs.append((a, b))
    plan = AdasumPlan(lc, DTYPE["float32"])
    torch.cuda.synchronize()
    guard = math.sqrt(2.2250738585072014e-308)
    turn = [0]

    def one():
        i = turn[0] = (turn[0] + 1) % len(pairs)
        a, b = pairs[i]
        plan.dot_norms(a.data_ptr(), b.data_ptr(), s)
        nd, _ = plan.read(s)  # blocks until the triples are on the host
        co = []
        for k in range(len(lc)):
            d, an, bn = nd[3 * k:3 * k + 3]
            co += [1.0 - d / an * 0.5 if an >= guard else 1.0, 1.0 - d / bn * 0.5 if bn >= guard else 1.0]
        plan.set_coeffs(co, s)
        plan.scaled_add(a.data_ptr(), b.data_ptr(), s)

    sec, each = timed_batches(one, s.synchronize, steps, 3)
    plan.destroy()
    del pairs
    torch.cuda.empty_cache()
    ab = 5 * n * 4
    return {"algorithmic_GB/s": round(ab / sec / 1e9, 1), "algorithmic_frac_of_8TBps": round(ab / sec / 1e9 / HBM_PEAK_GBS, 4),
            "ms": round(sec * 1e3, 4), "ms_median_min_max": spread(each, 1e3, 4), "algorithmic_MB": round(ab / 1e6, 1),
            "streams": 1, "replicas_rotated": 4,
            "note": "dot_norms, blocking read of 64 triples, coefficients on the host, set_coeffs, scaled_add"}


def extras(headline_cases_block):
    import torch
    from horovod_amd import DTYPE, workloads as W
    F32, F16 = DTYPE["float32"], DTYPE["float16"]
    out = {}

    def pipeline(name, shapes, tdt, bdt, std, peers, fraction, streams, replicas, steps, arrays=False, note=None,
                 completion_events=None, record_with_unpack=False, postscale=1.0):
        run = PipelineRun(shapes, tdt, bdt, std, peers, fraction, streams, replicas, arrays=arrays,
                          completion_events=completion_events, record_with_unpack=record_with_unpack,
                          postscale=postscale)
        sec, each = timed_batches(run.one_pass, run.sync, steps, max(2, steps // 10))
        out[name] = pipeline_figures(run, sec, streams, note)
        out[name]["ms_median_min_max"] = spread(each, 1e3, 4)
        run.destroy()

    def through_adapter(name, shapes, dt, std, slots, replicas, steps, beside):
        run = AdapterRun(shapes, dt, std, slots, replicas)
        sec, each = timed_batches(run.one_pass, run.sync, steps, max(2, steps // 10))
        ab = run.algorithmic_bytes()
        out[name] = {"algorithmic_GB/s": round(ab / sec / 1e9, 1),
                     "algorithmic_frac_of_8TBps": round(ab / sec / 1e9 / HBM_PEAK_GBS, 4), "ms": round(sec * 1e3, 4),
                     "ms_median_min_max": spread(each, 1e3, 4), "algorithmic_MB": round(ab / 1e6, 1),
                     "cycles": len(run.groups), "streams": slots, "peers": 1, "replicas_rotated": len(run.reps),
                     "vs_python_pipeline": round(out[beside]["ms"] / (sec * 1e3), 4),
                     "note": "every response through the C++ adapter's GPUAllreduce::Execute on %d stream slot(s), completion "
                             "on finalizer threads; vs_python_pipeline = time of %s / this time" % (slots, beside)}
        run.destroy()

    def kernels(name, cfg):
        cases = build_cases(cfg)
        blocks = measure_cases(cases)
        release(cases)
        del cases
        torch.cuda.empty_cache()
        out[name]["kernels"] = blocks
        out[name]["roofline_case"] = max((b for b in blocks if "+" not in b["case"]), key=lambda b: b["launch_us"])["case"]
        out[name]["traffic_profile"] = TRAFFIC_PROFILE.get(cfg.rstrip("h"))

    # C1 on two streams (the headline is the one-stream figure); its kernel blocks come from the headline
    pipeline("c1_resnet50_fp32_one_stream", W.resnet50_shapes(), F32, F32, 1e-3, 1, 1.0, 1, 4, 200,
             completion_events=True, record_with_unpack=True,
             note="the headline pipeline with the completion event of every cycle bound to its unpack kernel "
                  "(hvdhip_fusion_unpack_record) and waited for by the host: what the adapter's Execute queues")
    through_adapter("c1_resnet50_fp32_one_slot_through_the_adapter", W.resnet50_shapes(), F32, 1e-3, 1, 4, 200,
                    "c1_resnet50_fp32_one_stream")
    pipeline("c1_resnet50_fp32_two_streams", W.resnet50_shapes(), F32, F32, 1e-3, 1, 1.0, 2, 4, 200)
    out["c1_resnet50_fp32_two_streams"]["kernels"] = headline_cases_block
    pipeline("c1_resnet50_fp32_one_stream_completion_events", W.resnet50_shapes(), F32, F32, 1e-3, 1, 1.0, 1, 4, 200,
             completion_events=True,
             note="the headline pipeline with a pooled completion event recorded behind every cycle and waited for by "
                  "the host, as GPUOpContext::FinalizeGPUQueue does once per response (ops/gpu_operations.cc:50-98)")

    # C2: fusion stress, pack + unpack, 200 repetitions
    stress = [(c,) for c in W.stress_counts(seed=3)]
    pipeline("c2_fusion_stress", stress, F32, F32, 1.0, 0, 1.0, 1, 8, 200,
             note="1,024 fp32 tensors, log-uniform 256..65,536 elements (seed 3): pack with prescale 0.125, unpack; "
                  "200 repetitions timed; every kernel behind its predecessor on one stream")
    kernels("c2_fusion_stress", "c2")
    pipeline("c2_fusion_stress_one_stream_completion_events", stress, F32, F32, 1.0, 0, 1.0, 1, 8, 200,
             completion_events=True,
             note="one stream, a pooled completion event behind every repetition")
    pipeline("c2_fusion_stress_one_stream_completion_events_with_unpack", stress, F32, F32, 1.0, 0, 1.0, 1, 8, 200,
             completion_events=True, record_with_unpack=True,
             note="one stream, the completion event of every repetition bound to its unpack kernel")
    pipeline("c2_fusion_stress_two_streams", stress, F32, F32, 1.0, 0, 1.0, 2, 8, 200,
             note="consecutive repetitions alternate over two stream slots, each with its own fusion buffer; a pooled "
                  "completion event behind every repetition, as GPUOpContext::FinalizeGPUQueue records one per response")
    pipeline("c2_fusion_stress_two_streams_no_completion_events", stress, F32, F32, 1.0, 0, 1.0, 2, 8, 200,
             completion_events=False,
             note="the same without the per-repetition completion event (the streams are synchronised at the end)")
    try:
        out["c2_fusion_stress"]["execute_vs_per_tensor_copies"] = per_tensor_comparator()
    except Exception as e:  # pragma: no cover
        out["c2_fusion_stress"]["execute_vs_per_tensor_copies"] = {"error": "%s: %s" % (type(e).__name__, e)}

    # C3: BERT-large fp32 -> fp16, 7 peers on the 1/8 share; postscale 1.0 and a non-trivial power of two
    pipeline("c3_bert_large_fp32_to_fp16_7peers_eighth_share", W.bert_large_shapes(), F32, F16, 1e-4, 7, 0.125, 1, 1, 20)
    kernels("c3_bert_large_fp32_to_fp16_7peers_eighth_share", "c3")
    pipeline("c3_bert_large_postscale_4", W.bert_large_shapes(), F32, F16, 1e-4, 7, 0.125, 1, 1, 20, postscale=4.0,
             note="the same pipeline with postscale 4.0 in the widening unpack (the kernel multiplies either way)")
    pipeline("c3_bert_large_two_streams", W.bert_large_shapes(), F32, F16, 1e-4, 7, 0.125, 2, 1, 20)

    # C4: Adasum combine, fp32 (the configuration) and fp16
    for cfg, name in (("c4", "c4_adasum_fp32_2x32M_64layers"), ("c4h", "c4_adasum_fp16_2x32M_64layers")):
        cases = build_cases(cfg)
        blocks = measure_cases(cases, steps=50, warmup=4)
        release(cases)
        del cases
        torch.cuda.empty_cache()
        b = blocks[0]
        out[name] = {"algorithmic_GB/s": b["achieved"], "algorithmic_frac_of_8TBps": b["frac"],
                     "ms": round(b["launch_us"] / 1e3, 4), "ms_median_min_max": [round(x / 1e3, 4) for x in b["launch_us_median_min_max"]],
                     "algorithmic_MB": round(b["algorithmic_bytes_per_launch"] / 1e6, 1),
                     "replicas_rotated": 4, "kernels": blocks, "roofline_case": b["case"], "traffic_profile": TRAFFIC_PROFILE["c4"],
                     "note": "two launches timed together with HIP events; per-kernel durations and traffic are in the profile"}

    # C4 through the split entry points, as more than one GPU needs them: the partial sums leave the device
    # for the exchange between ranks and the coefficients come back (ops/adasum/adasum.h:380-404)
    out["c4_adasum_fp32_split_with_host_round_trip"] = adasum_split_extra()

    # C5: GPT-2 XL fp16 on two streams (the configuration), on one, through the array-taking entry points
    # and through the adapter on two stream slots
    pipeline("c5_gpt2_xl_fp16_two_streams", W.gpt2_xl_shapes(), F16, F16, 1e-3, 1, 1.0, 2, 1, 10)
    kernels("c5_gpt2_xl_fp16_two_streams", "c5")
    through_adapter("c5_gpt2_xl_fp16_two_slots_through_the_adapter", W.gpt2_xl_shapes(), F16, 1e-3, 2, 1, 10,
                    "c5_gpt2_xl_fp16_two_streams")
    pipeline("c5_gpt2_xl_fp16_one_stream", W.gpt2_xl_shapes(), F16, F16, 1e-3, 1, 1.0, 1, 1, 10)
    pipeline("c5_gpt2_xl_fp16_array_entry_points", W.gpt2_xl_shapes(), F16, F16, 1e-3, 1, 1.0, 2, 1, 10, arrays=True,
             note="pack and unpack of every cycle through hvdhip_batched_scaled_d2d_memcpy (the by-value launchers "
                  "of ops/gpu_operations.cc:186-206) instead of explicit plans: 96 distinct copy sets per step, "
                  "their tables resident in the library's cache after the first step")

    out.update(allgather_extra())
    out["device_copy_1GiB_three_ways"] = device_ceiling_extra()
    return out


# ----------------------------------------------------------------------------------------------
# HBM traffic of the headline's kernels, measured in this run
# ----------------------------------------------------------------------------------------------

def _counter_rows(path):
    import csv
    csv.field_size_limit(1 << 30)
    with open(path, newline="") as f:
        rows = list(csv.DictReader(f))
    rows.sort(key=lambda r: int(r["Start_Timestamp"]))
    return rows


def live_traffic(cfg="c1", launches=(2, 6), budget_s=240):
    """HBM bytes per launch of every kernel loop of `cfg`, from rocprofv3 runs started by this process:
    `bench.py --kernel-only cfg` under --pmc FETCH_SIZE and under --pmc WRITE_SIZE (KiB per dispatch),
    each scaled by what the same counter reads for `bench.py --calibrate`, two plain 256 MiB copies that
    are not the library's kernels.  Returns ({case: bytes}, note) or (None, why not).  Runs before this
    process touches the GPU; any failure only means that the committed figures are reported instead."""
    import glob
    import shutil
    import subprocess
    import tempfile
    if any(k.startswith("ROCPROF") or k.startswith("ROCP_") for k in os.environ):
        return None, "this run is itself under a profiler"
    if not shutil.which("rocprofv3"):
        return None, "rocprofv3 is not on PATH"
    warm, steps = launches
    per = warm + steps
    tmp = tempfile.mkdtemp(prefix="hvdhip_bench_", dir="/tmp")
    t0 = time.time()
    try:
        def run(tag, counter, tail):
            left = budget_s - (time.time() - t0)
            if left < 20:
                raise RuntimeError("out of time")
            cmd = ["rocprofv3", "--pmc", counter, "--output-format", "csv", "-d", os.path.join(tmp, tag), "-o", "c", "--",
                   sys.executable, os.path.join(ROOT, "bench.py")] + tail + ["--steps", str(steps), "--warmup", str(warm)]
            r = subprocess.run(cmd, cwd=ROOT, env=dict(os.environ, TMPDIR="/tmp"), stdout=subprocess.PIPE,
                               stderr=subprocess.DEVNULL, timeout=min(left, 120))
            if r.returncode != 0:
                raise RuntimeError("%s exited with %d" % (tag, r.returncode))
            found = glob.glob(os.path.join(tmp, tag, "**", "*counter_collection.csv"), recursive=True)
            if not found:
                raise RuntimeError("%s wrote no counter file" % tag)
            return r.stdout.decode(errors="replace"), _counter_rows(found[0])

        factors = {}
        for counter in ("FETCH_SIZE", "WRITE_SIZE"):
            _, rows = run("cal_" + counter, counter, ["--calibrate"])
            seen = []
            for frag in ("__amd_rocclr_copyBuffer", "vectorized_elementwise_kernel"):
                v = [float(r["Counter_Value"]) for r in rows if frag in r["Kernel_Name"] and r["Counter_Name"] == counter][-per:]
                if len(v) == per:
                    seen.append(262144.0 * len(v) / sum(v))
            if not seen or max(seen) / min(seen) > 1.01:
                raise RuntimeError("calibration kernels disagree or are missing: %s" % seen)
            factors[counter] = sum(seen) / len(seen)
        totals = {}
        for counter in ("FETCH_SIZE", "WRITE_SIZE"):
            out, rows = run(cfg + "_" + counter, counter, ["--kernel-only", cfg])
            info = json.loads(next(l for l in out.splitlines() if l.startswith("CASES "))[6:])
            lib = [r for r in rows if "hvdhip" in r["Kernel_Name"] and r["Counter_Name"] == counter]
            need = sum(per * len(c["parts"]) for c in info["cases"])
            if len(lib) < need:
                raise RuntimeError("%d dispatches of the library's kernels, %d expected" % (len(lib), need))
            lib = lib[len(lib) - need:]
            at = 0
            for c in info["cases"]:
                n = per * len(c["parts"])
                seg = lib[at + warm * len(c["parts"]):at + n]  # the warm-up launches lead
                at += n
                kib = sum(float(r["Counter_Value"]) for r in seg) / steps  # all kernels of one call together
                totals[c["case"]] = totals.get(c["case"], 0.0) + kib * 1024 * factors[counter]
        note = ("this run: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE over `bench.py --kernel-only %s` (%d launches), scaled by "
                "the same counters over `bench.py --calibrate` (x %.4f, x %.4f)"
                % (cfg, steps, factors["FETCH_SIZE"], factors["WRITE_SIZE"]))
        return {k: int(round(v)) for k, v in totals.items()}, note
    except Exception as e:  # the committed figures stand in
        return None, "%s: %s" % (type(e).__name__, e)
    finally:
        shutil.rmtree(tmp, ignore_errors=True)


# ----------------------------------------------------------------------------------------------
# output: one compact JSON line on stdout (it has to fit a reader's 8 KB window), everything on stderr
# ----------------------------------------------------------------------------------------------

# (a case's kernel is named in the profile that `case` leads to -- profiles/<config>_*_kernels.txt -- and on stderr)
KERNEL_COLUMNS = ["case", "launch_us", "us_median", "us_min", "us_max", "frac_of_8TBps", "algorithmic_B", "traffic_B",
                  "in_pipeline_us"]
PIPELINE_COLUMNS = ["algorithmic_GB/s", "frac_of_8TBps", "ms", "ms_median", "ms_min", "ms_max", "streams", "cpu_GB/s_1core"]


def kernel_row(b):
    m = b.get("launch_us_median_min_max") or [None, None, None]
    return [b["case"], b["launch_us"], m[0], m[1], m[2], b["frac"], b["algorithmic_bytes_per_launch"], b.get("traffic"),
            b.get("in_pipeline_us")]


def compact(result):
    """The line for stdout: the contract's keys in full, every other configuration as one row per
    pipeline and one row per kernel loop (columns named once)."""
    out = {k: v for k, v in result.items() if k != "extra"}
    out["config"] = {k: v for k, v in result["config"].items() if k != "value_is"}
    extra = result.get("extra")
    if not extra:
        return out
    if "error" in extra:
        out["extra"] = extra
        return out
    pipes, rows, seen = {}, [], set()
    for name, d in extra.items():
        if not isinstance(d, dict):
            continue
        if "algorithmic_GB/s" in d:
            m = d.get("ms_median_min_max") or [None, None, None]
            pipes[name] = [d["algorithmic_GB/s"], d["algorithmic_frac_of_8TBps"], d["ms"], m[0], m[1], m[2],
                           d.get("streams"), d.get("cpu_GB/s")]
            if "vs_python_pipeline" in d:
                pipes[name].append(d["vs_python_pipeline"])
        for b in d.get("kernels", []):
            if b["case"] not in seen:
                seen.add(b["case"])
                rows.append(kernel_row(b))
    out["extra"] = {"pipeline_columns": PIPELINE_COLUMNS + ["(adapter rows: python pipeline's ms / this ms)"],
                    "pipelines": pipes, "kernel_columns": KERNEL_COLUMNS, "kernels": rows}
    ex = extra.get("c2_fusion_stress", {}).get("execute_vs_per_tensor_copies")
    if ex:
        out["extra"]["c2_execute_vs_per_tensor_copies"] = ex
    if "cpu_error" in extra:
        out["extra"]["cpu_error"] = extra["cpu_error"]
    return out


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU's share of the hot path: this build has no inter-GPU collectives, "
              "run it with --gpus 1", file=sys.stderr)
        sys.exit(2)
    # The counter runs come first: child processes are started before this one has touched the GPU.
    measured, traffic_note = None, None
    if not (args.kernel_only or args.calibrate or args.no_live_traffic):
        measured, traffic_note = live_traffic("c1")
        if measured:
            TRAFFIC_BYTES_MEASURED.update(measured)
    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    import horovod_amd
    from horovod_amd import DTYPE, workloads as W
    from horovod_amd import build as native
    native.ensure_built()  # loads what is built; builds only if nothing is
    horovod_amd.lib()  # fails loudly if the HIP library cannot be loaded

    stream = stream_pair()[0]
    F32 = DTYPE["float32"]
    if args.calibrate:
        # Two plain 256 MiB device copies that are none of the library's kernels: the runtime's
        # hipMemcpyAsync (its own copy kernel) and an elementwise kernel of torch.  Each reads exactly
        # 262,144 KiB and writes exactly 262,144 KiB; what rocprofv3's FETCH_SIZE and WRITE_SIZE read
        # for them gives the factors that turn those counters into bytes.
        n = 256 << 20
        a = randn_bytes(n, torch.float32, 1.0, 77)
        b = torch.empty(n, dtype=torch.uint8, device="cuda")
        torch.cuda.synchronize()
        memcpy = horovod_amd.lib().hvdhip_memcpy_async
        ext = torch.cuda.ExternalStream(stream.handle.value)
        for _ in range(args.warmup + args.steps):
            horovod_amd.check(memcpy(b.data_ptr(), a.data_ptr(), n, 3, stream.handle), "hvdhip_memcpy_async")
        stream.synchronize()
        for _ in range(args.warmup + args.steps):
            with torch.cuda.stream(ext):
                torch.mul(a.view(torch.float32), 1.0, out=b.view(torch.float32))
        stream.synchronize()
        return

    if args.kernel_only:
        cases = build_cases(args.kernel_only)
        # what the launches below are, for whoever reads the profiler's output
        print("CASES " + json.dumps({"launches_per_case": args.warmup + args.steps,
                                     "cases": [{"case": c.key, "parts": c.parts, "workgroups": c.workgroups,
                                                "what": c.what} for c in cases]}), flush=True)
        for c in cases:
            for _ in range(args.warmup + args.steps):
                c.fn()
            stream.synchronize()
        return

    # ---- headline: C1, the whole pipeline on one stream
    run = PipelineRun(W.resnet50_shapes(), F32, F32, 1e-3, 1, 1.0, 1, 4)

    def step():
        for _ in range(REPS):
            run.one_pass()

    sec, each = timed(step, run.sync, args.steps, args.warmup, stream=stream)
    ab = run.algorithmic_bytes()
    value = REPS * ab / sec / 1e9
    payload = 4 * sum(run.counts)
    config = {"workload": "C1: ResNet-50 fp32 gradients, 161 tensors, 25,557,032 elements, N(0,1e-3); fused at a 64 MiB "
                          "threshold into %d cycles; per cycle pack with prescale 0.125 -> reduce-sum of the whole buffer "
                          "with one peer buffer on the device -> unpack (postscale 1.0); one stream, one persistent fusion "
                          "buffer; tensor sets rotate over %d replicas" % (len(run.pipe.cycles), len(run.reps)),
              "tensors": len(run.counts), "payload_bytes": payload, "cycles": len(run.pipe.cycles),
              "cycle_buffer_bytes": [c.plan.buffer_len for c in run.pipe.cycles], "fusion_threshold": W.FUSION_THRESHOLD,
              "peers": 1, "prescale": 0.125, "postscale": 1.0, "passes_per_step": REPS,
              "algorithmic_bytes_per_step": REPS * ab, "replicas_rotated": len(run.reps), "streams": 1,
              "value_is": "algorithmic bytes (pack P_in+P_buf, reduce 3C, unpack P_buf+P_out = 7P) / wall time; within a "
                          "cycle the fusion buffer passes from kernel to kernel through the Infinity Cache, so this is "
                          "not an HBM counter; the HBM claim is roofline.frac"}
    run.destroy()

    # ---- roofline: every kernel of the C1 cycle, the dominant one as the headline's block
    cases = build_cases("c1")
    blocks = measure_cases(cases, steps=200, warmup=20)
    release(cases)
    del cases
    torch.cuda.empty_cache()
    roofline = dict(next(b for b in blocks if b["case"] == "c1.reduce"))
    roofline.pop("timed", None)
    roofline["why_this_kernel"] = "the reduce-sum takes the largest share of the pipeline's kernel time (3C of 7P bytes)"
    roofline["traffic_from"] = traffic_note if measured else (
        "the committed summary %s (not measured in this run: %s)" % (TRAFFIC_PROFILE["c1"], traffic_note or "--no-live-traffic"))

    result = {
        "metric": "achieved HBM GB/s (% of 8 TB/s) for fused pack+scale+reduce+unpack; Adasum GB/s",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(sec * 1e3, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic", "config": config,
        # `value` counts algorithmic bytes over wall time; these three name what is what
        "value_kind": "algorithmic GB/s of the whole pipeline (hand-overs through the Infinity Cache included)",
        "hbm_GB/s": round(roofline["traffic"] / (roofline["launch_us"] * 1e-6) / 1e9, 1) if roofline.get("traffic") else None,
        "hbm_GB/s_is": "roofline.traffic / the roofline kernel's launch time",
        "algorithmic_frac_of_8TBps": round(value / HBM_PEAK_GBS, 4),
        "ms_per_step_median_min_max": spread(each, 1e3, 5),
        "ms_per_step_from": "a HIP event pair around each timed step",
        "roofline": roofline,
        "traffic_profile": TRAFFIC_PROFILE["c1"],
    }
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline_resnet()
    if not args.no_extra:
        # the extra configurations must never cost the headline line
        try:
            result["extra"] = extras(blocks)
        except Exception as e:  # pragma: no cover
            result["extra"] = {"error": "%s: %s" % (type(e).__name__, e)}
        if not args.no_cpu and "error" not in result["extra"]:
            try:
                for name, v in cpu_extras().items():
                    result["extra"][name].update(v)
            except Exception as e:  # pragma: no cover
                result["extra"]["cpu_error"] = "%s: %s" % (type(e).__name__, e)
    # everything, with the descriptions of what was timed, for whoever keeps stderr
    print("DETAIL " + json.dumps(result), file=sys.stderr, flush=True)
    line = json.dumps(compact(result), separators=(",", ":"))
    if len(line) > 8000:
        print("note: the stdout line is %d bytes" % len(line), file=sys.stderr)
    print(line)


if __name__ == "__main__":
    main()
