"""Host-side arithmetic of the bench/test driver that needs no GPU."""
import os

from horovod_amd import workloads as W

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_reduce_scatter_share_follows_the_reference():
    # ops/nccl_operations.cc:289-316: a fused buffer grows to a multiple of local_size * 64 elements
    # (FUSION_BUFFER_ATOMIC_UNIT, common/common.h:146) and is divided evenly
    assert W.reduce_scatter_share(512, 8) == 64
    assert W.reduce_scatter_share(513, 8) == 128          # rounded up to 1,024, not down to 512
    assert W.reduce_scatter_share(1023, 8) == 128
    assert W.reduce_scatter_share(1, 8) == 64
    assert W.reduce_scatter_share(0, 8) == 0
    assert W.reduce_scatter_share(33554432, 8) == 4194304  # a full 64 MiB fp16 cycle divides exactly
    assert W.reduce_scatter_share(33554433, 8) == 4194304 + 64
    for world in (2, 4, 8, 16):
        for n in (1, 63, 64, 65, 1000003, 2 ** 25 - 1):
            per = W.reduce_scatter_share(n, world)
            assert per % 64 == 0 and per * world >= n and (per - 64) * world < n
    # a single tensor is not grown: its remainder is reduced separately at the last rank
    assert W.reduce_scatter_share(1003, 8, fused=False) == 125


def test_reduce_scatter_ranges_cover_the_buffer_once():
    # ops/nccl_operations.cc:308-330: shares at rank * share; the non-divisible rest of a single tensor
    # goes to the last rank, right behind its share
    for world in (1, 2, 3, 8):
        for n in (0, 1, 7, 64, 1003, 65537):
            for fused in (True, False):
                ranges = W.reduce_scatter_ranges(n, world, fused)
                assert len(ranges) == world
                at = 0
                for first, count in ranges:
                    assert first == at and count >= 0
                    at += count
                if fused:
                    assert at >= n and at % (world * 64) == 0 and at - n < world * 64
                else:
                    assert at == n
                    assert all(c == n // world for _, c in ranges[:-1])
    assert W.reduce_scatter_ranges(1003, 8, fused=False)[-1] == (875, 128)


def test_bert_large_cycles_reduce_an_eighth():
    counts = [W.numel(s) for s in W.bert_large_shapes()]
    groups = W.fuse([2 * c for c in counts])
    assert len(groups) == 11
    for g in groups:
        n = sum((2 * counts[i] + 15) // 16 * 16 for i in g) // 2  # padded fp16 elements of the cycle
        per = W.reduce_scatter_share(n, 8)
        assert 0 <= per - n / 8 < 64


def _profile_rows(path):
    """(factors, rows) of a kernel summary under profiles/: the calibration factors and the table."""
    import re
    text = open(os.path.join(ROOT, path)).read()
    m = re.search(r"calibration factors: FETCH_SIZE x ([0-9.]+)\s+WRITE_SIZE x ([0-9.]+)", text)
    factors = (float(m.group(1)), float(m.group(2)))
    lines = text.splitlines()
    head = next(i for i, l in enumerate(lines) if l.startswith("case | kernel |"))
    cols = [c.strip() for c in lines[head].split("|")]
    rows = []
    for l in lines[head + 1:]:
        if "|" not in l:
            break
        rows.append(dict(zip(cols, [c.strip() for c in l.split("|")])))
    return factors, rows


def test_traffic_constants_of_the_bench_follow_from_the_profiles():
    """bench.py reports `roofline.traffic` from constants measured once with rocprofv3; each must be
    what the committed summary's own counter averages and calibration factors give.  The factors
    come from two copy kernels that are not the library's (the runtime's and torch's), each of known
    size: FETCH_SIZE counts in units of two KiB-counts per KiB read on this device, so its factor is
    2.  With them no kernel may read less than its algorithmic read bytes: everything comes from HBM."""
    import importlib.util
    spec = importlib.util.spec_from_file_location("bench_module", os.path.join(ROOT, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    seen, in_pipeline = {}, {}
    for cfg, path in bench.TRAFFIC_PROFILE.items():
        (ff, wf), rows = _profile_rows(path)
        assert 1.99 < ff < 2.01 and 0.99 < wf < 1.01, (path, ff, wf)
        text = open(os.path.join(ROOT, path)).read()
        assert "__amd_rocclr_copyBuffer" in text and "vectorized_elementwise_kernel" in text  # the calibration kernels
        for r in rows:
            read_b = float(r["FETCH_KiB"]) * 1024 * ff
            written_b = float(r["WRITE_KiB"]) * 1024 * wf
            assert abs(read_b - int(r["read_B"])) <= 1 and abs(written_b - int(r["written_B"])) <= 1, r
            assert abs(read_b + written_b - int(r["traffic_B"])) <= 1, r
            alg = int(r["algorithmic_B"])
            assert abs(int(r["traffic_B"]) / alg - float(r["traffic/algorithmic"])) < 1e-3
            assert abs(alg / float(r["avg_ns"]) / 8000.0 - float(r["frac"])) < 1e-4
            # every byte comes from HBM: no row reads less than it must, and none re-reads (within 4 %)
            alg_read = int(r["algorithmic_read_B"])
            assert 0 < alg_read <= alg
            # (the fetch factor is an average over the calibration launches, good to 1 part in 10^4)
            assert int(r["read_B"]) >= 0.9998 * alg_read, r
            assert int(r["written_B"]) >= 0.9998 * (alg - alg_read), r
            assert 0.9998 < int(r["traffic_B"]) / alg < 1.04, r
            # the same reads counted request by request (32, 64 and 128-byte requests, exact sizes): never
            # less than the algorithmic reads, and at most 2 % more (the chunk table, fetched once)
            by_request = 32 * float(r["RDREQ_32B"]) + 64 * float(r["RDREQ_64B"]) + 128 * float(r["RDREQ_128B"])
            assert abs(by_request - int(r["read_B_by_request"])) <= 64, r
            assert alg_read <= by_request <= 1.02 * alg_read, r
            assert by_request <= int(r["read_B"]) * 1.0003, r
            seen[r["case"]] = seen.get(r["case"], 0) + int(r["traffic_B"])
            pair = r["case"].split("+")
            if len(pair) == 2 and "xfer_k" in r["kernel"]:  # the unpack behind its reduce-sum
                in_pipeline[pair[0].split(".")[0] + "." + pair[1]] = float(r["avg_ns"])
    assert seen == bench.TRAFFIC_BYTES_MEASURED
    assert in_pipeline == bench.IN_PIPELINE_NS_MEASURED


def _bench():
    import importlib.util
    spec = importlib.util.spec_from_file_location("bench_module", os.path.join(ROOT, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    return bench


def test_spread_is_median_min_max():
    bench = _bench()
    assert bench.spread([3.0, 1.0, 2.0]) == [2.0, 1.0, 3.0]
    assert bench.spread([4.0, 1.0, 2.0, 3.0]) == [2.5, 1.0, 4.0]
    assert bench.spread([0.001234567], scale=1e3, digits=3) == [1.235, 1.235, 1.235]


def test_the_stdout_line_stays_inside_a_readers_window():
    """bench.py prints one JSON line that a reader who keeps the last 8 KB must see whole: built here
    from a result of the shape a full run produces (every pipeline and kernel loop the benchmark has,
    with realistic figures), the compact line has every contract key and stays under 8,000 bytes."""
    import json
    bench = _bench()
    block = {"bound": "hbm", "kernel": "reduce_k<_Float16, 7, 1> + xfer_k<Copy<unsigned short>, 1, 0>", "case": "c1.pack_rotating_destination",
             "launch_us": 123.45, "launch_us_median_min_max": [123.45, 122.22, 125.67], "timed_batches": 10,
             "algorithmic_bytes_per_launch": 2147483648, "achieved": 6543.2, "peak": 8000.0, "unit": "GB/s", "frac": 0.8179,
             "traffic": 2164248147, "workgroups": 262144, "timed": "x" * 300, "in_pipeline_us": 18.11}
    pipe = {"algorithmic_GB/s": 6543.2, "algorithmic_frac_of_8TBps": 0.8179, "ms": 3.1453, "ms_median_min_max": [3.1481, 3.1155, 3.1734],
            "algorithmic_MB": 21468.2, "cycles": 49, "streams": 2, "peers": 1, "reduce": "k-way", "cpu_GB/s": 52.04,
            "completion_event_per_cycle": True, "replicas_rotated": 1, "note": "y" * 400, "vs_python_pipeline": 0.9956}
    names = ["c1_resnet50_fp32_one_stream", "c1_resnet50_fp32_one_slot_through_the_adapter", "c1_resnet50_fp32_two_streams",
             "c1_resnet50_fp32_one_stream_completion_events", "c2_fusion_stress", "c2_fusion_stress_one_stream_completion_events",
             "c2_fusion_stress_one_stream_completion_events_with_unpack", "c2_fusion_stress_two_streams",
             "c2_fusion_stress_two_streams_no_completion_events", "c3_bert_large_fp32_to_fp16_7peers_eighth_share",
             "c3_bert_large_postscale_4", "c3_bert_large_two_streams", "c4_adasum_fp32_2x32M_64layers", "c4_adasum_fp16_2x32M_64layers",
             "c4_adasum_fp32_split_with_host_round_trip", "c5_gpt2_xl_fp16_two_streams", "c5_gpt2_xl_fp16_two_slots_through_the_adapter", "c5_gpt2_xl_fp16_one_stream",
             "c5_gpt2_xl_fp16_array_entry_points", "allgather_fusion_8ranks_128entries_6MB_slab",
             "allgather_fusion_8ranks_128entries_66MB_slab"]
    extra = {}
    k = 0
    for i, n in enumerate(names):
        extra[n] = dict(pipe)
        if i < 5:  # 30 kernel loops in all, as a full run has
            extra[n]["kernels"] = []
            for _ in range(6):
                b = dict(block)
                b["case"] = "c%d.unpack_postscale%02d" % (i % 5 + 1, k)
                k += 1
                extra[n]["kernels"].append(b)
    extra["c2_fusion_stress"]["execute_vs_per_tensor_copies"] = {"offset_table_kernels_ms": 0.075, "per_tensor_copies_ms": 4.7525, "speedup": 63.4}
    roofline = dict(block, why_this_kernel="z" * 90, traffic_from="w" * 200)
    roofline.pop("timed")
    result = {"metric": "achieved HBM GB/s (% of 8 TB/s) for fused pack+scale+reduce+unpack; Adasum GB/s", "value": 6716.0, "unit": "GB/s",
              "n_gpus": 1, "steps": 20, "warmup": 5, "ms_per_step": 5.32758, "higher_is_better": True, "scaling": "weak",
              "vs_baseline": None, "dtype": "f32", "data": "synthetic",
              "config": {"workload": "v" * 340, "tensors": 161, "payload_bytes": 102228128, "cycles": 2,
                         "cycle_buffer_bytes": [62529792, 39698432], "fusion_threshold": 67108864, "peers": 1, "prescale": 0.125,
                         "postscale": 1.0, "passes_per_step": 50, "algorithmic_bytes_per_step": 35779845000, "replicas_rotated": 4,
                         "streams": 1, "value_is": "u" * 300},
              "value_kind": "t" * 100, "hbm_GB/s": 6295.3, "hbm_GB/s_is": "s" * 55, "algorithmic_frac_of_8TBps": 0.8395,
              "ms_per_step_median_min_max": [5.32095, 5.31297, 5.32813], "ms_per_step_from": "r" * 40, "roofline": roofline,
              "traffic_profile": "profiles/c1_resnet50_fp32_kernels.txt",
              "cpu_baseline": {"value": 53.094, "unit": "GB/s", "cores": 1, "kind": "port", "sample": "q" * 210}, "extra": extra}
    line = json.dumps(bench.compact(result), separators=(",", ":"))
    assert len(line) < 7800, len(line)  # every row here is as long as the longest real one: a real line is under 6,500
    back = json.loads(line)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in back
    assert len(back["extra"]["pipelines"]) == len(names) and len(back["extra"]["kernels"]) == 30
    assert back["extra"]["kernel_columns"][0] == "case" and len(back["extra"]["kernels"][0]) == len(back["extra"]["kernel_columns"])
