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
