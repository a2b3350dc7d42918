"""Pins the oracle's fusion planner (common/controller.cc:463-481,793-866) with
hand-computed cases and a brute-force replay of the queue discipline."""
from collections import deque

import numpy as np


def _replay(sizes, keys, threshold, pad16):
    """Independent queue-based replay of the greedy fusion with look-ahead."""
    pad = (lambda s: 16 * ((s + 15) // 16)) if pad16 else (lambda s: s)
    q = deque(range(len(sizes)))
    groups = [-1] * len(sizes)
    g = 0
    while q:
        head = q.popleft()
        groups[head] = g
        total = pad(sizes[head])
        skipped, skipped_size = [], 0
        while q:
            j = q[0]
            if keys[j] == keys[head] and total + pad(sizes[j]) <= threshold:
                total += pad(sizes[j])
                groups[j] = g
                q.popleft()
            else:
                skipped_size += pad(sizes[j])
                if total + skipped_size <= threshold:
                    skipped.append(q.popleft())
                else:
                    break
        for j in reversed(skipped):
            q.appendleft(j)
        g += 1
    return g, groups


def test_threshold_rounding(orc):
    # local_size * 8 * 64 granularity on a homogeneous cluster
    assert orc.fusion_threshold(64 * 1024 * 1024, 8) == 64 * 1024 * 1024
    assert orc.fusion_threshold(1000, 1) == 1024
    assert orc.fusion_threshold(4097, 8) == 8192
    assert orc.fusion_threshold(1000, 8, homogeneous=False) == 1000


def test_hand_computed_groups(orc):
    # threshold 100, no padding: [40,40] [30,60] [200] [10]
    n, g = orc.fuse_responses([40, 40, 30, 60, 200, 10], 100, pad16=False)
    # 40+40=80; +30 does not fit -> skipped (80+30=110 > 100) -> close.  30+60=90; 200 cannot be skipped.
    assert n == 4 and list(g) == [0, 0, 1, 1, 2, 3]


def test_lookahead_skips_an_incompatible_response(orc):
    # keys: the fp16 tensor in the middle is skipped while it still fits in the look-ahead budget
    n, g = orc.fuse_responses([16, 16, 16, 16], 64, pad16=False, keys=[0, 1, 0, 0])
    assert n == 2 and list(g) == [0, 1, 0, 0]
    # with a tighter budget the look-ahead stops at the incompatible one
    n, g = orc.fuse_responses([32, 32, 16, 16], 48, pad16=False, keys=[0, 1, 0, 0])
    assert list(g) == [0, 1, 2, 2]


def test_padding_counts_toward_the_threshold(orc):
    # three 17-byte tensors pad to 32 each: only two fit in 64
    n, g = orc.fuse_responses([17, 17, 17], 64, pad16=True)
    assert list(g) == [0, 0, 1]
    n, g = orc.fuse_responses([17, 17, 17], 64, pad16=False)
    assert list(g) == [0, 0, 0]


def test_oversized_tensor_is_alone(orc):
    n, g = orc.fuse_responses([10, 1000, 10, 10], 100, pad16=False)
    assert list(g) == [0, 1, 2, 2]


def test_against_queue_replay(orc):
    rng = np.random.default_rng(21)
    for trial in range(200):
        n = int(rng.integers(1, 40))
        sizes = [int(x) for x in rng.integers(1, 300, n)]
        keys = [int(x) for x in rng.integers(0, 3, n)]
        thr = int(rng.integers(50, 800))
        pad16 = bool(trial % 2)
        want_n, want = _replay(sizes, keys, thr, pad16)
        got_n, got = orc.fuse_responses(sizes, thr, pad16=pad16, keys=keys)
        assert got_n == want_n and list(got) == want, (sizes, keys, thr, pad16)
