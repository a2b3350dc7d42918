"""Pins the oracle's allgather fusion-buffer restatement
(ops/collective_operations.cc:200-275) by its closed form: output ec is the
concatenation over ranks of that entry's per-rank tensor."""
import numpy as np

from oracle_util import F32, U8


def _case(rng, size, n, np_t):
    return [[rng.integers(0, 200, int(rng.integers(0, 50))).astype(np_t) for _ in range(n)] for _ in range(size)]


def test_outputs_are_rank_wise_concatenations(orc):
    rng = np.random.default_rng(41)
    for size, n in ((1, 1), (2, 3), (4, 5), (8, 2), (3, 7)):
        per_rank = _case(rng, size, n, np.float32)
        outs, displ, offs = orc.allgather(per_rank, F32)
        for ec in range(n):
            want = np.concatenate([per_rank[rc][ec] for rc in range(size)])
            assert np.array_equal(outs[ec], want)
        # displacements are the exclusive prefix sum of the per-rank totals
        totals = [sum(t.size for t in per_rank[rc]) for rc in range(size)]
        assert list(displ) == [sum(totals[:rc]) for rc in range(size)]
        # inside rank rc's slab the entries follow one another
        for rc in range(size):
            for ec in range(n):
                assert offs[ec, rc] == displ[rc] + sum(per_rank[rc][k].size for k in range(ec))


def test_hand_computed_offsets(orc):
    # 2 ranks, 2 entries; sizes[entry][rank] = [[2, 3], [1, 4]] -> recvcounts [3, 7], displacements [0, 3]
    per_rank = [[np.arange(2, dtype=np.uint8), np.arange(1, dtype=np.uint8) + 10],
                [np.arange(3, dtype=np.uint8) + 20, np.arange(4, dtype=np.uint8) + 30]]
    outs, displ, offs = orc.allgather(per_rank, U8)
    assert list(displ) == [0, 3]
    assert offs.tolist() == [[0, 3], [2, 6]]
    assert outs[0].tolist() == [0, 1, 20, 21, 22] and outs[1].tolist() == [10, 30, 31, 32, 33]
