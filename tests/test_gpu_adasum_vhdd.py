"""How the Adasum path shards: vector halving, distance doubling on one GPU.

The reference combines W ranks' fused gradients with Adasum::FusedAllreduce
(ops/adasum/adasum.h:194-340): at level 1, 2, 4 ... every rank keeps one half of what it
holds, receives the matching half from rank ^ level, computes per-layer {dot, |a|^2, |b|^2}
on its piece, the pieces' triples are summed over the ranks that share the two vectors
(:380-382), and every rank applies the scaled add to its piece; the halves are gathered back
in reverse order.  Here the W ranks are W buffers on one device: the send/recv steps are
device copies, the small allreduce of triples is a host sum, and all arithmetic on vector
data goes through the library's split entry points (dot_norms / read / set_coeffs /
scaled_add) at exactly the slice shapes and per-slice layer counts a rank would see.  The
result must equal the pairwise tree that the oracle computes on whole vectors."""
import numpy as np
import pytest

from oracle_util import F16, F32, NP_OF, SIZE_OF

pytestmark = pytest.mark.gpu


def _split_counts(tensor_counts, my_count_total, upper):
    """The slicing of adasum.h:237-296 for one rank: returns (mine, neighbour's) per-layer counts.
    upper: the rank keeps the second half ((rank & level) != 0)."""
    first = my_count_total >> 1
    second = my_count_total - first
    mine, theirs = list(tensor_counts), [0] * len(tensor_counts)
    if upper:
        nghr, sofar = first, 0
        for i, c in enumerate(tensor_counts):
            if sofar <= nghr:
                if sofar + c <= nghr:
                    theirs[i], mine[i] = c, 0
                else:
                    theirs[i], mine[i] = nghr - sofar, c - (nghr - sofar)
            else:
                theirs[i] = 0
            sofar += theirs[i]
        return mine, theirs, second, first
    keep, sofar = first, 0
    for i, c in enumerate(tensor_counts):
        if sofar <= keep:
            if sofar + c <= keep:
                theirs[i] = 0
            else:
                theirs[i], mine[i] = c - (keep - sofar), keep - sofar
        else:
            theirs[i], mine[i] = c, 0
        sofar += mine[i]
    return mine, theirs, first, second


@pytest.mark.parametrize("world", [2, 4, 8])
@pytest.mark.parametrize("dtype", [F32, F16])
def test_vhdd_on_one_device_matches_the_pairwise_tree(gpu, orc, world, dtype):
    import horovod_amd
    L = horovod_amd.lib()
    rng = np.random.default_rng(40 + world)
    np_t, es = NP_OF[dtype], SIZE_OF[dtype]
    layer_counts = [7, 4099, 1, 30000, 12345, 2, 65536, 999]
    n = sum(layer_counts)
    host = [rng.standard_normal(n).astype(np_t) for _ in range(world)]
    raw = (lambda v: v.view(np.uint16)) if np_t == np.float16 else (lambda v: v)

    # the oracle: pairwise tree on whole vectors, distances 1, 2, 4 ...
    tree = [raw(v).copy() for v in host]
    d = 1
    while d < world:
        for i in range(0, world, 2 * d):
            tree[i] = orc.adasum_pairwise(tree[i], tree[i + d], layer_counts, dtype)[0]
        d *= 2
    want = tree[0]

    grad = [gpu.upload(raw(v)) for v in host]
    recv = [gpu.empty(n * es) for _ in range(world)]
    s = gpu.stream
    counts = [list(layer_counts) for _ in range(world)]
    my_count = [n] * world
    start = [0] * world            # element offset of the piece a rank currently holds
    history = []                   # per level: per rank (neighbour's counts, neighbour's total)
    plans = []

    def copy(dst, dst_off, src, src_off, nelem):
        if nelem:
            horovod_amd.check(L.hvdhip_memcpy_async(dst.data_ptr() + dst_off * es, src.data_ptr() + src_off * es,
                                                    nelem * es, 3, s.handle), "hvdhip_memcpy_async")

    level = 1
    while level < world:
        split = []
        for r in range(world):
            upper = (r & level) != 0
            mine, theirs, keep, give = _split_counts(counts[r], my_count[r], upper)
            split.append((upper, mine, theirs, keep, give))
        # send/recv: every rank receives, from rank ^ level, the half that it keeps
        for r in range(world):
            upper, mine, theirs, keep, give = split[r]
            nb = r ^ level
            new_start = start[r] + (give if upper else 0)
            copy(recv[r], new_start, grad[nb], new_start, keep)
        s.synchronize()
        triples = []
        level_plans = []
        for r in range(world):
            upper, mine, theirs, keep, give = split[r]
            if upper:
                start[r] += give
            counts[r], my_count[r] = mine, keep
            plan = gpu.H.AdasumPlan(mine, dtype)
            level_plans.append(plan)
            plan.dot_norms(grad[r].data_ptr() + start[r] * es, recv[r].data_ptr() + start[r] * es, s)
            nd, _ = plan.read(s)
            nd = np.array(nd).reshape(-1, 3)
            if upper:  # the right neighbour stores its own norm in the third place (adasum.h:370-376)
                nd = nd[:, [0, 2, 1]]
            triples.append(nd)
        history.append([(split[r][2], split[r][4]) for r in range(world)])
        # the allreduce of 3 doubles per layer over the ranks that share the two vectors
        group = 2 * level
        for g0 in range(0, world, group):
            total = np.zeros_like(triples[g0])
            for r in range(g0, g0 + group):
                total = total + triples[r]
            for r in range(g0, g0 + group):
                upper = (r & level) != 0
                coeffs = []
                for dot, left, right in total:
                    an, bn = (right, left) if upper else (left, right)
                    ca, cb = orc.adasum_coeffs(dot, an, bn)
                    coeffs += [ca, cb]
                level_plans[r].set_coeffs(coeffs, s)
                level_plans[r].scaled_add(grad[r].data_ptr() + start[r] * es, recv[r].data_ptr() + start[r] * es, s)
        s.synchronize()
        plans += level_plans
        level <<= 1

    # gather the halves back, largest distance first (adasum.h:310-338)
    level = world >> 1
    while level > 0:
        theirs_now = history.pop()
        moves = []
        for r in range(world):
            nb = r ^ level
            upper = (r & level) != 0
            give = theirs_now[r][1]
            src_off = start[nb]
            moves.append((r, nb, src_off, my_count[nb]))
        for r, nb, src_off, nelem in moves:
            copy(grad[r], src_off, grad[nb], src_off, nelem)
        s.synchronize()
        for r in range(world):
            upper = (r & level) != 0
            nghr_counts, give = theirs_now[r]
            if upper:
                start[r] -= give
            my_count[r] += give
            counts[r] = [a + b for a, b in zip(counts[r], nghr_counts)]
        level >>= 1

    out = [gpu.download(g, np.uint16 if np_t == np.float16 else np_t) for g in grad]
    for p in plans:
        p.destroy()
    assert all(c == layer_counts for c in counts) and all(m == n for m in my_count) and all(x == 0 for x in start)
    for r in range(1, world):
        assert np.array_equal(out[r], out[0]), "rank %d differs from rank 0" % r
    if dtype == F16:
        diff = np.abs(out[0].view(np.float16).astype(np.float32) - want.view(np.float16).astype(np.float32))
        scale = np.abs(want.view(np.float16).astype(np.float32)) + 1e-3
        assert np.max(diff / scale) <= 2e-3 * world  # one half ulp per level, compounded
    else:
        ulp = np.abs(out[0].view(np.int32).astype(np.int64) - want.view(np.int32).astype(np.int64))
        assert ulp.max() <= 4 * world, ulp.max()
