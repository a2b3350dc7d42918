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


def test_bert_large_cycles_reduce_an_eighth():
    counts = [W.numel(s) for s in W.bert_large_shapes()]
    groups = W.fuse([2 * c for c in counts])
    assert len(groups) == 11
    for g in groups:
        n = sum((2 * counts[i] + 15) // 16 * 16 for i in g) // 2  # padded fp16 elements of the cycle
        per = W.reduce_scatter_share(n, 8)
        assert 0 <= per - n / 8 < 64
