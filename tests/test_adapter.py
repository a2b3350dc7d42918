"""Host-side adapter (the C++ mirror of the reference's op-layer classes):
what can be checked without a GPU."""
import ctypes
import os

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ADAPTER = os.path.join(ROOT, "horovod_amd", "lib", "libhvdhip_adapter.so")


def _load():
    import horovod_amd
    horovod_amd.lib()
    assert os.path.exists(ADAPTER), "build the adapter first: make -C horovod_amd/csrc"
    return ctypes.CDLL(ADAPTER)


def test_adapter_loads_and_exports_its_test_surface():
    lib = _load()
    for name in ("hvd_adapter_create", "hvd_adapter_destroy", "hvd_adapter_allreduce", "hvd_adapter_state",
                 "hvd_adapter_adasum_pairwise", "hvd_adapter_adasum_dispatch", "hvd_adapter_fuse",
                 "hvd_adapter_fuse_keyed", "hvd_adapter_allreduce_wire"):
        assert hasattr(lib, name)


def test_fuse_responses_matches_the_oracle(orc):
    lib = _load()
    rng = np.random.default_rng(31)
    for trial in range(200):
        n = int(rng.integers(1, 60))
        sizes = rng.integers(1, 400, n).astype(np.int64)
        thr = int(rng.integers(50, 1200))
        pad = trial % 2
        groups = np.full(n, -1, np.int32)
        got_n = lib.hvd_adapter_fuse(ctypes.c_void_p(sizes.ctypes.data), n, ctypes.c_int64(thr), pad,
                                     ctypes.c_void_p(groups.ctypes.data))
        want_n, want = orc.fuse_responses(sizes, thr, pad16=bool(pad))
        assert got_n == want_n and np.array_equal(groups, want)


def test_fuse_responses_with_mixed_keys_matches_the_oracle(orc):
    """Mixed-precision queues: responses of another dtype or with other scale factors are
    looked past, not fused (common/controller.cc:831-856)."""
    lib = _load()
    rng = np.random.default_rng(32)
    for trial in range(300):
        n = int(rng.integers(1, 60))
        sizes = rng.integers(1, 400, n).astype(np.int64)
        keys = rng.integers(0, int(rng.integers(1, 4)), n).astype(np.int32)
        thr = int(rng.integers(50, 1200))
        pad = trial % 2
        groups = np.full(n, -1, np.int32)
        got_n = lib.hvd_adapter_fuse_keyed(ctypes.c_void_p(sizes.ctypes.data), ctypes.c_void_p(keys.ctypes.data), n,
                                           ctypes.c_int64(thr), pad, ctypes.c_void_p(groups.ctypes.data))
        want_n, want = orc.fuse_responses(sizes, thr, pad16=bool(pad), keys=keys)
        assert got_n == want_n and np.array_equal(groups, want)
        for g in range(got_n):
            assert len(set(keys[groups == g])) == 1


def test_python_planner_matches_the_oracle(orc):
    from horovod_amd import workloads as W
    for shapes, es in ((W.resnet50_shapes(), 4), (W.gpt2_xl_shapes(), 2), (W.bert_large_shapes(), 2)):
        nbytes = [es * W.numel(s) for s in shapes]
        groups = W.fuse(nbytes, W.FUSION_THRESHOLD)
        n, g = orc.fuse_responses(nbytes, W.FUSION_THRESHOLD, pad16=True)
        assert n == len(groups)
        for gi, members in enumerate(groups):
            assert all(g[i] == gi for i in members)
    # tensor counts named by the configurations
    assert len(W.resnet50_shapes()) == 161 and sum(W.numel(s) for s in W.resnet50_shapes()) == 25557032
    assert len(W.gpt2_xl_shapes()) == 580 and sum(W.numel(s) for s in W.gpt2_xl_shapes()) == 1557611200
    assert len(W.bert_large_shapes()) == 397
    c = W.adasum_layer_counts()
    assert len(c) == 64 and sum(c) == 1 << 25 and min(c) >= 1
    c = W.stress_counts()
    assert len(c) == 1024 and min(c) >= 256 and max(c) <= 65536
