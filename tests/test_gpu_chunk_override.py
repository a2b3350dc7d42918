"""Library settings that are read from the environment once per process, exercised in child
processes.  The chunk size and the store-policy mask are tuning settings that only
libhvdhip_tuning.so reads (the same sources built with -DHVDHIP_TUNING; the shipped library reads
neither): the child processes load that build through HVDHIP_LIBRARY.

The kernels' multi-vector (unrolled) inner loops only run when a workgroup's chunk holds more
than 1,024 vectors; the default 4 KiB chunks never reach them for transfers: the pack / scale /
reduce parity tests run once more with 64 KiB chunks.

Every streaming kernel exists with write-through buffer stores and with non-temporal global
stores, and a built-in table picks one per kernel family: the same parity tests run with every
family forced to the one and to the other.

Pooled events can be created without the system-scope fence; the tests that depend on completion
events run once more that way."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TUNING = os.path.join(ROOT, "horovod_amd", "lib", "libhvdhip_tuning.so")


def test_parity_with_64_kib_chunks(gpu):
    env = dict(os.environ, HVDHIP_CHUNK_BYTES="65536", HVDHIP_LIBRARY=TUNING)
    cmd = [sys.executable, "-m", "pytest", "-q", "-x", "-m", "gpu", "--timeout", "300", "--timeout-method", "thread",
           os.path.join(ROOT, "tests", "test_gpu_pack.py"), os.path.join(ROOT, "tests", "test_gpu_scale_reduce.py"),
           os.path.join(ROOT, "tests", "test_gpu_adasum.py"), "-p", "no:cacheprovider"]
    r = subprocess.run(cmd, cwd=ROOT, env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, timeout=900)
    tail = r.stdout.decode(errors="replace")[-3000:]
    assert r.returncode == 0, tail
    assert " passed" in tail and "failed" not in tail


def test_parity_with_unpack_tables_of_their_own(gpu):
    """HVDHIP_UNPACK_CHUNK_BYTES=8192: every plan then keeps a second chunk table for its unpack (as
    the converting plans always do), cut into chunks of another size than its pack's."""
    env = dict(os.environ, HVDHIP_UNPACK_CHUNK_BYTES="8192", HVDHIP_LIBRARY=TUNING)
    cmd = [sys.executable, "-m", "pytest", "-q", "-x", "-m", "gpu", "--timeout", "300", "--timeout-method", "thread",
           os.path.join(ROOT, "tests", "test_gpu_pack.py"), os.path.join(ROOT, "tests", "test_gpu_configs.py"),
           "-p", "no:cacheprovider"]
    r = subprocess.run(cmd, cwd=ROOT, env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, timeout=900)
    tail = r.stdout.decode(errors="replace")[-3000:]
    assert r.returncode == 0, tail
    assert " passed" in tail and "failed" not in tail


@pytest.mark.parametrize("mask", ["0", "0x1ff"])
def test_parity_with_every_kernel_family_on_one_store_policy(gpu, mask):
    env = dict(os.environ, HVDHIP_WRITE_THROUGH=mask, HVDHIP_LIBRARY=TUNING)
    files = ["test_gpu_pack.py", "test_gpu_scale_reduce.py", "test_gpu_adasum.py", "test_gpu_configs.py"]
    cmd = [sys.executable, "-m", "pytest", "-q", "-x", "-m", "gpu", "--timeout", "300", "--timeout-method", "thread"] + \
          [os.path.join(ROOT, "tests", f) for f in files] + ["-p", "no:cacheprovider"]
    r = subprocess.run(cmd, cwd=ROOT, env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, timeout=900)
    tail = r.stdout.decode(errors="replace")[-3000:]
    assert r.returncode == 0, tail
    assert " passed" in tail and "failed" not in tail


def test_pooled_events_without_the_system_scope_fence(gpu):
    """HVDHIP_EVENT_SYSTEM_FENCE=0: completion events that order work on the device only.  The
    tests that wait on such events and then read results back must still pass."""
    env = dict(os.environ, HVDHIP_EVENT_SYSTEM_FENCE="0")
    files = ["test_gpu_context.py", "test_gpu_adapter.py", "test_gpu_torch_api.py", "test_gpu_torch_optimizer.py"]
    cmd = [sys.executable, "-m", "pytest", "-q", "-x", "-m", "gpu", "--timeout", "300", "--timeout-method", "thread"] + \
          [os.path.join(ROOT, "tests", f) for f in files] + ["-p", "no:cacheprovider"]
    r = subprocess.run(cmd, cwd=ROOT, env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, timeout=900)
    tail = r.stdout.decode(errors="replace")[-3000:]
    assert r.returncode == 0, tail
    assert " passed" in tail and "failed" not in tail
