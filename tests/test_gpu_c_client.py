"""The library driven from a plain C99 program (horovod_amd/csrc/examples/c_client.c): plan,
pack with prescale, reduce with a peer buffer, unpack with postscale, checked in C against
float arithmetic on the host.  No Python, torch or C++ is involved in the child process."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_c_client_round_trip(gpu):
    exe = os.path.join(ROOT, "horovod_amd", "lib", "c_client")
    assert os.path.exists(exe), "make -C horovod_amd/csrc"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=100)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "mismatches 0" in r.stdout
    print(r.stdout)


def test_native_cache_stress(gpu):
    """horovod_amd/csrc/examples/cache_stress.cc: copy-table cache with evictions on every call from
    two threads, a stream destroyed under it, the cache at its default size, single-layer Adasum
    plans beyond their capacity from two threads, plan and event lifetimes."""
    exe = os.path.join(ROOT, "horovod_amd", "lib", "cache_stress")
    assert os.path.exists(exe), "make -C horovod_amd/csrc"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=100)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "stress ok" in r.stdout
    print(r.stdout)
