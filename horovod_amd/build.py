"""Builds the in-tree native libraries with make (hipcc for gfx950, g++ for the adapter, gcc for the
C99 example client)."""
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")


def build(force=False, jobs=8):
    """Runs make in csrc/; force=True rebuilds everything."""
    cmd = ["make", "-j%d" % jobs, "-C", CSRC]
    if force:
        cmd.insert(1, "-B")
    subprocess.check_call(cmd)


def ensure_built():
    """Builds the libraries only if one of them is missing; never replaces an existing build."""
    need = [os.path.join(_HERE, "lib", n) for n in ("libhvdhip.so", "libhvdhip_tuning.so", "libhvdhip_adapter.so", "c_client", "cache_stress")]
    if not all(os.path.exists(p) for p in need):
        build()
