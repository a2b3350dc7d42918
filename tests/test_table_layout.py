"""The chunk tables' host side without a GPU: tests/native/table_layout.cc is compiled (host code
only) together with horovod_amd/csrc/context.cc and checks, over random sets of segments and over
sizes around the group boundaries, that every chunk appears exactly once at the entry its workgroup
reads, that padding entries are empty, that the four workgroups of one XCD in a group of 32 share a
128-byte table line, that XCDs walk runs of consecutive chunks, and that the branch-free tile order
of the contiguous kernels is the same permutation."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_chunk_table_layout(tmp_path):
    exe = str(tmp_path / "table_layout")
    cmd = ["hipcc", "-std=c++17", "-O1", "-x", "hip", "--cuda-host-only", "-Wno-unused-function",
           "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(ROOT, "horovod_amd", "csrc"),
           os.path.join(ROOT, "tests", "native", "table_layout.cc"),
           os.path.join(ROOT, "horovod_amd", "csrc", "context.cc"), "-o", exe]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-3000:]
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and "table layout ok" in r.stdout, r.stdout[-2000:] + r.stderr[-2000:]
