"""The adapter's finalizer threads on the CPU, under ThreadSanitizer.

The reference hands the wait for a response's events to a finalizer thread so that its background
thread can launch the next response on the other stream slot (ops/gpu_operations.cc:50-99,
common/thread_pool.cc:30-64, one thread per slot common/operations.cc:449).  Here the adapter's own
sources are compiled with -fsanitize=thread against tests/native/fake_hvdhip.cc, a host-only model
of the C ABI (streams are worker threads, kernels are closures on host memory), and driven by
tests/native/finalizer_stress.cc: 300 responses over two slots with results checked, two responses
in flight at once, a failed event wait reaching every callback, inline completion without threads,
asynchronous completion, elastic polling with the timeline's events, the pool's own semantics, the
wait for tensors that another stream produces, and the allgather op's fusion-buffer offsets and copies.
ThreadSanitizer cannot run with the real device runtime (it does not find the GPU under the
sanitizer's memory layout), which is why the device is modelled."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_finalizer_threads_are_correct_and_race_free(tmp_path):
    exe = str(tmp_path / "finalizer_stress")
    srcs = [os.path.join(ROOT, "tests", "native", "finalizer_stress.cc"),
            os.path.join(ROOT, "tests", "native", "fake_hvdhip.cc"),
            os.path.join(ROOT, "horovod_amd", "csrc", "adapter", "hvd_hip_adapter.cc")]
    cmd = ["g++", "-std=c++14", "-O1", "-g", "-fsanitize=thread", "-Wall",
           "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(ROOT, "horovod_amd", "csrc", "adapter")] + srcs + \
          ["-pthread", "-o", exe]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-3000:]
    env = dict(os.environ, TSAN_OPTIONS="halt_on_error=0 exitcode=66")
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120, env=env)
    out = r.stdout + r.stderr
    assert r.returncode == 0, out[-4000:]
    assert "finalizer ok" in out
    assert "ThreadSanitizer" not in out, out[-4000:]
