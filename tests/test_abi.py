"""The C-ABI library loads and exports every function that include/hvdhip.h
declares (no GPU needed: nothing is launched)."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "hvdhip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hvdhip_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_surface():
    names = _declared()
    for must in ("hvdhip_batched_d2d_memcpy", "hvdhip_batched_scaled_d2d_memcpy", "hvdhip_scale_buffer",
                 "hvdhip_fusion_pack", "hvdhip_fusion_unpack", "hvdhip_reduce_sum", "hvdhip_reduce_sum_k",
                 "hvdhip_adasum_dot_and_norm_sqrds", "hvdhip_adasum_dispatch_scaled_add",
                 "hvdhip_adasum_combine", "hvdhip_stream_create", "hvdhip_event_acquire"):
        assert must in names


def test_library_exports_every_declared_symbol():
    import horovod_amd
    path = horovod_amd.lib_path()
    assert os.path.exists(path), "build the library first: make -C horovod_amd/csrc"
    cdll = ctypes.CDLL(path)
    missing = [n for n in _declared() if not hasattr(cdll, n)]
    assert not missing, missing


def test_python_prototypes_cover_the_header():
    from horovod_amd import _lib
    assert sorted(_lib._PROTOTYPES) == _declared()


def test_error_strings_and_dtype_sizes():
    import horovod_amd
    L = horovod_amd.lib()
    assert L.hvdhip_error_string(0) == b"success"
    assert b"not supported" in L.hvdhip_error_string(-2)
    sizes = [L.hvdhip_dtype_size(d) for d in range(10)]
    assert sizes == [1, 1, 2, 2, 4, 8, 2, 4, 8, 1]  # common/message.cc:66-92
    assert L.hvdhip_dtype_size(42) == -1


def test_argument_errors_need_no_gpu():
    import horovod_amd
    L = horovod_amd.lib()
    # dtype table of ScaleBuffer (ops/collective_operations.cc:141-144): UINT16 is rejected
    assert L.hvdhip_scale_buffer(None, None, 0, 0.5, horovod_amd.DTYPE["uint16"], None) == -2
    assert L.hvdhip_reduce_sum_k(None, None, 0, 10, horovod_amd.DTYPE["float32"], None) == -1
    assert b"outside 1..16" in L.hvdhip_last_error()
    assert L.hvdhip_reduce_sum(None, None, 0, horovod_amd.DTYPE["bool"], None) == -2


def test_missing_library_fails_loudly(monkeypatch):
    from horovod_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "lib_path", lambda: "/nonexistent/libhvdhip.so")
    try:
        _lib.lib()
    except RuntimeError as e:
        assert "no fallback" in str(e)
    else:
        raise AssertionError("loading a missing library must raise")


def test_header_is_plain_c99():
    """The boundary is a C ABI: the header must compile as C, warnings as errors."""
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-fsyntax-only", "-x", "c",
                        os.path.join(root, "include", "hvdhip.h")], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr


def test_c_client_is_built_with_the_library():
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    assert os.path.exists(os.path.join(root, "horovod_amd", "lib", "c_client")), \
        "make -C horovod_amd/csrc builds the C99 example next to the library"
