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


def test_more_argument_errors_are_caught_before_the_device_is_touched():
    """Validation comes first in every entry point, so these calls must fail the same way on a
    machine without a GPU."""
    import horovod_amd
    L = horovod_amd.lib()
    D = horovod_amd.DTYPE
    one = (ctypes.c_void_p * 1)(16)
    cnt = (ctypes.c_int64 * 1)(-4)
    plan = ctypes.c_void_p()
    # a negative element count
    assert L.hvdhip_fusion_plan_create(one, one, cnt, 1, D["float32"], D["float32"], ctypes.byref(plan)) == -1
    assert b"negative" in L.hvdhip_last_error()
    cnt[0] = 4
    # only float32 tensors may travel in a float16 buffer
    assert L.hvdhip_fusion_plan_create(one, one, cnt, 1, D["int32"], D["float16"], ctypes.byref(plan)) == -2
    assert L.hvdhip_fusion_plan_create(one, one, cnt, 1, D["float16"], D["float32"], ctypes.byref(plan)) == -2
    assert L.hvdhip_fusion_plan_create(one, one, cnt, 1, 42, 42, ctypes.byref(plan)) == -2
    # misaligned for its element size
    odd = (ctypes.c_void_p * 1)(18)
    assert L.hvdhip_fusion_plan_create(odd, one, cnt, 1, D["float32"], D["float32"], ctypes.byref(plan)) == -1
    assert b"aligned" in L.hvdhip_last_error()
    # a NULL tensor with elements in it
    null = (ctypes.c_void_p * 1)(None)
    assert L.hvdhip_fusion_plan_create(null, one, cnt, 1, D["float32"], D["float32"], ctypes.byref(plan)) == -1
    assert L.hvdhip_fusion_plan_create(one, one, cnt, 1, D["float32"], D["float32"], None) == -1
    # pack / unpack / reduce / Adasum without a plan or with impossible arguments
    assert L.hvdhip_fusion_pack(None, None, 1.0, 0, None) == -1
    assert L.hvdhip_fusion_unpack(None, None, 1.0, None) == -1
    assert L.hvdhip_fusion_plan_buffer_len(None) == -1 and L.hvdhip_fusion_plan_num_chunks(None) == -1
    assert L.hvdhip_reduce_sum(None, None, -1, D["float32"], None) == -1
    assert L.hvdhip_reduce_sum(None, None, 0, D["bool"], None) == -2
    ad = ctypes.c_void_p()
    neg = (ctypes.c_int * 2)(5, -1)
    assert L.hvdhip_adasum_plan_create(neg, 2, D["float32"], ctypes.byref(ad)) == -1
    assert L.hvdhip_adasum_plan_create(neg, 2, D["int32"], ctypes.byref(ad)) == -2
    assert L.hvdhip_adasum_combine(None, None, None, None) == -1
    assert L.hvdhip_adasum_dispatch_scaled_add(D["float32"], -3, 1.0, None, 1.0, None, None) == -1
    sizes = (ctypes.c_size_t * 1)(6)
    assert L.hvdhip_batched_d2d_memcpy(one, one, sizes, -1, None) == -1
    assert L.hvdhip_batched_scaled_d2d_memcpy(one, one, sizes, 1, 0.5, D["float32"], None) == -1  # 6 is no multiple of 4
    assert L.hvdhip_batched_scaled_d2d_memcpy(one, one, sizes, 1, 0.5, D["bool"], None) == -2
    assert L.hvdhip_set_fp16_scale_mode(3) == -1 and L.hvdhip_get_fp16_scale_mode() == 0
    assert L.hvdhip_memcpy_async(None, None, 0, 9, None) == -1
    for code in (-1, -2, -3, -4, 1, 2, 700):
        assert L.hvdhip_error_string(code)


def test_shipped_library_reads_no_tuning_settings():
    """The chunk size and the store-policy table are fixed in the shipped library; only the tuning
    build (-DHVDHIP_TUNING, loaded by tests through HVDHIP_LIBRARY) looks at the environment for
    them.  HVDHIP_EVENT_SYSTEM_FENCE is a documented user setting and stays."""
    lib_dir = os.path.join(ROOT, "horovod_amd", "lib")
    shipped = open(os.path.join(lib_dir, "libhvdhip.so"), "rb").read()
    tuning = open(os.path.join(lib_dir, "libhvdhip_tuning.so"), "rb").read()
    for name in (b"HVDHIP_CHUNK_BYTES", b"HVDHIP_WRITE_THROUGH"):
        assert name not in shipped
        assert name in tuning
    assert b"HVDHIP_EVENT_SYSTEM_FENCE" in shipped
