"""The reference scales fp16 buffers with two arithmetics: its CPU path multiplies in fp32
by the fp32 factor (ops/collective_operations.h:99-127), its CUDA kernels round the factor
to half first and multiply half by half (ops/cuda/cuda_kernels.cu:96-136,167,306-309).
hvdhip_set_fp16_scale_mode selects which one every fp16 scale of the library reproduces;
each must match its oracle bit for bit on every entry point that scales fp16."""
import numpy as np
import pytest

from oracle_util import F16, F32

pytestmark = pytest.mark.gpu

FACTORS = [0.1915194503788923, 1.0 / 3.0, 7.7, 1e-3, 0.125]


@pytest.fixture()
def half_factor_mode(gpu):
    assert gpu.H.get_fp16_scale_mode() == gpu.H.FP16_SCALE_FP32_FACTOR
    gpu.H.set_fp16_scale_mode(gpu.H.FP16_SCALE_HALF_FACTOR)
    yield
    gpu.H.set_fp16_scale_mode(gpu.H.FP16_SCALE_FP32_FACTOR)


def _all_halves():
    h = np.arange(65536, dtype=np.uint16)
    return h[~np.isnan(h.view(np.float16))]


def test_mode_is_validated(gpu):
    import horovod_amd
    with pytest.raises(horovod_amd.HvdHipError) as e:
        gpu.H.set_fp16_scale_mode(7)
    assert e.value.code == -1
    assert gpu.H.get_fp16_scale_mode() == gpu.H.FP16_SCALE_FP32_FACTOR


@pytest.mark.parametrize("factor", FACTORS)
def test_scale_buffer_and_scaled_copy(gpu, orc, half_factor_mode, factor):
    h = _all_halves()
    want = orc.scale_half_cuda(h, factor)
    d = gpu.upload(h)
    out = gpu.empty(h.nbytes)
    gpu.H.scale_buffer(d.data_ptr(), out.data_ptr(), h.size, factor, F16, gpu.stream)
    assert np.array_equal(gpu.download(out, np.uint16), want)
    out2 = gpu.empty(h.nbytes)
    half = h.size // 2
    gpu.H.batched_scaled_d2d_memcpy([out2.data_ptr(), out2.data_ptr() + 2 * half],
                                    [d.data_ptr(), d.data_ptr() + 2 * half],
                                    [2 * half, 2 * (h.size - half)], factor, F16, gpu.stream)
    assert np.array_equal(gpu.download(out2, np.uint16), want)


def test_reference_test_vector_for_device_half_tensors(gpu, orc, half_factor_mode):
    """test/parallel/test_torch.py:339-388 on one rank: 17, 17x17 and 17x17x17 integers in
    [-100, 100) as half, prescale np.random.seed(1234) -> uniform(); expected
    factor.type(half) * tensor.type(half), compared with threshold 0."""
    np.random.seed(1234)
    factor = np.random.uniform()
    rng = np.random.default_rng(1234)
    for dim in (1, 2, 3):
        x = rng.integers(-100, 100, 17 ** dim).astype(np.float16)
        want = np.float16(factor) * x
        d = gpu.upload(x.view(np.uint16))
        gpu.H.scale_buffer(d.data_ptr(), d.data_ptr(), x.size, factor, F16, gpu.stream)
        assert np.array_equal(gpu.download(d, np.uint16), want.view(np.uint16))


@pytest.mark.parametrize("factor", FACTORS[:3])
def test_fp16_plan_pack_and_unpack(gpu, orc, half_factor_mode, factor):
    rng = np.random.default_rng(3)
    counts = [1, 7, 2049, 0, 30001]
    xs = [(rng.standard_normal(c) * 4).astype(np.float16) for c in counts]
    d_in = [gpu.upload(x.view(np.uint16)) for x in xs]
    d_out = [gpu.empty(2 * c) for c in counts]
    plan = gpu.H.FusionPlan([t.data_ptr() for t in d_in], [t.data_ptr() for t in d_out], counts, F16)
    fb = gpu.empty(plan.buffer_len)
    try:
        plan.pack(fb.data_ptr(), factor, gpu.stream)
        plan.unpack(fb.data_ptr(), 1.0, gpu.stream)
        for x, o, c in zip(xs, d_out, counts):
            if c:
                assert np.array_equal(gpu.download(o, np.uint16)[:c], orc.scale_half_cuda(x.view(np.uint16), factor))
        plan.pack(fb.data_ptr(), 1.0, gpu.stream)
        plan.unpack(fb.data_ptr(), factor, gpu.stream)
        for x, o, c in zip(xs, d_out, counts):
            if c:
                assert np.array_equal(gpu.download(o, np.uint16)[:c], orc.scale_half_cuda(x.view(np.uint16), factor))
    finally:
        plan.destroy()


@pytest.mark.parametrize("factor", FACTORS[:3])
def test_converting_plan(gpu, orc, half_factor_mode, factor):
    """Cast-then-scale pack = compression cast, then the fp16 scale; unpack = fp16 postscale,
    then the exact widening.  The fused scale-then-cast pack keeps multiplying in fp32."""
    rng = np.random.default_rng(4)
    counts = [5, 4099, 1]
    xs = [rng.standard_normal(c).astype(np.float32) for c in counts]
    d_in = [gpu.upload(x) for x in xs]
    d_out = [gpu.empty(4 * c) for c in counts]
    plan = gpu.H.FusionPlan([t.data_ptr() for t in d_in], [t.data_ptr() for t in d_out], counts, F32, F16)
    fb = gpu.empty(plan.buffer_len)
    offs = plan.offsets()
    try:
        plan.pack(fb.data_ptr(), factor, gpu.stream, 1)  # HVDHIP_PACK_CAST_THEN_SCALE
        buf = gpu.download(fb, np.uint8)
        for x, off, c in zip(xs, offs, counts):
            got = buf[off:off + 2 * c].view(np.uint16)
            assert np.array_equal(got, orc.scale_half_cuda(x.astype(np.float16).view(np.uint16), factor))
        plan.pack(fb.data_ptr(), factor, gpu.stream, 0)
        buf = gpu.download(fb, np.uint8).copy()
        for x, off, c in zip(xs, offs, counts):
            got = buf[off:off + 2 * c].view(np.uint16)
            assert np.array_equal(got, orc.scale_cast_f32_to_f16(x, factor))
        plan.unpack(fb.data_ptr(), factor, gpu.stream)
        for x, off, o, c in zip(xs, offs, d_out, counts):
            h = buf[off:off + 2 * c].view(np.uint16)
            want = orc.scale_half_cuda(h, factor).view(np.float16).astype(np.float32)
            assert np.array_equal(gpu.download(o, np.float32)[:c].view(np.uint32), want.view(np.uint32))
    finally:
        plan.destroy()
