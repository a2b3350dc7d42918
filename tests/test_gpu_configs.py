"""The five benchmark configurations at their full sizes, through the same
op sequence as the reference's allreduce (pipeline.AllreducePipeline), checked
against the CPU oracle on identical seeded inputs.  The 3.1 GB GPT-2 XL case
is checked by the oracle over every tensor and, over every byte, against
an independent elementwise evaluation on the device."""
import numpy as np
import pytest
import torch

from oracle_util import F16, F32

pytestmark = pytest.mark.gpu


def _carve(counts, es):
    offs, cur = [], 0
    for c in counts:
        offs.append(cur)
        cur += (c * es + 255) // 256 * 256
    return offs, max(cur, 256)


def _host_set(counts, es, gen):
    """Host image (uint8) of tensors at 256-byte aligned offsets; gen(n) makes one tensor."""
    offs, total = _carve(counts, es)
    img = np.zeros(total, np.uint8)
    vals = []
    for o, c in zip(offs, counts):
        v = gen(c)
        img[o:o + c * es] = v.view(np.uint8)
        vals.append(v)
    return offs, img, vals


def _peer_images(pipe, counts, es_buf, gen):
    """One peer buffer image per fusion cycle, laid out like that cycle's fusion buffer
    (or like the single tensor); returns (device tensors, per-tensor peer values)."""
    per_tensor = {}
    images = []
    for cyc in pipe.cycles:
        if cyc.plan is not None:
            offs = cyc.plan.offsets()
            img = np.zeros(cyc.plan.buffer_len, np.uint8)
            for i, o in zip(cyc.indices, offs):
                v = gen(counts[i])
                img[o:o + v.nbytes] = v.view(np.uint8)
                per_tensor[i] = v
        else:
            i = cyc.indices[0]
            v = gen(counts[i])
            img = v.view(np.uint8).copy()
            per_tensor[i] = v
        images.append(torch.from_numpy(img).cuda())
    torch.cuda.synchronize()
    return images, per_tensor


def test_c1_resnet50_fp32_pack_prescale_sum_unpack(gpu, orc):
    from horovod_amd import workloads as W
    from horovod_amd.pipeline import AllreducePipeline
    counts = [W.numel(s) for s in W.resnet50_shapes()]
    rng, prng = np.random.default_rng(1), np.random.default_rng(2)
    offs, img, vals = _host_set(counts, 4, lambda n: (rng.standard_normal(n) * 1e-3).astype(np.float32))
    d_in = torch.from_numpy(img).cuda()
    d_out = torch.zeros_like(d_in)
    pipe = AllreducePipeline([d_in.data_ptr() + o for o in offs], [d_out.data_ptr() + o for o in offs], counts, F32,
                             completion_events=True)
    assert len(pipe.cycles) == 2  # 102.2 MB through a 64 MiB threshold
    peers, peer_vals = _peer_images(pipe, counts, 4, lambda n: (prng.standard_normal(n) * 1e-3).astype(np.float32))
    pipe.run(0.125, 1.0, lambda ci, p: peers[ci].data_ptr(), 1)
    pipe.synchronize()
    out = d_out.cpu().numpy()
    for i, (o, c, v) in enumerate(zip(offs, counts, vals)):
        want = orc.sum(peer_vals[i], orc.scale_buffer(v, 0.125, F32), F32)
        assert np.array_equal(out[o:o + 4 * c].view(np.uint32), want.view(np.uint32)), "tensor %d" % i
    pipe.destroy()


def test_c1_through_the_array_taking_entry_points(gpu, orc):
    """The same configuration with every pack and unpack through hvdhip_batched_scaled_d2d_memcpy (the launcher
    that takes the copies as arrays, ops/gpu_operations.cc:186-206) on two stream slots: the pack's destinations
    lie back to back, which the library recognises and stores like a pack; results equal the oracle's."""
    from horovod_amd import workloads as W
    from horovod_amd.pipeline import AllreducePipeline
    counts = [W.numel(s) for s in W.resnet50_shapes()]
    rng, prng = np.random.default_rng(1), np.random.default_rng(2)
    offs, img, vals = _host_set(counts, 4, lambda n: (rng.standard_normal(n) * 1e-3).astype(np.float32))
    d_in = torch.from_numpy(img).cuda()
    d_out = torch.zeros_like(d_in)
    pipe = AllreducePipeline([d_in.data_ptr() + o for o in offs], [d_out.data_ptr() + o for o in offs], counts, F32,
                             num_streams=2, array_entry_points=True)
    peers, peer_vals = _peer_images(pipe, counts, 4, lambda n: (prng.standard_normal(n) * 1e-3).astype(np.float32))
    for rep in range(2):  # the second pass finds its copy tables in the cache
        pipe.run(0.125, 0.5, lambda ci, p: peers[ci].data_ptr(), 1)
        pipe.synchronize()
    out = d_out.cpu().numpy()
    for i, (o, c, v) in enumerate(zip(offs, counts, vals)):
        want = orc.scale_buffer(orc.sum(peer_vals[i], orc.scale_buffer(v, 0.125, F32), F32), 0.5, F32)
        assert np.array_equal(out[o:o + 4 * c].view(np.uint32), want.view(np.uint32)), "tensor %d" % i
    pipe.destroy()


def test_c2_fusion_stress_pack_unpack(gpu, orc):
    from horovod_amd import workloads as W
    from horovod_amd.pipeline import AllreducePipeline
    counts = W.stress_counts(seed=3)
    rng = np.random.default_rng(4)
    offs, img, vals = _host_set(counts, 4, lambda n: rng.uniform(-1, 1, n).astype(np.float32))
    d_in = torch.from_numpy(img).cuda()
    d_out = torch.zeros_like(d_in)
    pipe = AllreducePipeline([d_in.data_ptr() + o for o in offs], [d_out.data_ptr() + o for o in offs], counts, F32)
    assert len(pipe.cycles) == 1 and pipe.cycles[0].plan.n == 1024
    for _ in range(3):
        pipe.run(0.125, 1.0)
    pipe.synchronize()
    out = d_out.cpu().numpy()
    for o, c, v in zip(offs, counts, vals):
        assert np.array_equal(out[o:o + 4 * c].view(np.uint32), orc.scale_buffer(v, 0.125, F32).view(np.uint32))
    # the batched-copy comparator of the configuration: the same bytes moved by per-tensor copies
    import horovod_amd
    L = horovod_amd.lib()
    d_cmp = torch.zeros_like(d_in)
    for o, c in zip(offs, counts):
        horovod_amd.check(L.hvdhip_memcpy_async(d_cmp.data_ptr() + o, d_in.data_ptr() + o, 4 * c, 3,
                                                gpu.stream.handle), "memcpy")
    d_one = torch.zeros_like(d_in)
    gpu.H.batched_d2d_memcpy([d_one.data_ptr() + o for o in offs], [d_in.data_ptr() + o for o in offs],
                             [4 * c for c in counts], gpu.stream)
    gpu.sync()
    assert torch.equal(d_cmp, d_one)
    pipe.destroy()


def test_c3_bert_large_fp16_compression_seven_peers(gpu, orc):
    """fp32 N(0,1e-4) -> prescale 1/8 in fp32 -> fp16 (mostly subnormal halves) -> the resident 1/8 chunk of
    every cycle accumulates 7 peer chunks in order, rounding to half after each -> postscale -> fp32 -> unpack."""
    from horovod_amd import workloads as W
    from horovod_amd.pipeline import AllreducePipeline
    counts = [W.numel(s) for s in W.bert_large_shapes()]
    rng = np.random.default_rng(5)
    offs, img, vals = _host_set(counts, 4, lambda n: (rng.standard_normal(n, dtype=np.float32) * np.float32(1e-4)))
    d_in = torch.from_numpy(img).cuda()
    d_out = torch.zeros_like(d_in)
    del img
    pipe = AllreducePipeline([d_in.data_ptr() + o for o in offs], [d_out.data_ptr() + o for o in offs], counts,
                             F32, F16)
    assert len(pipe.cycles) == 11
    # 7 peers, each a 1/8-size chunk per cycle (seeds 6..12)
    peer_host, peer_dev = [], []
    for p in range(7):
        prng = np.random.default_rng(6 + p)
        chunks = []
        for cyc in pipe.cycles:
            n = pipe.reduce_elems(cyc, 0.125)
            chunks.append((prng.standard_normal(n, dtype=np.float32) * np.float32(1e-4) * np.float32(0.125)).astype(np.float16))
        peer_host.append(chunks)
        peer_dev.append([torch.from_numpy(c.view(np.uint8)).cuda() for c in chunks])
    torch.cuda.synchronize()
    for postscale in (1.0, 4.0):
        pipe.run(0.125, postscale, lambda ci, p: peer_dev[p][ci].data_ptr(), 7, 0.125, True)
        pipe.synchronize()
        out = d_out.cpu().numpy()
        bad = 0
        for ci, cyc in enumerate(pipe.cycles):
            # oracle image of this cycle's fusion buffer
            cof = cyc.plan.offsets()
            buf = np.zeros(cyc.plan.buffer_len // 2, np.uint16)
            for i, o in zip(cyc.indices, cof):
                buf[o // 2:o // 2 + counts[i]] = orc.scale_cast_f32_to_f16(vals[i], 0.125)
            n = pipe.reduce_elems(cyc, 0.125)
            res = buf[:n].copy()
            for p in range(7):
                res = orc.float16_sum(peer_host[p][ci].view(np.uint16), res)
            buf[:n] = res
            for i, o in zip(cyc.indices, cof):
                want = orc.scale_cast_f16_to_f32(buf[o // 2:o // 2 + counts[i]], postscale)
                got = out[offs[i]:offs[i] + 4 * counts[i]].view(np.uint32)
                bad += int((got != want.view(np.uint32)).sum())
        assert bad == 0, "postscale %r: %d elements differ" % (postscale, bad)
    # most packed values are subnormal halves, as the configuration intends
    sample = orc.scale_cast_f32_to_f16(vals[5], 0.125)
    assert np.mean((sample & 0x7c00) == 0) > 0.9
    pipe.destroy()


def test_c3_cast_then_scale_variant_is_the_other_rounding(gpu, orc):
    rng = np.random.default_rng(5)
    v = (rng.standard_normal(1 << 20) * 1e-4).astype(np.float32)
    d_in, d_out = gpu.upload(v), gpu.empty(v.nbytes)
    plan = gpu.H.FusionPlan([d_in.data_ptr()], [d_out.data_ptr()], [v.size], F32, F16)
    fb = gpu.empty(plan.buffer_len)
    plan.pack(fb.data_ptr(), 0.125, gpu.stream, flags=1)
    got = gpu.download(fb, np.uint16)[:v.size]
    assert np.array_equal(got, orc.scale_cast_f32_to_f16(v, 0.125, cast_first=True))
    assert not np.array_equal(got, orc.scale_cast_f32_to_f16(v, 0.125))
    plan.destroy()


def test_c4_adasum_32m_64_layers(gpu, orc):
    from horovod_amd import workloads as W
    n = 1 << 25
    counts = W.adasum_layer_counts(n, 64, seed=13)
    a = np.random.default_rng(14).standard_normal(n, dtype=np.float32)
    z = np.random.default_rng(15).standard_normal(n, dtype=np.float32)
    b = (np.float32(0.3) * a + np.float32(np.sqrt(1 - 0.09)) * z).astype(np.float32)
    del z
    d_a, d_b = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
    torch.cuda.synchronize()
    plan = gpu.H.AdasumPlan(counts, F32)
    plan.combine(d_a.data_ptr(), d_b.data_ptr(), gpu.stream)
    nd, co = plan.read(gpu.stream)
    want, nd_w, co_w = orc.adasum_pairwise(a, b, counts, F32)
    nd, co = np.array(nd), np.array(co)
    # per-layer cosine is about 0.3 by construction
    cos = nd_w[0::3] / np.sqrt(nd_w[1::3] * nd_w[2::3])
    assert np.all(np.abs(cos - 0.3) < 0.05)
    assert np.all(np.abs(co - co_w) <= 1e-6 * np.abs(co_w)), "coefficient gate of 1e-6 relative"
    assert np.max(np.abs(co - co_w) / np.abs(co_w)) < 1e-11
    assert np.all(np.abs(nd - nd_w) <= 1e-11 * np.abs(nd_w))
    got = d_a.cpu().numpy()
    ulp = np.spacing(np.abs(want))
    assert np.all(np.abs(got - want) <= ulp)
    assert np.mean(got.view(np.uint32) == want.view(np.uint32)) > 0.999
    plan.destroy()


def test_c5_gpt2_xl_fp16_two_streams(gpu, orc):
    """1.56 B fp16 elements streamed through 64 MiB cycles on two streams with two fusion buffers."""
    from horovod_amd import workloads as W
    from horovod_amd.pipeline import AllreducePipeline
    counts = [W.numel(s) for s in W.gpt2_xl_shapes()]
    offs, total = _carve(counts, 2)
    g = torch.Generator(device="cuda")
    g.manual_seed(16)
    d_in = torch.empty(total // 2, dtype=torch.float16, device="cuda")
    step = 1 << 28
    for s in range(0, d_in.numel(), step):  # bounded temporaries
        e = min(d_in.numel(), s + step)
        d_in[s:e] = (torch.randn(e - s, generator=g, device="cuda") * 1e-3).half()
    d_out = torch.zeros_like(d_in)
    base_in, base_out = d_in.data_ptr(), d_out.data_ptr()
    pipe = AllreducePipeline([base_in + o for o in offs], [base_out + o for o in offs], counts, F16,
                             num_streams=2)
    singles = [c for c in pipe.cycles if c.plan is None]
    assert len(singles) == 1 and counts[singles[0].indices[0]] == 50257 * 1600  # the embedding is not fused
    assert 45 <= len(pipe.cycles) <= 50
    # one peer buffer per stream slot would be overwritten mid-flight; give every cycle its own peer
    g.manual_seed(17)
    peers = []
    for cyc in pipe.cycles:
        peers.append((torch.randn(cyc.buffer_elems, generator=g, device="cuda") * 1e-3).half())
    torch.cuda.synchronize()
    pipe.run(0.125, 1.0, lambda ci, p: peers[ci].data_ptr(), 1)
    pipe.synchronize()
    torch.cuda.synchronize()
    # (1) every element against an independent evaluation on the device:
    #     RNE16(fp32(RNE16(0.125f * fp32(x))) + fp32(peer))
    total_bad = 0
    for ci, cyc in enumerate(pipe.cycles):
        if cyc.plan is not None:
            cof = cyc.plan.offsets()
            for i, o in zip(cyc.indices, cof):
                x = d_in[offs[i] // 2:offs[i] // 2 + counts[i]]
                p = peers[ci][o // 2:o // 2 + counts[i]]
                want = ((x.float() * 0.125).half().float() + p.float()).half()
                got = d_out[offs[i] // 2:offs[i] // 2 + counts[i]]
                total_bad += int((want.view(torch.int16) != got.view(torch.int16)).sum())
        else:
            i = cyc.indices[0]
            x = d_in[offs[i] // 2:offs[i] // 2 + counts[i]]
            want = ((x.float() * 0.125).half().float() + peers[ci][:counts[i]].float()).half()
            got = d_out[offs[i] // 2:offs[i] // 2 + counts[i]]
            total_bad += int((want.view(torch.int16) != got.view(torch.int16)).sum())
    assert total_bad == 0
    # (2) the oracle over every tensor of every cycle, whole (the unfused embedding included)
    for ci, cyc in enumerate(pipe.cycles):
        cof = cyc.plan.offsets() if cyc.plan is not None else [0]
        for i, o in zip(cyc.indices, cof):
            n = counts[i]
            x = d_in[offs[i] // 2:offs[i] // 2 + n].cpu().numpy().view(np.uint16)
            p = peers[ci][o // 2:o // 2 + n].cpu().numpy().view(np.uint16)
            want = orc.sum(p, orc.scale_buffer(x, 0.125, F16), F16)
            got = d_out[offs[i] // 2:offs[i] // 2 + n].cpu().numpy().view(np.uint16)
            assert np.array_equal(got, want), "cycle %d tensor %d" % (ci, i)
    # (3) identity round trip over all 3.1 GB: scale 1, no peers -> outputs equal inputs bit for bit
    d_out.zero_()
    torch.cuda.synchronize()
    pipe.run(1.0, 1.0)
    pipe.synchronize()
    for o, c in zip(offs, counts):
        assert torch.equal(d_in[o // 2:o // 2 + c].view(torch.int16), d_out[o // 2:o // 2 + c].view(torch.int16))
    pipe.destroy()
