"""torch.ops.lyradiff.* registration: schema and shape inference on the CPU, parity with the direct
wrappers on the GPU (the operator bodies call the same C ABI entry points)."""
import numpy as np
import pytest
import torch
from torch._subclasses.fake_tensor import FakeTensorMode


@pytest.fixture(scope="module")
def tops():
    import lyradiff_amd.torch_ops as t

    return t


def test_every_operator_is_registered(tops):
    for name in tops.NAMES:
        assert hasattr(torch.ops.lyradiff, name), name
        getattr(torch.ops.lyradiff, name).default  # resolves the overload


def test_shape_inference_without_a_gpu(tops):
    with FakeTensorMode():
        dev = "cuda"
        x = torch.empty(4, 77, 640, dtype=torch.float16, device=dev)
        q, s = torch.ops.lyradiff.sq_quant_dynamic(x, None)
        assert q.shape == x.shape and q.dtype == torch.int8 and s.shape == (4 * 77,) and s.dtype == torch.float32
        w = torch.empty(1280, 640, dtype=torch.int8, device=dev)
        y = torch.ops.lyradiff.int8_linear(q.reshape(-1, 640), w, s, s, None, torch.float16)
        assert y.shape == (308, 1280) and y.dtype == torch.float16
        h = torch.empty(308, 5120, dtype=torch.float16, device=dev)
        q2, s2 = torch.ops.lyradiff.geglu_int8_dynamic(h)
        assert q2.shape == (308, 2560) and s2.shape == (308,)
        xb = torch.empty(4608, 3072, dtype=torch.bfloat16, device=dev)
        qf, sf = torch.ops.lyradiff.fp8_quant(xb)
        assert qf.dtype == torch.uint8 and qf.shape == xb.shape and sf.shape == (1,)
        wf = torch.empty(12288, 3072, dtype=torch.uint8, device=dev)
        yf = torch.ops.lyradiff.fp8_linear(qf, wf, sf, sf, None, True)
        assert yf.shape == (4608, 12288) and yf.dtype == torch.bfloat16
        qa, sa = torch.ops.lyradiff.w4a4_quant(xb, None, torch.float16)
        assert qa.shape == (4608, 384) and qa.dtype == torch.int32 and sa.shape == (4608, 48) and sa.dtype == torch.float16
        w4 = torch.empty(3072, 1536, dtype=torch.uint8, device=dev)
        y4 = torch.ops.lyradiff.w4a4_linear(qa, w4, sa, sa[:3072], None)
        assert y4.shape == (4608, 3072) and y4.dtype == torch.bfloat16
        assert torch.ops.lyradiff.repack_weight(w4).shape == w4.shape
        # FLUX FP8 block pieces
        xs = torch.empty(2, 2304, 3072, dtype=torch.bfloat16, device=dev)
        mod = torch.empty(2, 3072, dtype=torch.bfloat16, device=dev)
        one = torch.empty(1, dtype=torch.float32, device=dev)
        codes, hidden = torch.ops.lyradiff.gate_residual_layernorm_mod_fp8(xs, mod, xs, mod, mod, one)
        assert codes.shape == xs.shape and codes.dtype == torch.uint8 and hidden.shape == xs.shape and hidden.dtype == xs.dtype
        assert torch.ops.lyradiff.layernorm_mod_fp8(xs, mod, mod, one).dtype == torch.uint8
        c2 = torch.ops.lyradiff.fp8_linear_codes(qf, wf, sf, sf, None, one, 1)
        assert c2.shape == (4608, 12288) and c2.dtype == torch.uint8
        wd = torch.empty(3072, 12288, dtype=torch.uint8, device=dev)
        yg = torch.ops.lyradiff.fp8_linear_gated(c2, wd, one, one, None, mod[:1], xb, 4608)
        assert yg.shape == (4608, 3072) and yg.dtype == torch.bfloat16
        msa = torch.empty(6, 2, 3072, dtype=torch.bfloat16, device=dev)
        b1, b2 = torch.empty(12288, dtype=torch.bfloat16, device=dev), torch.empty(3072, dtype=torch.bfloat16, device=dev)
        out = torch.ops.lyradiff.flux_attn_post_fp8(xs, xs, msa, wf, one, one, b1, wd, one, one, b2)
        assert out.shape == xs.shape and out.dtype == xs.dtype
        assert torch.ops.lyradiff.lora_down(xb, torch.empty(32, 3072, dtype=torch.bfloat16, device=dev)).shape == (4608, 32)
        # the running-maximum chain and the one-pass W4A4 quantiser
        u = torch.ops.lyradiff.fp8_linear_max(qf, wf, sf, sf, None, one)
        assert u.shape == (4608, 12288) and u.dtype == torch.bfloat16
        qh, sh = torch.ops.lyradiff.fp8_gelu_quant(u, one)
        assert qh.shape == u.shape and qh.dtype == torch.uint8 and sh.shape == (1,) and sh.dtype == torch.float32
        qp, sp = torch.ops.lyradiff.fp8_quant_panels(xb)
        assert qp.shape == (48, 4608, 64) and qp.dtype == torch.uint8 and sp.shape == (1,)
        up = torch.ops.lyradiff.fp8_linear_panels(qp, wf, sp, sf, None, one)
        assert up.shape == (4608, 12288) and up.dtype == torch.bfloat16
        qhp, shp = torch.ops.lyradiff.fp8_gelu_quant_panels(up, one)
        assert qhp.shape == (192, 4608, 64) and qhp.dtype == torch.uint8 and shp.shape == (1,)
        w_, s_, a_ = torch.ops.lyradiff.w4a4_quant_lora_down(xb, None, torch.empty(32, 3072, dtype=torch.bfloat16, device=dev))
        assert w_.shape == (4608, 384) and s_.shape == (4608, 48) and a_.shape == (4608, 32) and a_.dtype == torch.bfloat16


def test_host_tensors_are_rejected(tops):
    # the reference's CHECK_TH_CUDA (src/lyradiff/th_op/th_utils.h:14-33): no silent CPU path
    with pytest.raises(ValueError, match="CUDA"):
        torch.ops.lyradiff.repack_weight(torch.zeros(32, 64, dtype=torch.int8))
    with pytest.raises(ValueError, match="CUDA"):
        torch.ops.lyradiff.fp8_quant(torch.zeros(8, 64, dtype=torch.bfloat16))


@pytest.mark.gpu
def test_operators_match_direct_wrappers(tops, dev):
    from lyradiff_amd import ops

    g = torch.Generator().manual_seed(7)
    x = torch.randn(300, 640, generator=g).half().to(dev)
    w = torch.randint(-127, 128, (320, 640), generator=g, dtype=torch.int8).to(dev)
    ws = (torch.rand(320, generator=g) * 1e-2).to(dev)
    q, s = torch.ops.lyradiff.sq_quant_dynamic(x, None)
    q0, s0 = ops.sq_quant_dynamic(x, None)
    assert torch.equal(q, q0) and torch.equal(s, s0)
    qp, sp = torch.ops.lyradiff.sq_quant_dynamic_panels(x, None)
    assert torch.equal(ops.fp8_panels_to_rows(qp), q0) and torch.equal(sp, s0)
    assert torch.equal(torch.ops.lyradiff.int8_linear_panels(qp, ops.repack_weight(w), ws, sp, None),
                       ops.int8_linear(q0, ops.repack_weight(w), ws, s0, None))
    wp = torch.ops.lyradiff.repack_weight(w)
    assert torch.equal(torch.ops.lyradiff.int8_linear(q, wp, ws, s, None, torch.float16), ops.int8_linear(q0, wp, ws, s0))
    xb = torch.randn(256, 512, generator=g).bfloat16().to(dev)
    qf, sf = torch.ops.lyradiff.fp8_quant(xb)
    qf0, sf0 = ops.fp8_quant(xb)
    assert torch.equal(qf, qf0) and torch.equal(sf, sf0)
    wf = torch.ops.lyradiff.repack_weight(qf[:128].contiguous())
    assert torch.equal(torch.ops.lyradiff.fp8_linear(qf, wf, sf, sf, None, True), ops.fp8_linear(qf, wf, sf, sf, None, True))
    qa, sa = torch.ops.lyradiff.w4a4_quant(xb, None, torch.float16)
    w4 = torch.ops.lyradiff.repack_weight(qa[:128].contiguous().view(torch.uint8).reshape(128, 256))
    assert torch.equal(torch.ops.lyradiff.w4a4_linear(qa, w4, sa, sa[:128].contiguous(), None),
                       ops.w4a4_linear(qa, w4, sa, sa[:128].contiguous(), None))
    assert np.isfinite(torch.ops.lyradiff.fp8_scale_cast(xb, sf).float().cpu().numpy()).all()
    um, um0 = torch.zeros(1, device=dev), torch.zeros(1, device=dev)
    u = torch.ops.lyradiff.fp8_linear_max(qf, wf, sf, sf, None, um)
    assert torch.equal(u, ops.fp8_linear_max(qf, wf, sf, sf, None, um0)) and torch.equal(um, um0) and um.item() > 0
    qh, sh = torch.ops.lyradiff.fp8_gelu_quant(u, um)
    qh0, sh0 = ops.fp8_gelu_quant(u, um)
    assert torch.equal(qh, qh0) and torch.equal(sh, sh0)
    qp, sp = torch.ops.lyradiff.fp8_quant_panels(xb)
    assert torch.equal(ops.fp8_panels_to_rows(qp), qf) and torch.equal(sp, sf)
    um2 = torch.zeros(1, device=dev)
    assert torch.equal(torch.ops.lyradiff.fp8_linear_panels(qp, wf, sp, sf, None, um2), u) and torch.equal(um2, um)
    qhp, shp = torch.ops.lyradiff.fp8_gelu_quant_panels(u, um)
    assert torch.equal(ops.fp8_panels_to_rows(qhp), qh) and torch.equal(shp, sh)
    dn = (torch.randn(32, 512, generator=g) * 0.05).bfloat16().to(dev)
    sm = (torch.rand(512, generator=g) + 0.5).to(dev)
    got3, ref3 = torch.ops.lyradiff.w4a4_quant_lora_down(xb, sm, dn), ops.w4a4_quant_lora_down(xb, sm, dn)
    assert all(torch.equal(a, b) for a, b in zip(got3, ref3))


@pytest.mark.gpu
def test_block_operators_match_the_python_functions(tops, dev):
    from lyradiff_amd import flux_fp8 as F

    g = torch.Generator().manual_seed(9)
    b, s, d = 1, 160, 256
    bf = lambda *shape, sc=1.0: (sc * torch.randn(*shape, generator=g)).bfloat16()
    sd = {"p.net.0.proj.weight": bf(4 * d, d, sc=0.03), "p.net.0.proj.bias": bf(4 * d, sc=0.1),
          "p.net.2.weight": bf(d, 4 * d, sc=0.03), "p.net.2.bias": bf(d, sc=0.1),
          "p.net.0.proj_input_scale": torch.tensor([5.0 / 448]), "p.net.2_input_scale": torch.tensor([2.0 / 448]),
          "p.proj_mlp.weight": bf(4 * d, d, sc=0.03), "p.proj_mlp.bias": bf(4 * d, sc=0.1),
          "p.proj_out.weight": bf(d, 5 * d, sc=0.03), "p.proj_out.bias": bf(d, sc=0.1),
          "p.proj_mlp_input_scale": torch.tensor([5.0 / 448]), "p.proj_out_input_scale": torch.tensor([4.0 / 448])}
    wp, ws = F.load_flux_attn_post_fp8(sd, "p.", d, torch.bfloat16, dev), F.load_flux_single_mlp_fp8(sd, "p.", d, 4, torch.bfloat16, dev)
    x, attn, norm = bf(b, s, d).to(dev), bf(b, s, d).to(dev), bf(b, s, d).to(dev)
    msa = bf(6, b, d, sc=0.5).to(dev)
    flat = lambda l: (l.weight_rows32, l.weight_scale, l.input_scale, l.bias)
    got = torch.ops.lyradiff.flux_attn_post_fp8(x, attn, msa, *flat(wp.gelu_proj), *flat(wp.ff_linear))
    assert torch.equal(got, F.flux_attn_post_fp8(x, attn, msa, wp))
    gate = msa[2].contiguous()
    got = torch.ops.lyradiff.flux_single_mlp_fp8(x, norm, attn, gate, *flat(ws.proj_mlp), *flat(ws.proj_out))
    assert torch.equal(got, F.flux_single_mlp_fp8(x, norm, attn, gate, ws))


def test_lyrallms_utility_operators_on_the_cpu(tops):
    """torch.ops.lyrallms.* as the reference registers them (WeightOnlyQuantOps.cc:326-351): CPU tensors in and out."""
    for name in tops._LLM:
        assert hasattr(torch.ops.lyrallms, name), name
    q = torch.randint(-8, 8, (2, 5, 8), generator=torch.Generator().manual_seed(3), dtype=torch.int8)
    packed = torch.ops.lyrallms.pack_int8_tensor_to_packed_int4(q)
    assert packed.shape == (2, 5, 4) and packed.dtype == torch.int8
    assert torch.equal(torch.ops.lyrallms.unpack_int4_packed_tensor_to_int8(packed), q)
    assert packed[0, 0, 0].item() == ((int(q[0, 0, 0]) & 0xF) | ((int(q[0, 0, 1]) & 0xF) << 4)) - (256 if (int(q[0, 0, 1]) & 0x8) else 0)
    with pytest.raises(RuntimeError, match="int4 or int8"):
        torch.ops.lyrallms.preprocess_weights_for_mixed_gemm(torch.zeros(64, 32, dtype=torch.int8), torch.float16)
    with pytest.raises(RuntimeError, match="BF16/FP16"):
        torch.ops.lyrallms.symmetric_quantize_last_axis_of_batched_matrix(torch.zeros(64, 32), torch.int8)


@pytest.mark.gpu
@pytest.mark.parametrize("quant_type,kind", [(torch.int8, "int8"), (torch.quint4x2, "int4")])
def test_lyrallms_quantise_preprocess_and_gemm(tops, dev, quant_type, kind):
    """symmetric_quantize_last_axis_of_batched_matrix -> (processed weight, scales) feeds the weight-only GEMM directly;
    the underscore form also returns the unprocessed codes, and preprocessing those gives the same processed weight."""
    from lyradiff_amd import ops
    from oracle import oracle as O

    g = torch.Generator().manual_seed(11)
    k, n, m = 256, 96, 40
    w = (0.05 * torch.randn(k, n, generator=g)).half()
    x = torch.randn(m, k, generator=g).half()
    processed, scales = torch.ops.lyrallms.symmetric_quantize_last_axis_of_batched_matrix(w, quant_type)
    unprocessed, processed2, scales2 = torch.ops.lyrallms._symmetric_quantize_last_axis_of_batched_matrix(w, quant_type)
    assert not processed.is_cuda and torch.equal(processed, processed2) and torch.equal(scales, scales2)
    assert torch.equal(torch.ops.lyrallms.preprocess_weights_for_mixed_gemm(unprocessed, quant_type), processed)
    bits = 8 if kind == "int8" else 4
    q_ref, s_ref = O.weight_only_quantize(w.float().numpy(), bits, "f16")
    assert np.array_equal(scales.float().numpy(), s_ref)
    y = ops.weight_only_linear(x.to(dev), processed.view(torch.uint8).to(dev), scales.to(dev), None, kind)
    ref = O.weight_only_gemm_f64(x.float().numpy(), q_ref, s_ref, None, "f16")
    assert np.allclose(y.float().cpu().numpy(), ref, rtol=1e-2, atol=2e-3)
    # a batch of matrices ("experts") is processed one by one
    w3 = torch.stack([w, -w])
    p3, s3 = torch.ops.lyrallms.symmetric_quantize_last_axis_of_batched_matrix(w3, quant_type)
    assert p3.shape[0] == 2 and torch.equal(p3[0], processed) and torch.equal(s3[0], scales)
