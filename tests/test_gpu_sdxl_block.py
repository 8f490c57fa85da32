"""The SDXL transformer block with SmoothQuant INT8 linears (lyradiff_amd/sdxl_int8.py) on the GPU.

Two checks per quant level: the block equals its own steps called one by one (each step is compared with the CPU oracle in
tests/test_gpu_quant.py, test_gpu_gemm.py and test_gpu_layernorm.py), and its output stays within the INT8 quantisation noise of
an fp32 PyTorch evaluation of the same block with the unquantised weights -- a wrong residual, bias, scale or weight key moves
the output by far more than that."""
import pytest
import torch

from tests.helpers import rng_t

pytestmark = pytest.mark.gpu


def _float_block(x, enc, W, heads, eps=1e-5):
    """fp32 reference; returns (output, {linear name: its input}) for calibrating the static activation scales."""
    F = torch.nn.functional
    seen = {}
    b, s, d = x.shape

    def att(q, k, v):
        sp = lambda t: t.view(b, t.shape[1], heads, d // heads).transpose(1, 2)
        return F.scaled_dot_product_attention(sp(q), sp(k), sp(v)).transpose(1, 2).reshape(b, s, d)

    n1 = F.layer_norm(x, (d,), W["norm1.weight"], W["norm1.bias"], eps)
    seen["attn1.to_qkv"] = n1
    q, k, v = F.linear(n1, W["attn1.to_qkv.weight"]).split(d, dim=-1)
    a1 = att(q, k, v)
    seen["attn1.to_out.0"] = a1
    h1 = F.linear(a1, W["attn1.to_out.0.weight"], W["attn1.to_out.0.bias"]) + x
    n2 = F.layer_norm(h1, (d,), W["norm2.weight"], W["norm2.bias"], eps)
    seen["attn2.to_q"] = n2
    a2 = att(F.linear(n2, W["attn2.to_q.weight"]), F.linear(enc, W["attn2.to_k.weight"]), F.linear(enc, W["attn2.to_v.weight"]))
    seen["attn2.to_out.0"] = a2
    h2 = F.linear(a2, W["attn2.to_out.0.weight"], W["attn2.to_out.0.bias"]) + h1
    n3 = F.layer_norm(h2, (d,), W["norm3.weight"], W["norm3.bias"], eps)
    seen["ff.net.0.proj"] = n3
    up = F.linear(n3, W["ff.net.0.proj.weight"], W["ff.net.0.proj.bias"])
    hh, gg = up.split(4 * d, dim=-1)
    inner = hh * F.gelu(gg, approximate="tanh")
    seen["ff.net.2"] = inner
    return F.linear(inner, W["ff.net.2.weight"], W["ff.net.2.bias"]) + h2, seen


def _int8_entries(name, w, act, g):
    """SmoothQuant export of one linear: smoothing vector, per-channel weight scales, calibrated per-tensor activation scale."""
    k = w.shape[1]
    amax_x = act.reshape(-1, k).abs().amax(dim=0).clamp_min(1e-3)
    smooth = (amax_x.sqrt() / w.abs().amax(dim=0).clamp_min(1e-3).sqrt())
    pre = 1.0 / smooth
    ws = w * smooth[None, :]
    wscale = ws.abs().amax(dim=1) / 127.0
    wq = torch.clamp(torch.round(ws / wscale[:, None]), -127, 127).to(torch.int8)
    in_scale = ((act.reshape(-1, k) * pre[None, :]).abs().max() / 127.0).reshape(1)
    return {name + ".weight_int8": wq, name + ".weight_quant_scale": wscale.float(), name + ".input_quant_scale": in_scale.float(),
            name + ".pre_quant_scale": pre.float()}


@pytest.mark.parametrize("level", [1, 2, 3])
@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
def test_basic_transformer_int8_block(dev, level, dt):
    from lyradiff_amd import ops
    from lyradiff_amd import sdxl_int8 as S

    b, s, sc, d, dc, heads = 2, 160, 77, 320, 256, 5
    g = rng_t(500 + level)
    r = lambda *shape, scale=1.0: scale * torch.randn(*shape, generator=g)
    W = {"attn1.to_qkv.weight": r(3 * d, d, scale=d ** -0.5), "attn1.to_out.0.weight": r(d, d, scale=d ** -0.5),
         "attn1.to_out.0.bias": r(d, scale=0.05), "attn2.to_q.weight": r(d, d, scale=d ** -0.5),
         "attn2.to_k.weight": r(d, dc, scale=dc ** -0.5), "attn2.to_v.weight": r(d, dc, scale=dc ** -0.5),
         "attn2.to_out.0.weight": r(d, d, scale=d ** -0.5), "attn2.to_out.0.bias": r(d, scale=0.05),
         "ff.net.0.proj.weight": r(8 * d, d, scale=d ** -0.5), "ff.net.0.proj.bias": r(8 * d, scale=0.05),
         "ff.net.2.weight": r(d, 4 * d, scale=(4 * d) ** -0.5), "ff.net.2.bias": r(d, scale=0.05)}
    for n in ("norm1", "norm2", "norm3"):
        W[n + ".weight"] = 1 + 0.1 * r(d)
        W[n + ".bias"] = 0.05 * r(d)
    x, enc = r(b, s, d), r(b, sc, dc)
    x[..., 7] *= 6.0  # an outlier channel, the case SmoothQuant's smoothing vector exists for
    want, seen = _float_block(x, enc, W, heads)

    sd = {"p." + k: v.to(dt) for k, v in W.items() if not k.startswith("attn1.to_qkv")}
    for i, c in enumerate("qkv"):
        sd[f"p.attn1.to_{c}.weight"] = W["attn1.to_qkv.weight"][i * d:(i + 1) * d].to(dt)
    for name in ("attn1.to_qkv", "attn1.to_out.0", "attn2.to_q", "attn2.to_out.0", "ff.net.0.proj", "ff.net.2"):
        sd.update(_int8_entries("p." + name, W[name + ".weight"], seen[name], g))
    w = S.load_basic_transformer_int8(sd, "p.", d, dc, level, dt, dev)
    assert isinstance(w.attn1_qkv, S.Int8Linear) == (level >= 2) and isinstance(w.attn2_q, S.Int8Linear) == (level == 3)
    xd, ed = x.to(dt).to(dev), enc.to(dt).to(dev)
    out = S.basic_transformer_int8_block(xd, ed, w, heads)
    assert out.shape == x.shape and out.dtype == dt and torch.isfinite(out.float()).all()
    err = (out.float().cpu() - want).norm() / want.norm()
    assert err < 0.04, f"level {level}: relative error {err:.4f} against the fp32 block"

    if level == 3:  # the same steps, one kernel at a time
        F = torch.nn.functional
        q8, _, _ = ops.layernorm_int8(xd, *w.norm1, w.attn1_qkv.pre_quant_scale, w.attn1_qkv.input_quant_scale, eps=1e-5)
        qkv = S._gemm_int8(q8, w.attn1_qkv, dt)
        a1 = S._attention(*qkv.split(d, dim=-1), heads).contiguous()
        y1 = w.attn1_to_out.forward(a1)                                    # sq_quant + GEMM (no bias in the container)
        h1 = (y1 + xd) + w.attn1_to_out_bias                               # T arithmetic of the fused kernel: residual, then bias
        q8b, _, h1k = ops.layernorm_int8(y1, *w.norm2, w.attn2_q.pre_quant_scale, w.attn2_q.input_quant_scale, xd, w.attn1_to_out_bias, 1e-5)
        assert torch.equal(h1k, h1)
        q8c, _, _ = ops.layernorm_int8(h1, *w.norm2, w.attn2_q.pre_quant_scale, w.attn2_q.input_quant_scale, eps=1e-5)
        assert torch.equal(q8b, q8c)
        a2 = S._attention(S._gemm_int8(q8b, w.attn2_q, dt), w.attn2_k.forward(ed), w.attn2_v.forward(ed), heads).contiguous()
        y2 = w.attn2_to_out.forward(a2)
        q8d, _, h2 = ops.layernorm_int8(y2, *w.norm3, w.geglu.pre_quant_scale, w.geglu.input_quant_scale, h1, w.attn2_to_out_bias, 1e-5)
        up = S._gemm_int8(q8d, w.geglu, dt)
        q8e = ops.geglu_int8(up, w.geglu_bias, w.ffn.pre_quant_scale, w.ffn.input_quant_scale)
        steps = S._gemm_int8(q8e, w.ffn, dt, w.ffn.bias) + h2
        assert torch.equal(out, steps)

    with pytest.raises(ValueError):
        S.load_basic_transformer_int8(sd, "p.", d, dc, 4, dt, dev)
    with pytest.raises(KeyError):
        S.load_basic_transformer_int8(sd, "q.", d, dc, level, dt, dev)
