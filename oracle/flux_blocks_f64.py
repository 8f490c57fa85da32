"""fp64 restatement of the reference's FLUX FP8 and INT4 (W4A4 + low-rank) blocks (TEST INFRASTRUCTURE, NOT PRODUCT CODE).

Written from the reference's layer code, independently of lyradiff_amd/flux_fp8.py and lyradiff_amd/flux_int4.py, so that a wiring mistake in the
product's block functions (a wrong msa chunk, scale and shift swapped, the wrong concatenation order of text and image
tokens, a missing residual) shows up as an O(1) difference:

  double block   layers/flux_transformer_block/FluxTransformerFP8Block.cc:159-262
                 layers/ada_layer_norm/AdaFP8LayerNorm.cc:95-205       (msa = linear(temb); chunk 0 shift, chunk 1 scale)
                 layers/flux_attention_processor/FluxAttentionFP8Processor.cc:165-360
                 layers/flux_attn_post_processor/FluxAttnPostFP8Processor.cc:93-240 (chunks 2..5: gate_msa, shift_mlp,
                                                                                      scale_mlp, gate_mlp)
  single block   layers/flux_single_transformer_block/FluxSingleTransformerFP8Block.cc:163-291
                 layers/flux_single_attention_processor/FluxSingleAttentionFP8Processor.cc:155-213

  INT4 blocks    layers/w4a4_gemm_block/W4A4Gemm.cc:113-169   (quantise + low-rank down on the 16-bit input, fp32 -> T
                                                               copy of the low-rank activations, GEMM + low-rank up; no bias)
                 layers/flux_attention_processor/FluxAttentionInt4Processor.cc:206-331 (bias of QKV / output projections
                                                               added afterwards, invokeAddBias)
                 layers/flux_attn_post_processor/FluxAttnPostInt4Processor.cc:103-215  (net.0.proj W4A4, bias + GELU, net.2 FP8)
                 layers/flux_single_transformer_block/FluxSingleTransformerInt4Block.cc:196-316
                                                               (proj_mlp, proj_out.linears.0 on the attention output,
                                                               proj_out.linears.1.linear on the GELU output, summed)

Arithmetic: every FP8 linear quantises its (T-rounded) input with the calibrated static scale and its weight with the
per-tensor amax scale through the pinned codec of oracle.py and evaluates the product in fp64; LayerNorm, RMSNorm, the
rotary embedding, softmax attention, GELU, gates and residuals are fp64; tensors the reference stores in T between
kernels are rounded to T there.  A W4A4 linear quantises its input with the pinned
group quantiser of oracle.py (codes and scales), dequantises codes x scales on both sides and evaluates the product,
the low-rank branch and their sum in fp64.  Each part is pinned on its own in tests/test_oracle_pins.py (codec, GELU, LayerNorm
against torch in fp64); the composition is checked against closed forms in
tests/test_oracle_pins.py::test_flux_block_restatement_closed_forms.  `wiring` deliberately mis-wires the block so that
a test can show that it would notice."""
from __future__ import annotations

import numpy as np
import torch

from . import oracle as O


def _round(x: torch.Tensor, dtype: str) -> torch.Tensor:
    return torch.from_numpy(O.round_to(x.to(torch.float32).numpy(), dtype).astype(np.float64))


def fp8_linear(x: torch.Tensor, w16: torch.Tensor, bias: torch.Tensor, input_scale: float) -> torch.Tensor:
    """y = (s_in * s_w) * deq(e4m3(x / s_in)) . deq(e4m3(w / s_w))^T + bias, s_w = max|w| / 448; fp64 out."""
    k = x.shape[-1]
    s_in = np.float32(input_scale)
    qa = O.fp8_scale_cast(x.reshape(-1, k).to(torch.float32).numpy(), s_in, True)
    qw, s_w = O.fp8_amax_cast(w16.to(torch.float32).numpy())
    a = torch.from_numpy(O.e4m3_decode(qa).astype(np.float64))
    b = torch.from_numpy(O.e4m3_decode(qw).astype(np.float64))
    y = float(np.float32(s_in * np.float32(s_w))) * (a @ b.t()) + bias.double()
    return y.reshape(*x.shape[:-1], w16.shape[0])


def plain_linear(x: torch.Tensor, w16: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    return x.double() @ w16.double().t() + bias.double()


def layer_norm(x: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    x = x.double()
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps)


def gelu_tanh(x: torch.Tensor) -> torch.Tensor:
    x = x.double()
    return 0.5 * x * (1.0 + torch.tanh(0.7978845608028654 * (x + 0.044715 * x ** 3)))


def unpack_w4a4_weight(packed: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """packed int8 [N, K/2] (element 2j in the low nibble of byte j, two's complement) and group scales [N, K/64]
    -> dequantised weight [N, K] in fp64 (W4A4GemmWeight.h:18-24; nibble order of WeightOnlyQuantOps.cc:275-283)."""
    b = packed.contiguous().view(torch.uint8).to(torch.int16)
    lo, hi = b & 0xF, b >> 4
    lo, hi = torch.where(lo > 7, lo - 16, lo), torch.where(hi > 7, hi - 16, hi)
    q = torch.stack((lo, hi), dim=-1).reshape(packed.shape[0], -1).double()
    return q * scale.double().repeat_interleave(64, dim=1)


def w4a4_linear(sd, prefix, x: torch.Tensor, dtype: str, wiring=()) -> torch.Tensor:
    """W4A4Gemm::forward on T values x [..., K]; returns fp64 (the caller rounds to T where the reference stores T):
        codes, sA = group-64 quantiser of x / smooth                 (oracle.w4a4_quant_values, pinned)
        low       = T( x . lora_down^T )                             (the RAW input feeds the low-rank branch, fp32 -> T copy)
        y         = (codes * sA) . (wcodes * sB)^T + low . lora_up^T   -- no bias: the callers add it"""
    k = x.shape[-1]
    x2 = x.reshape(-1, k)
    smooth = sd[prefix + "smooth"].to(torch.float32).numpy()
    q, s_a = O.w4a4_quant_values(x2.to(torch.float32).numpy(), smooth, 64, "f32")
    a = torch.from_numpy(q.astype(np.float64)) * torch.from_numpy(s_a.astype(np.float64)).repeat_interleave(64, dim=1)
    w = unpack_w4a4_weight(sd[prefix + "packed_weight"], sd[prefix + "weight_scale"])
    y = a @ w.t()
    if "no_low_rank" not in wiring:
        src = x2.double() / torch.from_numpy(smooth.astype(np.float64)) if "low_rank_from_smoothed" in wiring else x2.double()
        low = _round(src @ sd[prefix + "lora_down"].double().t(), dtype)
        y = y + low @ sd[prefix + "lora_up"].double().t()
    return y.reshape(*x.shape[:-1], w.shape[0])


def _w4_bias(sd, prefix, x, dtype, wiring=()):
    """A W4A4 linear whose bias a later kernel adds in T (invokeAddBias / invokeFusedBiasAndGelu / invokeFusedBiasAndResidual)."""
    return _round(w4a4_linear(sd, prefix, x, dtype, wiring), dtype) + sd[prefix + "bias"].double()


def _lin(sd, prefix, name, x, full=True):
    w, b = sd[prefix + name + ".weight"], sd[prefix + name + ".bias"]
    if not full:
        return plain_linear(x, w, b)
    return fp8_linear(x, w, b, float(sd[prefix + name + "_input_scale"].reshape(-1)[0]))


def ada_msa(sd, prefix, temb, n_chunks, dtype, full):
    """[n_chunks, B, D]: the linear's output [B, n_chunks*D] split into chunks (invokeTranspose102)."""
    b, d = temb.shape
    flat = _round(_lin(sd, prefix, "linear", temb.double(), full), dtype)
    return flat.view(b, n_chunks, d).transpose(0, 1)


def modulate(x, scale, shift, dtype):
    """T( (1 + scale) * LayerNorm(x) + shift ) with scale/shift [B, D] broadcast over the sequence."""
    return _round((1.0 + scale.unsqueeze(1)) * layer_norm(x) + shift.unsqueeze(1), dtype)


def qk_norm_rope(t, wq, wk, rope, heads):
    """t [B, S, 3D] -> q, k, v [B, S, H, Dh]: per-head RMSNorm of q and k, then every pair (n0, n1) is multiplied by its
    2x2 rotation matrix rope[b, s, pair] (kernels/rope/flux_apply_rope.cu:74-156)."""
    b, s, d3 = t.shape
    dh = d3 // 3 // heads
    q, k, v = t.double().view(b, s, 3, heads, dh).unbind(2)
    r = rope.double().unsqueeze(2)  # [B, S, 1, Dh/2, 2, 2]

    def one(x, w):
        n = x / torch.sqrt((x ** 2).mean(-1, keepdim=True) + 1e-6) * w.double()
        p = n.reshape(b, s, heads, dh // 2, 2)
        o0 = p[..., 0] * r[..., 0, 0] + p[..., 1] * r[..., 0, 1]
        o1 = p[..., 0] * r[..., 1, 0] + p[..., 1] * r[..., 1, 1]
        return torch.stack([o0, o1], dim=-1).reshape(b, s, heads, dh)

    return one(q, wq), one(k, wk), v


def softmax_attention(q, k, v):
    w = torch.softmax(torch.einsum("bshd,bthd->bhst", q, k) / q.shape[-1] ** 0.5, dim=-1)
    return torch.einsum("bhst,bthd->bshd", w, v).reshape(q.shape[0], q.shape[1], -1)


def attn_post(sd, prefix, x, attn_out, msa, dtype, wiring=(), int4=False):
    """FluxAttnPostFP8Processor::forward: hidden = x + gate_msa * attn; ff = net.2(gelu(net.0.proj(adaLN(hidden))));
    out = hidden + gate_mlp * ff.  int4: FluxAttnPostInt4Processor::forward, the same with net.0.proj a W4A4 linear whose
    bias is added together with the GELU (net.2 stays FP8)."""
    gate_msa, shift_mlp, scale_mlp, gate_mlp = msa[2], msa[3], msa[4], msa[5]
    if "swap_mlp_scale_shift" in wiring:
        shift_mlp, scale_mlp = scale_mlp, shift_mlp
    if "swap_gates" in wiring:
        gate_msa, gate_mlp = gate_mlp, gate_msa
    hidden = _round(_round(attn_out * gate_msa.unsqueeze(1), dtype) + x.double(), dtype)
    norm = modulate(hidden, scale_mlp, shift_mlp, dtype)
    if int4:
        pre = _w4_bias(sd, prefix + "net.0.proj.", norm, dtype, wiring)
        inner = _round(pre if "no_gelu" in wiring else gelu_tanh(pre), dtype)
    else:
        inner = _round(gelu_tanh(_lin(sd, prefix, "net.0.proj", norm)), dtype)
    ff = _round(_lin(sd, prefix, "net.2", inner), dtype)
    if "no_second_residual" in wiring:
        return _round(ff * gate_mlp.unsqueeze(1), dtype)
    return _round(_round(ff * gate_mlp.unsqueeze(1), dtype) + hidden, dtype)


def flux_double_block(sd, prefix, x, ctx, temb, rope, heads, dtype="bf16", full=True, wiring=()):
    """Returns (output [B, S, D], context_output [B, Sc, D]) as fp64 tensors holding T values.  x [B, S, D] image tokens,
    ctx [B, Sc, D] text tokens, temb [B, D] (SiLU applied by the caller), rope [B, Sc + S, Dh/2, 2, 2] (text positions
    first)."""
    sc = ctx.shape[1]
    msa = ada_msa(sd, prefix + "norm1.", temb, 6, dtype, full)
    cmsa = ada_msa(sd, prefix + "norm1_context.", temb, 6, dtype, full)
    sh, scl = (msa[1], msa[0]) if "swap_scale_shift" in wiring else (msa[0], msa[1])
    norm = modulate(x, scl, sh, dtype)
    cnorm = modulate(ctx, cmsa[1], cmsa[0], dtype)
    qkv = _round(_lin(sd, prefix + "attn.", "to_qkv", norm), dtype)
    cqkv = _round(_lin(sd, prefix + "attn.", "to_added_qkv", cnorm), dtype)
    nrm = [sd[prefix + f"attn.{n}.weight"] for n in ("norm_q", "norm_k", "norm_added_q", "norm_added_k")]
    if "image_first" in wiring:  # the reference concatenates [text, image]
        a = qk_norm_rope(qkv, nrm[0], nrm[1], rope[:, : x.shape[1]], heads)
        c = qk_norm_rope(cqkv, nrm[2], nrm[3], rope[:, x.shape[1]:], heads)
        q, k, v = (torch.cat([a[i], c[i]], dim=1) for i in range(3))
        o = _round(softmax_attention(q, k, v), dtype)
        attn, cattn = o[:, : x.shape[1]], o[:, x.shape[1]:]
    else:
        c = qk_norm_rope(cqkv, nrm[2], nrm[3], rope[:, :sc], heads)
        a = qk_norm_rope(qkv, nrm[0], nrm[1], rope[:, sc:], heads)
        q, k, v = (torch.cat([c[i], a[i]], dim=1) for i in range(3))
        o = _round(softmax_attention(q, k, v), dtype)
        attn, cattn = o[:, sc:], o[:, :sc]
    a_out = _round(_lin(sd, prefix + "attn.", "to_out.0", attn), dtype)
    c_out = _round(_lin(sd, prefix + "attn.", "to_add_out", cattn), dtype)
    if "swap_out_projections" in wiring:
        a_out = _round(_lin(sd, prefix + "attn.", "to_add_out", attn), dtype)
        c_out = _round(_lin(sd, prefix + "attn.", "to_out.0", cattn), dtype)
    return (attn_post(sd, prefix + "ff.", x, a_out, msa, dtype, wiring),
            attn_post(sd, prefix + "ff_context.", ctx, c_out, cmsa, dtype, wiring))


def flux_single_block(sd, prefix, x, temb, rope, heads, dtype="bf16", full=True, wiring=()):
    """FluxSingleTransformerFP8Block::forward: norm = adaLN(x) (chunks shift, scale, gate); attn = attention(to_qkv(norm));
    mlp = gelu(T(proj_mlp(norm))); out = x + gate * proj_out([attn, mlp])."""
    msa = ada_msa(sd, prefix + "norm.", temb, 3, dtype, full)
    sh, scl = (msa[1], msa[0]) if "swap_scale_shift" in wiring else (msa[0], msa[1])
    norm = modulate(x, scl, sh, dtype)
    qkv = _round(_lin(sd, prefix + "attn.", "to_qkv", norm), dtype)
    q, k, v = qk_norm_rope(qkv, sd[prefix + "attn.norm_q.weight"], sd[prefix + "attn.norm_k.weight"], rope, heads)
    attn = _round(softmax_attention(q, k, v), dtype)
    mlp = _round(gelu_tanh(_round(_lin(sd, prefix, "proj_mlp", norm), dtype)), dtype)
    cat = torch.cat([mlp, attn], dim=-1) if "mlp_first" in wiring else torch.cat([attn, mlp], dim=-1)
    o = _round(_lin(sd, prefix, "proj_out", cat), dtype)
    gate = msa[0] if "gate_is_chunk0" in wiring else msa[2]
    return _round(_round(o * gate.unsqueeze(1), dtype) + x.double(), dtype)


def flux_double_block_int4(sd, prefix, x, ctx, temb, rope, heads, dtype="bf16", full=True, wiring=()):
    """FluxTransformerInt4Block::forward with FluxAttentionInt4Processor and FluxAttnPostInt4Processor: the double block
    with every attention projection and net.0.proj a W4A4 linear (+ low-rank branch); adaLN linear FP8 at level
    INT4_W4A4_FULL (`full`), 16-bit otherwise; net.2 FP8.  Same arguments and return as flux_double_block."""
    sc = ctx.shape[1]
    msa = ada_msa(sd, prefix + "norm1.", temb, 6, dtype, full)
    cmsa = ada_msa(sd, prefix + "norm1_context.", temb, 6, dtype, full)
    sh, scl = (msa[1], msa[0]) if "swap_scale_shift" in wiring else (msa[0], msa[1])
    norm = modulate(x, scl, sh, dtype)
    cnorm = modulate(ctx, cmsa[1], cmsa[0], dtype)
    names = ["to_qkv.", "to_added_qkv.", "to_out.0.", "to_add_out."]
    if "swap_qkv_projections" in wiring:
        names[0], names[1] = names[1], names[0]
    if "swap_out_projections" in wiring:
        names[2], names[3] = names[3], names[2]
    qkv = _round(_w4_bias(sd, prefix + "attn." + names[0], norm, dtype, wiring), dtype)
    cqkv = _round(_w4_bias(sd, prefix + "attn." + names[1], cnorm, dtype, wiring), dtype)
    nrm = [sd[prefix + f"attn.{n}.weight"] for n in ("norm_q", "norm_k", "norm_added_q", "norm_added_k")]
    c = qk_norm_rope(cqkv, nrm[2], nrm[3], rope[:, :sc], heads)
    a = qk_norm_rope(qkv, nrm[0], nrm[1], rope[:, sc:], heads)
    q, k, v = (torch.cat([c[i], a[i]], dim=1) for i in range(3))
    o = _round(softmax_attention(q, k, v), dtype)
    attn, cattn = o[:, sc:], o[:, :sc]
    a_out = _round(_w4_bias(sd, prefix + "attn." + names[2], attn, dtype, wiring), dtype)
    c_out = _round(_w4_bias(sd, prefix + "attn." + names[3], cattn, dtype, wiring), dtype)
    ff, cff = ("ff_context.", "ff.") if "swap_feed_forwards" in wiring else ("ff.", "ff_context.")
    return (attn_post(sd, prefix + ff, x, a_out, msa, dtype, wiring, int4=True),
            attn_post(sd, prefix + cff, ctx, c_out, cmsa, dtype, wiring, int4=True))


def flux_single_block_int4(sd, prefix, x, temb, rope, heads, dtype="bf16", full=True, wiring=()):
    """FluxSingleTransformerInt4Block::forward: norm = adaLN(x); attn = attention(to_qkv(norm) + b);
    mlp = gelu(proj_mlp(norm) + b); o = (proj_out.linears.0(attn) + b) + proj_out.linears.1.linear(mlp);
    out = x + gate * o, every linear W4A4 with its low-rank branch."""
    msa = ada_msa(sd, prefix + "norm.", temb, 3, dtype, full)
    sh, scl = (msa[1], msa[0]) if "swap_scale_shift" in wiring else (msa[0], msa[1])
    norm = modulate(x, scl, sh, dtype)
    qkv = _round(_w4_bias(sd, prefix + "attn.to_qkv.", norm, dtype, wiring), dtype)
    q, k, v = qk_norm_rope(qkv, sd[prefix + "attn.norm_q.weight"], sd[prefix + "attn.norm_k.weight"], rope, heads)
    attn = _round(softmax_attention(q, k, v), dtype)
    mlp_in = x if "mlp_from_block_input" in wiring else norm
    mlp = _round(gelu_tanh(_w4_bias(sd, prefix + "proj_mlp.", mlp_in, dtype, wiring)), dtype)
    h1_in = norm if "linears0_from_norm" in wiring else attn
    h1 = _round(w4a4_linear(sd, prefix + "proj_out.linears.0.", h1_in, dtype, wiring), dtype)
    h2 = _round(w4a4_linear(sd, prefix + "proj_out.linears.1.linear.", mlp, dtype, wiring), dtype)
    o = _round(h1 + sd[prefix + "proj_out.linears.0.bias"].double(), dtype)
    o = o if "drop_linears1" in wiring else _round(o + h2, dtype)
    gate = msa[0] if "gate_is_chunk0" in wiring else msa[2]
    return _round(_round(o * gate.unsqueeze(1), dtype) + x.double(), dtype)
