"""The SDXL transformer block with SmoothQuant INT8 linears, built from the quantized-linear kernels.

  BasicTransformerInt8Block<T>::forward (layers/basic_transformer/BasicTransformerInt8Block.cc:261-845), levels
  INT8_SMOOTH_QUANT_LEVEL1/2/3.  INT8 at every level: the GEGLU feed-forward (`ff.net.0.proj`, `ff.net.2`).  From level 2 on:
  the fused QKV projection of the self-attention (`attn1.to_qkv`).  At level 3 also `attn1.to_out.0`, `attn2.to_q`,
  `attn2.to_out.0`, with the residual + bias + LayerNorm + quantisation between them in one kernel:

      q8        = LayerNorm(x; norm1) -> int8                      invokeLayerNormInt8O                 (level >= 2)
      qkv       = q8 . Wqkv^T                                      runGemmInt8
      a1        = attention(qkv)                                   (caller-side core: no quantized linear inside)
      y1        = int8(a1) . Wo1^T                                 invokeSqInputQuant + runGemmInt8     (level 3)
      q8, h1    = LayerNorm(y1 + x + bo1; norm2) -> int8           invokeFusedResidualBiasLayerNormInt8O
      q         = q8 . Wq2^T                                       runGemmInt8
      a2        = attention(q, K/V of the text states)             (K/V projections are 16-bit at every level)
      y2        = int8(a2) . Wo2^T
      q8, h2    = LayerNorm(y2 + h1 + bo2; norm3) -> int8
      up        = q8 . Wgeglu^T                                    runGemmInt8
      q8        = int8( (up_h + b_h) * gelu(up_g + b_g) )          invokeFusedAddBiasGegluInt8O
      out       = (q8 . Wff^T + bff) + h2                          runGemmInt8, invokeFusedBiasResidualAdd

  The 16-bit linears of the lower levels and the text K/V projections are not quantized linears and run as plain PyTorch
  matmuls; softmax attention is PyTorch's as well.  Weight keys follow BasicTransformerInt8BlockWeight::loadWeights
  (BasicTransformerInt8BlockWeight.cc:232-288): `<name>.weight_int8`, `.weight_quant_scale`, `.input_quant_scale`,
  `.pre_quant_scale` for an INT8 linear (MACROLoadLinearInt8WeightFromBin, utils/common_macro_def.h:51-59), `.weight` /
  `.bias` for 16-bit tensors, `norm{1,2,3}.weight` / `.bias`.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Union

import torch

from . import ops
from .weights import Int8Linear, _source, load_int8_linear


@dataclass
class Linear16:
    weight: torch.Tensor               # T [N, K]
    bias: Optional[torch.Tensor] = None

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return torch.nn.functional.linear(x, self.weight, self.bias)


@dataclass
class BasicTransformerInt8Weights:
    level: int                           # 1, 2 or 3
    norm1: tuple                         # (gamma, beta)
    norm2: tuple
    norm3: tuple
    attn1_qkv: Union[Int8Linear, Linear16]      # [3D, D], no bias
    attn1_to_out: Union[Int8Linear, Linear16]   # [D, D]; the bias is kept apart (added with the residual)
    attn1_to_out_bias: torch.Tensor
    attn2_q: Union[Int8Linear, Linear16]        # [D, D], no bias
    attn2_k: Linear16                           # [D, Dc]
    attn2_v: Linear16
    attn2_to_out: Union[Int8Linear, Linear16]
    attn2_to_out_bias: torch.Tensor
    geglu: Int8Linear                           # [8D, D]; bias applied by the GEGLU kernel
    geglu_bias: torch.Tensor
    ffn: Int8Linear                             # [D, 4D], bias fused into the GEMM epilogue


def load_basic_transformer_int8(src, prefix: str, dim: int, cross_dim: int, level: int, dtype=torch.float16,
                                device="cuda") -> BasicTransformerInt8Weights:
    if level not in (1, 2, 3):
        raise ValueError("level must be 1, 2 or 3 (INT8_SMOOTH_QUANT_LEVEL1..3)")
    get = _source(src)
    t16 = lambda name, shape: get(prefix + name, shape, dtype).to(device)
    norm = lambda n: (t16(n + ".weight", (dim,)), t16(n + ".bias", (dim,)))
    i8 = lambda name, n, k: load_int8_linear(src, prefix, name, n, k, device)
    if level >= 2:
        qkv = i8("attn1.to_qkv", 3 * dim, dim)
    else:
        qkv = Linear16(torch.cat([t16(f"attn1.to_{c}.weight", (dim, dim)) for c in "qkv"], dim=0))
    if level == 3:
        o1, q2, o2 = i8("attn1.to_out.0", dim, dim), i8("attn2.to_q", dim, dim), i8("attn2.to_out.0", dim, dim)
    else:
        o1, q2, o2 = (Linear16(t16(n + ".weight", (dim, dim))) for n in ("attn1.to_out.0", "attn2.to_q", "attn2.to_out.0"))
    ffn = i8("ff.net.2", dim, 4 * dim)
    ffn.bias = t16("ff.net.2.bias", (dim,))
    return BasicTransformerInt8Weights(level, norm("norm1"), norm("norm2"), norm("norm3"), qkv, o1, t16("attn1.to_out.0.bias", (dim,)),
                                       q2, Linear16(t16("attn2.to_k.weight", (dim, cross_dim))),
                                       Linear16(t16("attn2.to_v.weight", (dim, cross_dim))), o2, t16("attn2.to_out.0.bias", (dim,)),
                                       i8("ff.net.0.proj", 8 * dim, dim), t16("ff.net.0.proj.bias", (8 * dim,)), ffn)


def _gemm_int8(q8: torch.Tensor, lin: Int8Linear, dtype, bias=None) -> torch.Tensor:
    """runGemmInt8 on codes that are already quantised with lin's static scale."""
    m = q8.numel() // q8.shape[-1]
    y = ops.int8_linear(q8.view(m, q8.shape[-1]), lin.weight_rows32, lin.weight_scale, lin.input_quant_scale, bias, dtype)
    return y.view(*q8.shape[:-1], y.shape[-1])


def _attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, heads: int) -> torch.Tensor:
    b, s, d = q.shape
    split = lambda t: t.view(b, t.shape[1], heads, d // heads).transpose(1, 2)
    o = torch.nn.functional.scaled_dot_product_attention(split(q), split(k), split(v))
    return o.transpose(1, 2).reshape(b, s, d)


def _ln16(x, gb, eps):
    return torch.nn.functional.layer_norm(x, (x.shape[-1],), gb[0], gb[1], eps)


def _to_out_and_norm(attn: torch.Tensor, residual: torch.Tensor, lin, bias, norm, consumer: Optional[Int8Linear], eps):
    """Output projection of an attention, residual + bias, and the LayerNorm in front of the next linear.
    Returns (codes for `consumer` or the 16-bit normalised tensor when consumer is None, new hidden state)."""
    if isinstance(lin, Int8Linear):  # level 3: quantise, GEMM without bias, then residual + bias + LayerNorm + quantisation fused
        y = _gemm_int8(ops.sq_quant(attn, lin.pre_quant_scale, lin.input_quant_scale), lin, attn.dtype)
        q8, _, hidden = ops.layernorm_int8(y, norm[0], norm[1], consumer.pre_quant_scale, consumer.input_quant_scale, residual, bias, eps)
        return q8, hidden
    hidden = torch.nn.functional.linear(attn, lin.weight, bias) + residual  # GemmWithResidualAndBias, beta = 1
    if consumer is None:
        return _ln16(hidden, norm, eps), hidden
    q8, _, _ = ops.layernorm_int8(hidden, norm[0], norm[1], consumer.pre_quant_scale, consumer.input_quant_scale, eps=eps)
    return q8, hidden


def basic_transformer_int8_block(x: torch.Tensor, encoder_hidden_states: torch.Tensor, w: BasicTransformerInt8Weights,
                                 heads: int, eps: float = 1e-5) -> torch.Tensor:
    """x [B, S, D], encoder_hidden_states [B, Sc, Dc] -> [B, S, D]."""
    b, s, d = x.shape
    x = x.contiguous()
    # self-attention
    if isinstance(w.attn1_qkv, Int8Linear):
        q8, _, _ = ops.layernorm_int8(x, w.norm1[0], w.norm1[1], w.attn1_qkv.pre_quant_scale, w.attn1_qkv.input_quant_scale, eps=eps)
        qkv = _gemm_int8(q8, w.attn1_qkv, x.dtype)
    else:
        qkv = w.attn1_qkv.forward(_ln16(x, w.norm1, eps))
    q, k, v = qkv.split(d, dim=-1)
    a1 = _attention(q, k, v, heads).contiguous()
    # to_out + residual + norm2 (+ quantisation for attn2.to_q at level 3)
    q2_consumer = w.attn2_q if isinstance(w.attn2_q, Int8Linear) else None
    n2, h1 = _to_out_and_norm(a1, x, w.attn1_to_out, w.attn1_to_out_bias, w.norm2, q2_consumer, eps)
    # cross-attention
    q = _gemm_int8(n2, w.attn2_q, x.dtype) if q2_consumer is not None else w.attn2_q.forward(n2)
    a2 = _attention(q, w.attn2_k.forward(encoder_hidden_states), w.attn2_v.forward(encoder_hidden_states), heads).contiguous()
    # to_out + residual + norm3 + quantisation for the GEGLU projection (INT8 at every level)
    q8, h2 = _to_out_and_norm(a2, h1, w.attn2_to_out, w.attn2_to_out_bias, w.norm3, w.geglu, eps)
    # feed-forward
    up = _gemm_int8(q8, w.geglu, x.dtype)
    q8 = ops.geglu_int8(up, w.geglu_bias, w.ffn.pre_quant_scale, w.ffn.input_quant_scale)
    return _gemm_int8(q8, w.ffn, x.dtype, w.ffn.bias) + h2
