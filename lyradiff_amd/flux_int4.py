"""The feed-forward halves of the reference's FLUX INT4 (W4A4 + low-rank) blocks, built from the quantized-linear
kernels.  Attention (QKV, rotary, flash attention) stays with the caller.

  FluxAttnPostInt4Processor<T>::forward   (layers/flux_attn_post_processor/FluxAttnPostInt4Processor.cc:103-215)
      hidden = input + gate_msa * attn                  invokeFusedGateAndResidual
      norm   = adaLN(hidden, scale_mlp, shift_mlp)      invokeLayerNormWithShiftAndScale
      inner  = W4A4Gemm(norm)                           quantise + low-rank down, GEMM + low-rank up   (2 launches + copy)
      inner  = gelu(inner + b1)                         invokeFusedBiasAndGelu
      q2     = e4m3(inner / s_in2)                      invokeCudaD2DScaleCpyConvert
      ff     = q2 . W2^T + b2   (FP8)                   GemmWithResidualAndBias
      out    = hidden + gate_mlp * ff                   invokeFusedGateAndResidual
    Here five launches: gate+residual+adaLN, W4A4 quantise, low-rank down, W4A4 GEMM whose epilogue adds the bias,
    applies GELU and stores only the e4m3 codes, FP8 GEMM whose epilogue applies gate and residual.

  FluxSingleTransformerInt4Block<T>::forward after the attention
  (layers/flux_single_transformer_block/FluxSingleTransformerInt4Block.cc:256-316)
      mlp = gelu(W4A4Gemm_mlp(norm_hidden) + bm); h1 = W4A4Gemm_out1(attn); h2 = W4A4Gemm_out2(mlp)
      o   = (h1 + b1) + h2                              invokeFusedBiasAndResidual
      out = input + gate * o                            invokeFusedGateAndResidual
    Here the bias/GELU, the sum of the two projections and the gate/residual all run in GEMM epilogues.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Union

import torch

from . import ops
from .flux_fp8 import AdaLinear16, ada_fp8_layernorm, load_ada_layernorm
from .weights import FP8Linear, W4A4Linear, load_fp8_linear, load_w4a4_linear


@dataclass
class FluxAttnPostInt4Weights:
    gelu_proj: W4A4Linear  # prefix + "net.0.proj." + {packed_weight, weight_scale, smooth, lora_up, lora_down, bias}
    ff_linear: FP8Linear   # prefix + "net.2" + {.weight, .bias, _input_scale}


@dataclass
class FluxSingleMlpInt4Weights:
    proj_mlp: W4A4Linear    # prefix + "proj_mlp."                    [mlp_scale*D, D], bias
    proj_out_1: W4A4Linear  # prefix + "proj_out.linears.0."          [D, D], bias
    proj_out_2: W4A4Linear  # prefix + "proj_out.linears.1.linear."   [D, mlp_scale*D], no bias


def load_flux_attn_post_int4(src, prefix: str, dim: int, dtype=torch.bfloat16, device="cuda", lora_rank: int = 32):
    """FluxAttnPostInt4ProcessorWeight.cc:18,76-100."""
    return FluxAttnPostInt4Weights(load_w4a4_linear(src, prefix + "net.0.proj.", 4 * dim, dim, lora_rank, True, dtype, device),
                                   load_fp8_linear(src, prefix, "net.2", dim, 4 * dim, dtype, device))


def load_flux_single_mlp_int4(src, prefix: str, dim: int, mlp_scale: int = 4, dtype=torch.bfloat16, device="cuda",
                              lora_rank: int = 32):
    """FluxSingleTransformerInt4BlockWeight.cc:35-37,79-83."""
    return FluxSingleMlpInt4Weights(
        load_w4a4_linear(src, prefix + "proj_mlp.", mlp_scale * dim, dim, lora_rank, True, dtype, device),
        load_w4a4_linear(src, prefix + "proj_out.linears.0.", dim, dim, lora_rank, True, dtype, device),
        load_w4a4_linear(src, prefix + "proj_out.linears.1.linear.", dim, mlp_scale * dim, lora_rank, False, dtype, device))


def _w4a4(lin: W4A4Linear, x2: torch.Tensor, **epilogue):
    """W4A4Gemm::forward (W4A4Gemm.cc:113-169) with epilogue options: quantise, low-rank down, GEMM."""
    if lin.lora_down is not None:
        q, s, act = ops.w4a4_quant_lora_down(x2, lin.smooth, lin.lora_down, torch.float32)
    else:
        (q, s), act = ops.w4a4_quant(x2, lin.smooth, torch.float32), None
    return ops.w4a4_linear(q, lin.weight_rows32, s, lin.weight_scale, lin.bias, x2.dtype, 64, act,
                           lin.lora_up if act is not None else None, **epilogue)


def flux_attn_post_int4(x: torch.Tensor, attn_output: torch.Tensor, msa: torch.Tensor, w: FluxAttnPostInt4Weights,
                        eps: float = 1e-6) -> torch.Tensor:
    """x, attn_output [B, S, D]; msa [6, B, D] -> output [B, S, D]."""
    b, s, d = x.shape
    if tuple(msa.shape) != (6, b, d):
        raise ValueError("msa must be [6, B, D]")
    norm, hidden = ops.gate_residual_layernorm_mod(x, msa[4], msa[3], attn_output, msa[2], eps)
    q2 = _w4a4(w.gelu_proj, norm.view(b * s, d), gelu=2, out_fp8_scale=w.ff_linear.input_scale, want_output=False)
    out = ops.fp8_linear_gated(q2, w.ff_linear.weight_rows32, w.ff_linear.input_scale, w.ff_linear.weight_scale,
                               w.ff_linear.bias, msa[5], hidden.view(b * s, d), rows_per_gate=s)
    return out.view(b, s, d)


def flux_single_mlp_int4(x: torch.Tensor, norm_hidden: torch.Tensor, attn_output: torch.Tensor, gate: torch.Tensor,
                         w: FluxSingleMlpInt4Weights) -> torch.Tensor:
    """x, norm_hidden, attn_output [B, S, D]; gate [B, D] -> output [B, S, D]."""
    b, s, d = x.shape
    m = b * s
    mlp = _w4a4(w.proj_mlp, norm_hidden.view(m, d), gelu=2)
    h1 = _w4a4(w.proj_out_1, attn_output.view(m, d))
    out = _w4a4(w.proj_out_2, mlp, addend=h1, gate=gate, residual=x.view(m, d), rows_per_gate=s)
    return out.view(b, s, d)


# ---- whole INT4 blocks around a caller-supplied attention core ------------------------------------------------------
def _load_ada(src, prefix: str, dim: int, n_chunks: int, full: bool, dtype, device) -> Union[FP8Linear, AdaLinear16]:
    return load_ada_layernorm(src, prefix, dim, n_chunks, full, dtype, device)


def ada_layernorm_int4(x: torch.Tensor, temb: torch.Tensor, linear: Union[FP8Linear, AdaLinear16], n_chunks: int,
                       eps: float = 1e-6):
    """AdaLayerNorm / AdaFP8LayerNorm in front of the W4A4 linears: returns (norm_hidden 16-bit [B, S, D], msa [n_chunks, B, D]).
    The 16-bit adaLN linear of level INT4_W4A4 is not a quantized linear and runs as a plain PyTorch matmul."""
    return ada_fp8_layernorm(x, temb, linear, n_chunks, (), eps=eps)


@dataclass
class FluxSingleBlockInt4Weights:
    norm: Union[FP8Linear, AdaLinear16]  # prefix + "norm.linear"
    to_qkv: W4A4Linear                   # prefix + "attn.to_qkv."  [3D, D], bias
    mlp: FluxSingleMlpInt4Weights


@dataclass
class FluxDoubleBlockInt4Weights:
    norm1: Union[FP8Linear, AdaLinear16]          # prefix + "norm1.linear"
    norm1_context: Union[FP8Linear, AdaLinear16]  # prefix + "norm1_context.linear"
    to_qkv: W4A4Linear        # prefix + "attn.to_qkv."
    to_added_qkv: W4A4Linear  # prefix + "attn.to_added_qkv."
    to_out: W4A4Linear        # prefix + "attn.to_out.0."
    to_add_out: W4A4Linear    # prefix + "attn.to_add_out."
    ff: FluxAttnPostInt4Weights          # prefix + "ff."
    ff_context: FluxAttnPostInt4Weights  # prefix + "ff_context."


def load_flux_single_block_int4(src, prefix: str, dim: int, mlp_scale: int = 4, full: bool = True, dtype=torch.bfloat16,
                                device="cuda", lora_rank: int = 32) -> FluxSingleBlockInt4Weights:
    """FluxSingleTransformerInt4BlockWeight (FluxSingleTransformerInt4BlockWeight.cc:24-37,79-83) and
    FluxSingleAttentionInt4ProcessorWeight::loadWeights (:66-78).  full: quant level INT4_W4A4_FULL (FP8 adaLN linear)."""
    return FluxSingleBlockInt4Weights(_load_ada(src, prefix + "norm.", dim, 3, full, dtype, device),
                                      load_w4a4_linear(src, prefix + "attn.to_qkv.", 3 * dim, dim, lora_rank, True, dtype, device),
                                      load_flux_single_mlp_int4(src, prefix, dim, mlp_scale, dtype, device, lora_rank))


def load_flux_double_block_int4(src, prefix: str, dim: int, full: bool = True, dtype=torch.bfloat16, device="cuda",
                                lora_rank: int = 32) -> FluxDoubleBlockInt4Weights:
    """FluxTransformerInt4BlockWeight (FluxTransformerInt4BlockWeight.cc:27-39,86-90) and
    FluxAttentionInt4ProcessorWeight (FluxAttentionInt4ProcessorWeight.cc:22-25,63-66)."""
    lin = lambda name, n: load_w4a4_linear(src, prefix + "attn." + name + ".", n, dim, lora_rank, True, dtype, device)
    return FluxDoubleBlockInt4Weights(_load_ada(src, prefix + "norm1.", dim, 6, full, dtype, device),
                                      _load_ada(src, prefix + "norm1_context.", dim, 6, full, dtype, device),
                                      lin("to_qkv", 3 * dim), lin("to_added_qkv", 3 * dim), lin("to_out.0", dim),
                                      lin("to_add_out", dim),
                                      load_flux_attn_post_int4(src, prefix + "ff.", dim, dtype, device, lora_rank),
                                      load_flux_attn_post_int4(src, prefix + "ff_context.", dim, dtype, device, lora_rank))


def _w4a4_3d(lin: W4A4Linear, x: torch.Tensor) -> torch.Tensor:
    y = _w4a4(lin, x.reshape(-1, x.shape[-1]))
    return y.view(*x.shape[:-1], y.shape[-1])


def flux_single_block_int4(x: torch.Tensor, temb: torch.Tensor, w: FluxSingleBlockInt4Weights, attention) -> torch.Tensor:
    """FluxSingleTransformerInt4Block<T>::forward (FluxSingleTransformerInt4Block.cc:178-316): adaLN, W4A4 QKV projection
    (its bias added in the GEMM epilogue; the reference adds it in a pass of its own), attention(qkv [B, S, 3D]) -> [B, S, D],
    then the feed-forward tail."""
    norm, msa = ada_layernorm_int4(x, temb, w.norm, 3)
    attn_out = attention(_w4a4_3d(w.to_qkv, norm))
    return flux_single_mlp_int4(x, norm, attn_out.contiguous(), msa[2].contiguous(), w.mlp)


def flux_double_block_int4(x: torch.Tensor, context: torch.Tensor, temb: torch.Tensor, w: FluxDoubleBlockInt4Weights, attention):
    """FluxTransformerInt4Block<T>::forward (FluxTransformerInt4Block.cc:159-246) with FluxAttentionInt4Processor
    (FluxAttentionInt4Processor.cc:206-331).  attention(qkv, context_qkv) -> (attn [B, S, D], context_attn [B, Sc, D]).
    Returns (output, context_output)."""
    n, msa = ada_layernorm_int4(x, temb, w.norm1, 6)
    nc, cmsa = ada_layernorm_int4(context, temb, w.norm1_context, 6)
    attn, cattn = attention(_w4a4_3d(w.to_qkv, n), _w4a4_3d(w.to_added_qkv, nc))
    a_out = _w4a4_3d(w.to_out, attn.contiguous())
    c_out = _w4a4_3d(w.to_add_out, cattn.contiguous())
    return flux_attn_post_int4(x, a_out, msa, w.ff), flux_attn_post_int4(context, c_out, cmsa, w.ff_context)
