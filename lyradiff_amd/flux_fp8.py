"""The FP8 feed-forward halves of the reference's FLUX blocks, built from the quantized-linear kernels.

Two reference call sequences are covered; attention itself (QKV/rotary/flash attention) is not part of the
quantized-linear path and stays with the caller, who passes its output in.

  FluxAttnPostFP8Processor<T>::forward   (layers/flux_attn_post_processor/FluxAttnPostFP8Processor.cc:93-240)
      hidden = input + gate_msa * attn          invokeFusedGateAndResidual
      norm   = adaLN(hidden, scale_mlp, shift_mlp)   invokeLayerNormWithShiftAndScale
      q1     = e4m3(norm / s_in1)               invokeCudaD2DScaleCpyConvert
      inner  = gelu(q1 . W1^T + b1)             GemmWithResidualAndBias (GELU_BIAS epilogue)
      q2     = e4m3(inner / s_in2)              invokeCudaD2DScaleCpyConvert
      ff     = q2 . W2^T + b2                   GemmWithResidualAndBias
      out    = hidden + gate_mlp * ff           invokeFusedGateAndResidual
    Seven launches and five 16-bit intermediate tensors there; three launches here, and only `hidden` is written
    in 16 bits: (1) gate+residual+adaLN+cast, (2) GEMM whose epilogue emits q2 directly, (3) GEMM whose epilogue
    applies the gate and the residual.

  FluxSingleTransformerFP8Block<T>::forward, after the attention (layers/flux_single_transformer_block/
  FluxSingleTransformerFP8Block.cc:209-290)
      q1   = e4m3(norm_hidden / s_mlp)          invokeCudaD2DScaleCpyConvert
      mlp  = q1 . Wm^T + bm                     GemmWithResidualAndBias
      cat  = [attn, gelu(mlp)]                  invokeFusedCatAndGelu
      q2   = e4m3(cat / s_out)                  invokeCudaD2DScaleCpyConvert
      o    = q2 . Wo^T + bo                     GemmWithResidualAndBias
      out  = input + gate * o                   invokeFusedGateAndResidual
    Here: the mlp GEMM writes the codes of gelu(mlp) straight into the right-hand columns of q2, a strided cast
    fills the left-hand (attention) columns, and the output GEMM applies gate and residual in its epilogue.

`msa` tensors follow the reference's layout [n_chunks, B, D] (AdaFP8LayerNorm.cc:100-175): for the double block
chunks 2..5 are gate_msa, shift_mlp, scale_mlp, gate_mlp; for the single block chunk 2 is the gate.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Union

import torch

from . import ops
from .weights import FP8Linear, _source, load_fp8_linear


@dataclass
class FluxAttnPostFP8Weights:
    gelu_proj: FP8Linear  # "net.0.proj": [4D, D]
    ff_linear: FP8Linear  # "net.2":      [D, 4D]


@dataclass
class FluxSingleMlpFP8Weights:
    proj_mlp: FP8Linear  # "proj_mlp": [mlp_scale*D, D]
    proj_out: FP8Linear  # "proj_out": [D, (mlp_scale+1)*D]


def load_flux_attn_post_fp8(src, prefix: str, dim: int, dtype=torch.bfloat16, device="cuda", keep_master: bool = False):
    """Keys prefix + {"net.0.proj", "net.2"} + {".weight", ".bias", "_input_scale"}
    (FluxAttnPostFP8ProcessorWeight.cc:70-89; the block passes prefix + "ff." / "ff_context.")."""
    return FluxAttnPostFP8Weights(load_fp8_linear(src, prefix, "net.0.proj", 4 * dim, dim, dtype, device, keep_master),
                                  load_fp8_linear(src, prefix, "net.2", dim, 4 * dim, dtype, device, keep_master))


def load_flux_single_mlp_fp8(src, prefix: str, dim: int, mlp_scale: int = 4, dtype=torch.bfloat16, device="cuda",
                             keep_master: bool = False):
    """Keys prefix + {"proj_mlp", "proj_out"} + {".weight", ".bias", "_input_scale"}
    (FluxSingleTransformerFP8BlockWeight.cc:94-121)."""
    return FluxSingleMlpFP8Weights(
        load_fp8_linear(src, prefix, "proj_mlp", mlp_scale * dim, dim, dtype, device, keep_master),
        load_fp8_linear(src, prefix, "proj_out", dim, (mlp_scale + 1) * dim, dtype, device, keep_master))


def load_ada_fp8_layernorm(src, prefix: str, dim: int, n_chunks: int, dtype=torch.bfloat16, device="cuda",
                           keep_master: bool = False) -> FP8Linear:
    """Keys prefix + "linear" + {".weight", ".bias", "_input_scale"}, weight [n_chunks*D, D]
    (AdaFP8LayerNormWeight.cc:36-92; the blocks pass prefix + "norm1." / "norm1_context." / "norm.")."""
    return load_fp8_linear(src, prefix, "linear", n_chunks * dim, dim, dtype, device, keep_master)


@dataclass
class AdaLinear16:
    """The 16-bit adaLN linear of the quant levels FP8_W8A8 and INT4_W4A4 (AdaLayerNormWeight, keys prefix +
    "linear.weight" / ".bias"; the blocks take this branch unless the level is ..._FULL,
    FluxTransformerFP8Block.cc:203-211); the _FULL levels hold an FP8Linear in its place (AdaFP8LayerNormWeight)."""
    weight: torch.Tensor  # T [n_chunks*D, D]
    bias: torch.Tensor    # T [n_chunks*D]


def load_ada_layernorm(src, prefix: str, dim: int, n_chunks: int, full: bool, dtype=torch.bfloat16, device="cuda",
                       keep_master: bool = False) -> Union[FP8Linear, AdaLinear16]:
    """full: the level's adaLN linear is FP8 (keys with `_input_scale`); otherwise a plain 16-bit linear."""
    if full:
        return load_ada_fp8_layernorm(src, prefix, dim, n_chunks, dtype, device, keep_master)
    get = _source(src)
    return AdaLinear16(get(prefix + "linear.weight", (n_chunks * dim, dim), dtype).to(device),
                       get(prefix + "linear.bias", (n_chunks * dim,), dtype).to(device))


def ada_fp8_layernorm(x: torch.Tensor, temb: torch.Tensor, linear: Union[FP8Linear, AdaLinear16], n_chunks: int, code_scales=(),
                      switch_scale: bool = False, eps: float = 1e-6, panels: bool = False):
    """AdaFP8LayerNorm<T>::forward (layers/ada_layer_norm/AdaFP8LayerNorm.cc:93-205): msa = FP8 linear of the
    (already SiLU'd) time embedding, stored [n_chunks, B, D]; output = (1 + msa[1]) * LayerNorm(x) + msa[0]
    (msa[0]/msa[1] swapped with switch_scale).  x [B, S, D], temb [B, D].
    code_scales: () -> the 16-bit normalised tensor as the reference writes it; one or two fp32 [1] input scales ->
    the e4m3 codes for the FP8 linears that consume it instead (cast fused, no 16-bit tensor); with panels=True the codes
    are k-panels [D/64, B*S, 64] (ops.fp8_quant_panels) instead of [B, S, D].
    Returns (norm | codes | (codes_a, codes_b), msa)."""
    b, s, d = x.shape
    if isinstance(linear, AdaLinear16):  # not a quantized linear: a plain 16-bit matmul (AdaLayerNorm.cc)
        flat = torch.nn.functional.linear(temb.reshape(b, d), linear.weight, linear.bias)
    else:
        q = ops.fp8_scale_cast(temb.reshape(b, d), linear.input_scale)
        flat = ops.fp8_linear(q, linear.weight_rows32, linear.input_scale, linear.weight_scale, linear.bias, out_dtype=x.dtype)
    msa = flat.view(b, n_chunks, d).transpose(0, 1).contiguous() if b > 1 else flat.view(n_chunks, 1, d)  # invokeTranspose102
    shift, scale = (msa[1], msa[0]) if switch_scale else (msa[0], msa[1])
    if len(code_scales) == 0:
        return ops.gate_residual_layernorm_mod(x, scale, shift, eps=eps), msa
    if len(code_scales) == 1:
        return ops.layernorm_mod_fp8(x, scale, shift, code_scales[0], eps, panels=panels), msa
    return ops.layernorm_mod_fp8_dual(x, scale, shift, code_scales[0], code_scales[1], eps, panels=panels), msa


def flux_attn_post_fp8(x: torch.Tensor, attn_output: torch.Tensor, msa: torch.Tensor, w: FluxAttnPostFP8Weights,
                       eps: float = 1e-6) -> torch.Tensor:
    """x, attn_output [B, S, D]; msa [6, B, D] -> output [B, S, D] in three launches."""
    b, s, d = x.shape
    if tuple(msa.shape) != (6, b, d):
        raise ValueError("msa must be [6, B, D]")
    gate_msa, shift_mlp, scale_mlp, gate_mlp = msa[2], msa[3], msa[4], msa[5]
    # the two FP8 activations of the sequence travel as k-panels [K/64, B*S, 64] (whole cache lines for the GEMMs' transfers)
    q1, hidden = ops.gate_residual_layernorm_mod_fp8(attn_output, gate_msa, x, scale_mlp, shift_mlp, w.gelu_proj.input_scale, eps,
                                                     panels=True)
    q2 = ops.fp8_linear_codes_panels(q1, w.gelu_proj.weight_rows32, w.gelu_proj.input_scale, w.gelu_proj.weight_scale,
                                     w.gelu_proj.bias, w.ff_linear.input_scale, gelu=1, round_dtype=x.dtype)
    out = ops.fp8_linear_gated_panels(q2, w.ff_linear.weight_rows32, w.ff_linear.input_scale, w.ff_linear.weight_scale,
                                      w.ff_linear.bias, gate_mlp, hidden.view(b * s, d), rows_per_gate=s)
    return out.view(b, s, d)


def flux_single_mlp_fp8(x: torch.Tensor, norm_hidden, attn_output: torch.Tensor, gate: torch.Tensor,
                        w: FluxSingleMlpFP8Weights, norm_in_panels: bool = False) -> torch.Tensor:
    """x, attn_output [B, S, D]; gate [B, D] (chunk 2 of the single block's msa) -> output [B, S, D].
    norm_hidden is either the 16-bit adaLN output [B, S, D] (cast here with proj_mlp's input scale) or its e4m3
    codes for proj_mlp: uint8 [B, S, D], or with norm_in_panels uint8 k-panels [D/64, B*S, 64] (the second output of
    ops.layernorm_mod_fp8_dual)."""
    b, s, d = x.shape
    m = b * s
    f = w.proj_mlp.weight_rows32.shape[0]
    if norm_hidden.dtype == torch.uint8 and not norm_in_panels:  # row-major codes from the caller: the row-major sequence
        q2 = torch.empty((m, d + f), dtype=torch.uint8, device=x.device)
        ops.fp8_scale_cast_into(attn_output.view(m, d), w.proj_out.input_scale, q2, 0)
        ops.fp8_linear_codes(norm_hidden.view(m, d), w.proj_mlp.weight_rows32, w.proj_mlp.input_scale, w.proj_mlp.weight_scale,
                             w.proj_mlp.bias, w.proj_out.input_scale, gelu=2, round_dtype=x.dtype, out=q2, col_offset=d)
        out = ops.fp8_linear_gated(q2, w.proj_out.weight_rows32, w.proj_out.input_scale, w.proj_out.weight_scale,
                                   w.proj_out.bias, gate, x.view(m, d), rows_per_gate=s)
        return out.view(b, s, d)
    # every FP8 activation as k-panels: the concatenated input of proj_out is [ (D + F)/64, M, 64 ], its two column blocks
    # (attention output, GELU of proj_mlp) are runs of whole panels
    q1 = norm_hidden if norm_hidden.dtype == torch.uint8 else ops.fp8_scale_cast_panels(norm_hidden.view(m, d), w.proj_mlp.input_scale)
    q2 = torch.empty(((d + f) // 64, m, 64), dtype=torch.uint8, device=x.device)
    ops.fp8_scale_cast_panels(attn_output.view(m, d), w.proj_out.input_scale, out=q2, col_offset=0)
    ops.fp8_linear_codes_panels(q1, w.proj_mlp.weight_rows32, w.proj_mlp.input_scale, w.proj_mlp.weight_scale,
                                w.proj_mlp.bias, w.proj_out.input_scale, gelu=2, round_dtype=x.dtype, out=q2, col_offset=d)
    out = ops.fp8_linear_gated_panels(q2, w.proj_out.weight_rows32, w.proj_out.input_scale, w.proj_out.weight_scale,
                                      w.proj_out.bias, gate, x.view(m, d), rows_per_gate=s)
    return out.view(b, s, d)


# ---- whole blocks around a caller-supplied attention --------------------------------------------------------------------
# Everything the reference's FP8 blocks run through a quantized linear is here; `attention` is the caller's function
# for the part in between (q/k RMSNorm, rotary embedding, scaled-dot-product attention), which is not quantized.

@dataclass
class FluxSingleBlockFP8Weights:
    norm: Union[FP8Linear, AdaLinear16]  # prefix + "norm.linear"  [3D, D]
    to_qkv: FP8Linear    # prefix + "attn.to_qkv"  [3D, D]
    mlp: FluxSingleMlpFP8Weights


@dataclass
class FluxDoubleBlockFP8Weights:
    norm1: Union[FP8Linear, AdaLinear16]          # prefix + "norm1.linear"          [6D, D]
    norm1_context: Union[FP8Linear, AdaLinear16]  # prefix + "norm1_context.linear"  [6D, D]
    to_qkv: FP8Linear          # prefix + "attn.to_qkv"
    to_added_qkv: FP8Linear    # prefix + "attn.to_added_qkv"
    to_out: FP8Linear          # prefix + "attn.to_out.0"
    to_add_out: FP8Linear      # prefix + "attn.to_add_out"
    ff: FluxAttnPostFP8Weights          # prefix + "ff."
    ff_context: FluxAttnPostFP8Weights  # prefix + "ff_context."


def load_flux_single_block_fp8(src, prefix: str, dim: int, mlp_scale: int = 4, dtype=torch.bfloat16, device="cuda",
                               keep_master: bool = False, full: bool = True) -> FluxSingleBlockFP8Weights:
    """FluxSingleTransformerFP8BlockWeight::loadWeights (FluxSingleTransformerFP8BlockWeight.cc:94-121).
    full: quant level FP8_W8A8_FULL (FP8 adaLN linear); False: level FP8_W8A8 (16-bit adaLN linear)."""
    return FluxSingleBlockFP8Weights(load_ada_layernorm(src, prefix + "norm.", dim, 3, full, dtype, device, keep_master),
                                     load_fp8_linear(src, prefix + "attn.", "to_qkv", 3 * dim, dim, dtype, device, keep_master),
                                     load_flux_single_mlp_fp8(src, prefix, dim, mlp_scale, dtype, device, keep_master))


def load_flux_double_block_fp8(src, prefix: str, dim: int, dtype=torch.bfloat16, device="cuda",
                               keep_master: bool = False, full: bool = True) -> FluxDoubleBlockFP8Weights:
    """FluxTransformerFP8BlockWeight::loadWeights (FluxTransformerFP8BlockWeight.cc:78-91) and
    FluxAttentionFP8ProcessorWeight::loadWeights (FluxAttentionFP8ProcessorWeight.cc:113-138)."""
    lin = lambda name, n, k: load_fp8_linear(src, prefix + "attn.", name, n, k, dtype, device, keep_master)
    return FluxDoubleBlockFP8Weights(load_ada_layernorm(src, prefix + "norm1.", dim, 6, full, dtype, device, keep_master),
                                     load_ada_layernorm(src, prefix + "norm1_context.", dim, 6, full, dtype, device, keep_master),
                                     lin("to_qkv", 3 * dim, dim), lin("to_added_qkv", 3 * dim, dim), lin("to_out.0", dim, dim),
                                     lin("to_add_out", dim, dim),
                                     load_flux_attn_post_fp8(src, prefix + "ff.", dim, dtype, device, keep_master),
                                     load_flux_attn_post_fp8(src, prefix + "ff_context.", dim, dtype, device, keep_master))


def _linear_from_panels(lin: FP8Linear, panels: torch.Tensor, batch: int, dtype) -> torch.Tensor:
    """FP8 linear on codes in k-panels [K/64, B*S, 64] -> [B, S, N]."""
    y = ops.fp8_linear_panels(panels, lin.weight_rows32, lin.input_scale, lin.weight_scale, lin.bias, None, dtype)
    return y.view(batch, y.shape[0] // batch, y.shape[1])


def flux_single_block_fp8(x: torch.Tensor, temb: torch.Tensor, w: FluxSingleBlockFP8Weights, attention) -> torch.Tensor:
    """FluxSingleTransformerFP8Block<T>::forward (FluxSingleTransformerFP8Block.cc:163-291).  x [B, S, D], temb [B, D]
    (SiLU already applied); attention(qkv [B, S, 3D]) -> [B, S, D].  One adaLN read yields the codes for to_qkv and for
    proj_mlp; five launches besides the attention."""
    (c_qkv, c_mlp), msa = ada_fp8_layernorm(x, temb, w.norm, 3, (w.to_qkv.input_scale, w.mlp.proj_mlp.input_scale), panels=True)
    attn_out = attention(_linear_from_panels(w.to_qkv, c_qkv, x.shape[0], x.dtype))
    return flux_single_mlp_fp8(x, c_mlp, attn_out.contiguous(), msa[2].contiguous(), w.mlp, norm_in_panels=True)


def flux_double_block_fp8(x: torch.Tensor, context: torch.Tensor, temb: torch.Tensor, w: FluxDoubleBlockFP8Weights, attention):
    """FluxTransformerFP8Block<T>::forward (FluxTransformerFP8Block.cc:159-262) with FluxAttentionFP8Processor
    (FluxAttentionFP8Processor.cc:165-360).  attention(qkv [B, S, 3D], context_qkv [B, Sc, 3D]) -> (attn [B, S, D],
    context_attn [B, Sc, D]).  Returns (output, context_output)."""
    c, msa = ada_fp8_layernorm(x, temb, w.norm1, 6, (w.to_qkv.input_scale,), panels=True)
    cc, cmsa = ada_fp8_layernorm(context, temb, w.norm1_context, 6, (w.to_added_qkv.input_scale,), panels=True)
    attn, cattn = attention(_linear_from_panels(w.to_qkv, c, x.shape[0], x.dtype),
                            _linear_from_panels(w.to_added_qkv, cc, context.shape[0], x.dtype))
    a_out = w.to_out.forward(attn.contiguous())
    c_out = w.to_add_out.forward(cattn.contiguous())
    return flux_attn_post_fp8(x, a_out, msa, w.ff), flux_attn_post_fp8(context, c_out, cmsa, w.ff_context)
