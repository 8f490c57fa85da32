"""torch.ops.lyradiff.* : the tensor-level functions of ops.py registered as PyTorch custom operators.

The reference exposes its kernels to Python through a TORCH_LIBRARY named `lyradiff`
(src/lyradiff/th_op/pybind.cc:9-97) and functional operators through torch::RegisterOperators
(src/lyradiff/layers/gemm_utils/WeightOnlyQuantOps.cc:326-351).  Here the same namespace carries
the quantized-linear operators; each one has a shape-only ("fake") implementation so that the
operators can be traced and shape-checked without a GPU, and a device implementation that calls the
C ABI on the current HIP stream.  Importing this module registers the operators once per process.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch
from torch import Tensor

from . import ops as _ops

_lib_op = torch.library.custom_op
NAMES = ("sq_quant", "sq_quant_dynamic", "geglu_int8_dynamic", "int8_linear", "fp8_quant", "fp8_scale_cast", "fp8_linear",
         "w4a4_quant", "w4a4_linear", "repack_weight", "lora_down", "layernorm_mod_fp8", "gate_residual_layernorm_mod_fp8",
         "fp8_linear_codes", "fp8_linear_gated", "flux_attn_post_fp8", "flux_single_mlp_fp8", "rmsnorm_rope",
         "fp8_linear_max", "fp8_gelu_quant", "w4a4_quant_lora_down", "fp8_quant_panels", "fp8_gelu_quant_panels",
         "fp8_linear_panels", "sq_quant_dynamic_panels", "int8_linear_panels")


@_lib_op("lyradiff::sq_quant", mutates_args=())
def sq_quant(x: Tensor, pre_quant_scale: Optional[Tensor], input_quant_scale: Tensor, per_token: bool = False) -> Tensor:
    return _ops.sq_quant(x, pre_quant_scale, input_quant_scale, per_token)


@sq_quant.register_fake
def _(x, pre_quant_scale, input_quant_scale, per_token=False):
    return x.new_empty(x.shape, dtype=torch.int8)


@_lib_op("lyradiff::sq_quant_dynamic", mutates_args=())
def sq_quant_dynamic(x: Tensor, pre_quant_scale: Optional[Tensor] = None) -> Tuple[Tensor, Tensor]:
    return _ops.sq_quant_dynamic(x, pre_quant_scale)


@sq_quant_dynamic.register_fake
def _(x, pre_quant_scale=None):
    rows = x.numel() // x.shape[-1] if x.shape[-1] else 0
    return x.new_empty(x.shape, dtype=torch.int8), x.new_empty((rows,), dtype=torch.float32)


@_lib_op("lyradiff::geglu_int8_dynamic", mutates_args=())
def geglu_int8_dynamic(hidden: Tensor, bias: Optional[Tensor] = None,
                       pre_quant_scale: Optional[Tensor] = None) -> Tuple[Tensor, Tensor]:
    return _ops.geglu_int8_dynamic(hidden, bias, pre_quant_scale)


@geglu_int8_dynamic.register_fake
def _(hidden, bias=None, pre_quant_scale=None):
    d = hidden.shape[-1] // 2
    rows = hidden.numel() // (2 * d) if d else 0
    return hidden.new_empty(tuple(hidden.shape[:-1]) + (d,), dtype=torch.int8), hidden.new_empty((rows,), dtype=torch.float32)


@_lib_op("lyradiff::int8_linear", mutates_args=())
def int8_linear(a_q: Tensor, w_rows32: Tensor, alpha_col: Optional[Tensor], alpha_row: Optional[Tensor],
                bias: Optional[Tensor] = None, out_dtype: torch.dtype = torch.float16) -> Tensor:
    return _ops.int8_linear(a_q, w_rows32, alpha_col, alpha_row, bias, out_dtype)


@int8_linear.register_fake
def _(a_q, w_rows32, alpha_col, alpha_row, bias=None, out_dtype=torch.float16):
    return a_q.new_empty((a_q.shape[0], w_rows32.shape[0]), dtype=out_dtype)


@_lib_op("lyradiff::sq_quant_dynamic_panels", mutates_args=())
def sq_quant_dynamic_panels(x: Tensor, pre_quant_scale: Optional[Tensor] = None) -> Tuple[Tensor, Tensor]:
    return _ops.sq_quant_dynamic_panels(x, pre_quant_scale)


@sq_quant_dynamic_panels.register_fake
def _(x, pre_quant_scale=None):
    return x.new_empty((x.shape[1] // 64, x.shape[0], 64), dtype=torch.int8), x.new_empty((x.shape[0],), dtype=torch.float32)


@_lib_op("lyradiff::int8_linear_panels", mutates_args=())
def int8_linear_panels(a_panels: Tensor, w_rows32: Tensor, alpha_col: Optional[Tensor], alpha_row: Optional[Tensor],
                       bias: Optional[Tensor] = None, out_dtype: torch.dtype = torch.float16) -> Tensor:
    return _ops.int8_linear_panels(a_panels, w_rows32, alpha_col, alpha_row, bias, out_dtype)


@int8_linear_panels.register_fake
def _(a_panels, w_rows32, alpha_col, alpha_row, bias=None, out_dtype=torch.float16):
    return a_panels.new_empty((a_panels.shape[1], w_rows32.shape[0]), dtype=out_dtype)


@_lib_op("lyradiff::fp8_quant", mutates_args=())
def fp8_quant(x: Tensor) -> Tuple[Tensor, Tensor]:
    return _ops.fp8_quant(x)


@fp8_quant.register_fake
def _(x):
    return x.new_empty(x.shape, dtype=torch.uint8), x.new_empty((1,), dtype=torch.float32)


@_lib_op("lyradiff::fp8_scale_cast", mutates_args=())
def fp8_scale_cast(x: Tensor, scale: Tensor, invert: bool = True) -> Tensor:
    return _ops.fp8_scale_cast(x, scale, invert)


@fp8_scale_cast.register_fake
def _(x, scale, invert=True):
    return x.new_empty(x.shape, dtype=torch.uint8)


@_lib_op("lyradiff::fp8_linear", mutates_args=())
def fp8_linear(a_q: Tensor, w_rows32: Tensor, a_scale: Tensor, b_scale: Tensor, bias: Optional[Tensor] = None,
               gelu: bool = False, residual: Optional[Tensor] = None, beta: float = 0.0,
               out_dtype: torch.dtype = torch.bfloat16) -> Tensor:
    return _ops.fp8_linear(a_q, w_rows32, a_scale, b_scale, bias, gelu, residual, beta, out_dtype)


@fp8_linear.register_fake
def _(a_q, w_rows32, a_scale, b_scale, bias=None, gelu=False, residual=None, beta=0.0, out_dtype=torch.bfloat16):
    return a_q.new_empty((a_q.shape[0], w_rows32.shape[0]), dtype=out_dtype)


@_lib_op("lyradiff::fp8_linear_max", mutates_args=("out_max",))
def fp8_linear_max(a_q: Tensor, w_rows32: Tensor, a_scale: Tensor, b_scale: Tensor, bias: Optional[Tensor], out_max: Tensor,
                   out_dtype: torch.dtype = torch.bfloat16) -> Tensor:
    return _ops.fp8_linear_max(a_q, w_rows32, a_scale, b_scale, bias, out_max, out_dtype)


@fp8_linear_max.register_fake
def _(a_q, w_rows32, a_scale, b_scale, bias, out_max, out_dtype=torch.bfloat16):
    return a_q.new_empty((a_q.shape[0], w_rows32.shape[0]), dtype=out_dtype)


@_lib_op("lyradiff::fp8_gelu_quant", mutates_args=())
def fp8_gelu_quant(y: Tensor, y_max: Tensor) -> Tuple[Tensor, Tensor]:
    return _ops.fp8_gelu_quant(y, y_max)


@fp8_gelu_quant.register_fake
def _(y, y_max):
    return y.new_empty(y.shape, dtype=torch.uint8), y.new_empty((1,), dtype=torch.float32)


@_lib_op("lyradiff::fp8_quant_panels", mutates_args=())
def fp8_quant_panels(x: Tensor) -> Tuple[Tensor, Tensor]:
    return _ops.fp8_quant_panels(x)


@fp8_quant_panels.register_fake
def _(x):
    return x.new_empty((x.shape[1] // 64, x.shape[0], 64), dtype=torch.uint8), x.new_empty((1,), dtype=torch.float32)


@_lib_op("lyradiff::fp8_gelu_quant_panels", mutates_args=())
def fp8_gelu_quant_panels(y: Tensor, y_max: Tensor) -> Tuple[Tensor, Tensor]:
    return _ops.fp8_gelu_quant_panels(y, y_max)


@fp8_gelu_quant_panels.register_fake
def _(y, y_max):
    return y.new_empty((y.shape[1] // 64, y.shape[0], 64), dtype=torch.uint8), y.new_empty((1,), dtype=torch.float32)


@_lib_op("lyradiff::fp8_linear_panels", mutates_args=("out_max",))
def fp8_linear_panels(a_panels: Tensor, w_rows32: Tensor, a_scale: Tensor, b_scale: Tensor, bias: Optional[Tensor],
                      out_max: Optional[Tensor] = None, out_dtype: torch.dtype = torch.bfloat16) -> Tensor:
    return _ops.fp8_linear_panels(a_panels, w_rows32, a_scale, b_scale, bias, out_max, out_dtype)


@fp8_linear_panels.register_fake
def _(a_panels, w_rows32, a_scale, b_scale, bias, out_max=None, out_dtype=torch.bfloat16):
    return a_panels.new_empty((a_panels.shape[1], w_rows32.shape[0]), dtype=out_dtype)


@_lib_op("lyradiff::w4a4_quant_lora_down", mutates_args=())
def w4a4_quant_lora_down(x: Tensor, smooth: Optional[Tensor], lora_down_w: Tensor,
                         scale_dtype: torch.dtype = torch.float32) -> Tuple[Tensor, Tensor, Tensor]:
    return _ops.w4a4_quant_lora_down(x, smooth, lora_down_w, scale_dtype)


@w4a4_quant_lora_down.register_fake
def _(x, smooth, lora_down_w, scale_dtype=torch.float32):
    m, k = x.shape
    return (x.new_empty((m, k // 8), dtype=torch.int32), x.new_empty((m, k // 64), dtype=scale_dtype),
            x.new_empty((m, lora_down_w.shape[0])))


@_lib_op("lyradiff::w4a4_quant", mutates_args=())
def w4a4_quant(x: Tensor, smooth: Optional[Tensor] = None, scale_dtype: torch.dtype = torch.float32,
               group: int = 64) -> Tuple[Tensor, Tensor]:
    return _ops.w4a4_quant(x, smooth, scale_dtype, group)


@w4a4_quant.register_fake
def _(x, smooth=None, scale_dtype=torch.float32, group=64):
    m, k = x.shape
    return x.new_empty((m, k // 8), dtype=torch.int32), x.new_empty((m, k // group), dtype=scale_dtype)


@_lib_op("lyradiff::w4a4_linear", mutates_args=())
def w4a4_linear(a_words: Tensor, w_rows32: Tensor, sA: Tensor, sB: Tensor, bias: Optional[Tensor] = None,
                out_dtype: torch.dtype = torch.bfloat16, group: int = 64) -> Tensor:
    return _ops.w4a4_linear(a_words, w_rows32, sA, sB, bias, out_dtype, group)


@w4a4_linear.register_fake
def _(a_words, w_rows32, sA, sB, bias=None, out_dtype=torch.bfloat16, group=64):
    return a_words.new_empty((a_words.shape[0], w_rows32.shape[0]), dtype=out_dtype)


@_lib_op("lyradiff::repack_weight", mutates_args=())
def repack_weight(w_bytes: Tensor) -> Tensor:
    return _ops.repack_weight(w_bytes)


@repack_weight.register_fake
def _(w_bytes):
    return torch.empty_like(w_bytes)


@_lib_op("lyradiff::lora_down", mutates_args=())
def lora_down(x: Tensor, lora_down_w: Tensor) -> Tensor:
    return _ops.lora_down(x, lora_down_w)


@lora_down.register_fake
def _(x, lora_down_w):
    return x.new_empty((x.shape[0], lora_down_w.shape[0]))


@_lib_op("lyradiff::rmsnorm_rope", mutates_args=())
def rmsnorm_rope(qkv: Tensor, norm_qk: Tensor, rope: Tensor, heads: int, context_qkv: Optional[Tensor] = None,
                 norm_added_qk: Optional[Tensor] = None, eps: float = 1e-6) -> Tensor:
    return _ops.rmsnorm_rope(qkv, norm_qk, rope, heads, context_qkv, norm_added_qk, eps)


@rmsnorm_rope.register_fake
def _(qkv, norm_qk, rope, heads, context_qkv=None, norm_added_qk=None, eps=1e-6):
    sc = 0 if context_qkv is None else context_qkv.shape[1]
    return qkv.new_empty((qkv.shape[0], sc + qkv.shape[1], 3, heads, qkv.shape[2] // (3 * heads)))


@_lib_op("lyradiff::layernorm_mod_fp8", mutates_args=())
def layernorm_mod_fp8(x: Tensor, scale: Tensor, shift: Tensor, input_scale: Tensor, eps: float = 1e-6) -> Tensor:
    return _ops.layernorm_mod_fp8(x, scale, shift, input_scale, eps)


@layernorm_mod_fp8.register_fake
def _(x, scale, shift, input_scale, eps=1e-6):
    return x.new_empty(x.shape, dtype=torch.uint8)


@_lib_op("lyradiff::gate_residual_layernorm_mod_fp8", mutates_args=())
def gate_residual_layernorm_mod_fp8(attn: Tensor, gate: Tensor, x: Tensor, scale: Tensor, shift: Tensor, input_scale: Tensor,
                                    eps: float = 1e-6) -> Tuple[Tensor, Tensor]:
    return _ops.gate_residual_layernorm_mod_fp8(attn, gate, x, scale, shift, input_scale, eps)


@gate_residual_layernorm_mod_fp8.register_fake
def _(attn, gate, x, scale, shift, input_scale, eps=1e-6):
    return x.new_empty(x.shape, dtype=torch.uint8), torch.empty_like(x)


@_lib_op("lyradiff::fp8_linear_codes", mutates_args=())
def fp8_linear_codes(a_q: Tensor, w_rows32: Tensor, a_scale: Tensor, b_scale: Tensor, bias: Optional[Tensor],
                     out_fp8_scale: Tensor, gelu: int = 0, round_dtype: torch.dtype = torch.bfloat16) -> Tensor:
    return _ops.fp8_linear_codes(a_q, w_rows32, a_scale, b_scale, bias, out_fp8_scale, gelu, round_dtype)


@fp8_linear_codes.register_fake
def _(a_q, w_rows32, a_scale, b_scale, bias, out_fp8_scale, gelu=0, round_dtype=torch.bfloat16):
    return a_q.new_empty((a_q.shape[0], w_rows32.shape[0]), dtype=torch.uint8)


@_lib_op("lyradiff::fp8_linear_gated", mutates_args=())
def fp8_linear_gated(a_q: Tensor, w_rows32: Tensor, a_scale: Tensor, b_scale: Tensor, bias: Optional[Tensor], gate: Tensor,
                     residual: Tensor, rows_per_gate: int) -> Tensor:
    return _ops.fp8_linear_gated(a_q, w_rows32, a_scale, b_scale, bias, gate, residual, rows_per_gate)


@fp8_linear_gated.register_fake
def _(a_q, w_rows32, a_scale, b_scale, bias, gate, residual, rows_per_gate):
    return residual.new_empty((a_q.shape[0], w_rows32.shape[0]))


# ---- block level: the FP8 feed-forward halves of the FLUX blocks as single operators --------------------------------
# Weights travel as flat tensor lists (rows32 codes, weight scale, input scale, bias per linear), the form a
# torch-side module keeps after loading a state dict with lyradiff_amd.flux_fp8.load_*.
def _fp8_lin(w: Tensor, ws: Tensor, s_in: Tensor, b: Tensor):
    from .weights import FP8Linear

    return FP8Linear(w, ws, s_in, b)


@_lib_op("lyradiff::flux_attn_post_fp8", mutates_args=())
def flux_attn_post_fp8(x: Tensor, attn_output: Tensor, msa: Tensor, w1: Tensor, w1_scale: Tensor, in1_scale: Tensor, b1: Tensor,
                       w2: Tensor, w2_scale: Tensor, in2_scale: Tensor, b2: Tensor) -> Tensor:
    from . import flux_fp8 as F

    return F.flux_attn_post_fp8(x, attn_output, msa, F.FluxAttnPostFP8Weights(_fp8_lin(w1, w1_scale, in1_scale, b1),
                                                                              _fp8_lin(w2, w2_scale, in2_scale, b2)))


@flux_attn_post_fp8.register_fake
def _(x, attn_output, msa, w1, w1_scale, in1_scale, b1, w2, w2_scale, in2_scale, b2):
    return torch.empty_like(x)


@_lib_op("lyradiff::flux_single_mlp_fp8", mutates_args=())
def flux_single_mlp_fp8(x: Tensor, norm_hidden: Tensor, attn_output: Tensor, gate: Tensor, wm: Tensor, wm_scale: Tensor,
                        inm_scale: Tensor, bm: Tensor, wo: Tensor, wo_scale: Tensor, ino_scale: Tensor, bo: Tensor) -> Tensor:
    from . import flux_fp8 as F

    return F.flux_single_mlp_fp8(x, norm_hidden, attn_output, gate,
                                 F.FluxSingleMlpFP8Weights(_fp8_lin(wm, wm_scale, inm_scale, bm), _fp8_lin(wo, wo_scale, ino_scale, bo)))


@flux_single_mlp_fp8.register_fake
def _(x, norm_hidden, attn_output, gate, wm, wm_scale, inm_scale, bm, wo, wo_scale, ino_scale, bo):
    return torch.empty_like(x)


# ---- torch.ops.lyrallms.*: the weight-only utility operators of the reference -----------------------------------------
# (torch::RegisterOperators("lyrallms::...") in src/lyradiff/layers/gemm_utils/WeightOnlyQuantOps.cc:326-351: CPU tensors in,
# CPU tensors out, used by conversion scripts).  quant_type is torch.int8 or torch.quint4x2 as there (:30-60).  The
# "processed" weight is this library's prepared layout (lq_repack_weight_only, a device kernel: the tensor makes a round
# trip to the GPU), the counterpart of the reference's NVIDIA-specific interleave.
_LLM = ("symmetric_quantize_last_axis_of_batched_matrix", "_symmetric_quantize_last_axis_of_batched_matrix",
        "preprocess_weights_for_mixed_gemm", "pack_int8_tensor_to_packed_int4", "unpack_int4_packed_tensor_to_int8")


def _bits(quant_type: torch.dtype) -> int:
    if quant_type == torch.int8:
        return 8
    if quant_type == torch.quint4x2:
        return 4
    raise RuntimeError("Must be int4 or int8 quantization")  # check_quant_type_allowed, WeightOnlyQuantOps.cc:30-37


def _prepare(q_unprocessed: Tensor, bits: int) -> Tensor:
    if q_unprocessed.dim() == 3:
        return torch.stack([_prepare(w, bits) for w in q_unprocessed])
    return _ops.repack_weight_only(q_unprocessed.cuda(), "int8" if bits == 8 else "int4").cpu().view(torch.int8)


@_lib_op("lyrallms::pack_int8_tensor_to_packed_int4", mutates_args=(), device_types="cpu")
def llm_pack_int4(weight: Tensor) -> Tensor:
    from .weights import pack_int8_tensor_to_packed_int4

    return pack_int8_tensor_to_packed_int4(weight)


@_lib_op("lyrallms::unpack_int4_packed_tensor_to_int8", mutates_args=(), device_types="cpu")
def llm_unpack_int4(weight: Tensor) -> Tensor:
    from .weights import unpack_int4_packed_tensor_to_int8

    return unpack_int4_packed_tensor_to_int8(weight)


@_lib_op("lyrallms::preprocess_weights_for_mixed_gemm", mutates_args=(), device_types="cpu")
def llm_preprocess(row_major_quantized_weight: Tensor, quant_type: torch.dtype) -> Tensor:
    if row_major_quantized_weight.dtype != torch.int8:
        raise RuntimeError("Quantized tensor must be int8 dtype")
    return _prepare(row_major_quantized_weight.contiguous(), _bits(quant_type))


@_lib_op("lyrallms::_symmetric_quantize_last_axis_of_batched_matrix", mutates_args=(), device_types="cpu")
def llm_squant_all(weight: Tensor, quant_type: torch.dtype) -> list[Tensor]:
    from .weights import symmetric_quantize_last_axis_of_batched_matrix as squant

    if weight.dtype not in (torch.float16, torch.bfloat16):
        raise RuntimeError("Invalid datatype. Weight must be BF16/FP16")
    bits = _bits(quant_type)
    q, scales = squant(weight.contiguous(), bits)
    return [q, _prepare(q, bits), scales]


@_lib_op("lyrallms::symmetric_quantize_last_axis_of_batched_matrix", mutates_args=(), device_types="cpu")
def llm_squant(weight: Tensor, quant_type: torch.dtype) -> list[Tensor]:
    return list(llm_squant_all(weight, quant_type)[1:])
