"""Loaders for the reference's on-disk / in-memory weight formats of the three quantized linears, and the
linear modules that run them.

The reference keeps each tensor of a linear either as a raw little-endian `.bin` file (`loadWeightFromBin`,
src/lyradiff/utils/memory_utils.cu:251-314: no header, the element type is implied by the caller) or as an entry of
a `{name: pointer}` cache filled from a state dict (`loadWeightsFromCache`).  The names:

  INT8 SmoothQuant  prefix + name + {".weight_int8", ".weight_quant_scale", ".input_quant_scale",
                    ".pre_quant_scale"}                       MACROLoadLinearInt8WeightFromBin,
                                                              src/lyradiff/utils/common_macro_def.h:51-59
  FP8               prefix + name + {".weight", ".bias", "_input_scale"}; the 16-bit weight is quantised to e4m3
                    with a per-tensor scale WHEN IT IS LOADED   MACROLoadFP8WeightFromBin / ...FromCache,
                                                              common_macro_def.h:66-92
  W4A4              prefix + {"packed_weight", "weight_scale", "lora_up", "lora_down", "smooth", "bias"}
                                                              src/lyradiff/layers/w4a4_gemm_block/W4A4GemmWeight.cc:65-83

Every loader ends with the one-time repack of the weight into the rows32 layout the GEMMs read.  The modules hold
device tensors only and call lyradiff_amd.ops (the C ABI); there is no CPU path.
"""
from __future__ import annotations

import os
from dataclasses import dataclass
from typing import Callable, Mapping, Optional

import numpy as np
import torch

from . import ops

_NP = {torch.float32: np.float32, torch.float16: np.float16, torch.int8: np.int8, torch.uint8: np.uint8}


def read_bin(path: str, shape, dtype: torch.dtype) -> torch.Tensor:
    """One raw `.bin` tensor (host).  bf16 files are read as 16-bit words and reinterpreted."""
    count = int(np.prod(shape))
    if dtype == torch.bfloat16:
        raw = np.fromfile(path, dtype=np.uint16)
    else:
        raw = np.fromfile(path, dtype=_NP[dtype])
    if raw.size != count:
        raise ValueError(f"{path}: holds {raw.size} elements, expected {count} for shape {tuple(shape)}")
    t = torch.from_numpy(raw.reshape(shape))
    return t.view(torch.bfloat16) if dtype == torch.bfloat16 else t


class BinFiles:
    """The reference's raw weight files under `root` (file name = root + tensor name + ".bin"), with the element type
    the files of the 16-bit members were written in (`model_dtype` "fp32", "fp16" or "bf16": the FtCudaDataType argument
    of loadWeights).  Members the reference always stores as fp32 or int8 (scales, smoothing vectors, packed codes) are
    read as such; 16-bit members are converted from the file type to the requested type with round-to-nearest-even, as
    loadWeightFromBin does (utils/memory_utils.cu:295-360)."""

    _FILE = {"fp32": torch.float32, "fp16": torch.float16, "bf16": torch.bfloat16}

    def __init__(self, root: str, model_dtype: str = "fp32"):
        if model_dtype not in self._FILE:
            raise ValueError("wrong model_dtype")  # the reference: std::invalid_argument("wrong model_dtype")
        self.root, self.file_dtype = root, self._FILE[model_dtype]

    def __call__(self, name: str, shape, dtype: torch.dtype) -> torch.Tensor:
        path = self.root + name + ".bin"
        if dtype in (torch.float16, torch.bfloat16):
            return read_bin(path, shape, self.file_dtype).to(dtype)
        return read_bin(path, shape, dtype)


def _source(src) -> Callable[[str, tuple, torch.dtype], torch.Tensor]:
    """`src` is a directory of .bin files, a BinFiles object or a mapping name -> tensor (a state dict)."""
    if isinstance(src, BinFiles):
        return src
    if isinstance(src, Mapping):
        def get(name, shape, dtype):
            if name not in src:
                raise KeyError(f"Cannot find a tensor of name {name}")
            t = src[name]
            if tuple(t.shape) != tuple(shape) and t.numel() == int(np.prod(shape)):
                t = t.reshape(shape)
            if tuple(t.shape) != tuple(shape) or t.dtype != dtype:
                raise ValueError(f"{name}: got {tuple(t.shape)} {t.dtype}, expected {tuple(shape)} {dtype}")
            return t
        return get
    return lambda name, shape, dtype: read_bin(os.path.join(src, name + ".bin"), shape, dtype)


@dataclass
class Int8Linear:
    """SmoothQuant W8A8 linear with the reference's calibrated static activation scale
    (BasicTransformerInt8Block.cc:427-452: invokeSqInputQuant -> runGemmInt8 -> bias)."""
    weight_rows32: torch.Tensor      # int8 [N, K], rows32
    weight_scale: torch.Tensor       # fp32 [N]
    input_quant_scale: torch.Tensor  # fp32 [1]
    pre_quant_scale: torch.Tensor    # fp32 [K]
    bias: Optional[torch.Tensor] = None

    def forward(self, x: torch.Tensor, dynamic: bool = False) -> torch.Tensor:
        k = x.shape[-1]
        x2 = x.reshape(-1, k)
        if dynamic:  # per-token scales computed on the fly instead of the calibrated one
            q, s = ops.sq_quant_dynamic(x2, self.pre_quant_scale)
        else:
            q, s = ops.sq_quant(x2, self.pre_quant_scale, self.input_quant_scale), self.input_quant_scale
        y = ops.int8_linear(q, self.weight_rows32, self.weight_scale, s, self.bias, x.dtype)
        return y.reshape(*x.shape[:-1], y.shape[-1])


@dataclass
class FP8Linear:
    """FP8 e4m3 per-tensor linear (FluxAttnPostFP8Processor.cc:135-163: scale-cast with `_input_scale`, then
    GemmWithResidualAndBias)."""
    weight_rows32: torch.Tensor  # uint8 e4m3 [N, K], rows32
    weight_scale: torch.Tensor   # fp32 [1]
    input_scale: torch.Tensor    # fp32 [1]
    bias: Optional[torch.Tensor] = None
    weight_h: Optional[torch.Tensor] = None  # host master copy of the 16-bit weight [N, K], kept for LoRA merges

    def _requantise(self, w16: torch.Tensor) -> None:
        self.weight_scale.zero_()
        ops.fp8_amax_scale(w16, self.weight_scale)
        ops.repack_weight(ops.fp8_scale_cast(w16, self.weight_scale), out=self.weight_rows32)

    def load_lora(self, lora_weight: torch.Tensor, lora_scale: float) -> None:
        """FP8LoraWeight::load_lora (interface/IFLoraWeight.h:100-112): master copy + lora_scale * delta in the
        weight's dtype, new per-tensor scale, new codes; the codes tensor and the scale are updated in place."""
        if self.weight_h is None:
            raise RuntimeError("this linear was loaded without its 16-bit master copy (keep_master=False)")
        w16 = self.weight_h.to(self.weight_rows32.device)
        ops.load_lora(w16, lora_weight.to(device=w16.device, dtype=w16.dtype).reshape(w16.shape).contiguous(), lora_scale)
        self._requantise(w16)

    def clear_lora(self) -> None:
        """FP8LoraWeight::clear_lora (IFLoraWeight.h:114-127): re-quantise the untouched master copy."""
        if self.weight_h is None:
            raise RuntimeError("this linear was loaded without its 16-bit master copy (keep_master=False)")
        self._requantise(self.weight_h.to(self.weight_rows32.device))

    def forward(self, x: torch.Tensor, gelu: bool = False, residual=None, beta: float = 0.0, dynamic: bool = False) -> torch.Tensor:
        k = x.shape[-1]
        x2 = x.reshape(-1, k)
        if not gelu and residual is None and k % 64 == 0 and x2.numel() < 2 ** 32:
            # scales and bias only: the codes travel as k-panels, which the GEMM fetches in whole cache lines (same bits)
            q, s = ops.fp8_quant_panels(x2) if dynamic else (ops.fp8_scale_cast_panels(x2, self.input_scale), self.input_scale)
            y = ops.fp8_linear_panels(q, self.weight_rows32, s, self.weight_scale, self.bias, None, x.dtype)
            return y.reshape(*x.shape[:-1], y.shape[-1])
        if dynamic:
            q, s = ops.fp8_quant(x2)
        else:
            q, s = ops.fp8_scale_cast(x2, self.input_scale), self.input_scale
        y = ops.fp8_linear(q, self.weight_rows32, s, self.weight_scale, self.bias, gelu, residual, beta, x.dtype)
        return y.reshape(*x.shape[:-1], y.shape[-1])


@dataclass
class W4A4Linear:
    """W4A4 group-64 linear with the SVDQuant low-rank branch (W4A4Gemm.cc:113-169)."""
    weight_rows32: torch.Tensor  # uint8 [N, K/2], rows32
    weight_scale: torch.Tensor   # fp32 [N, K/64]
    smooth: torch.Tensor         # fp32 [K]
    lora_up: Optional[torch.Tensor] = None    # T [N, R]
    lora_down: Optional[torch.Tensor] = None  # T [R, K]
    bias: Optional[torch.Tensor] = None

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        k = x.shape[-1]
        x2 = x.reshape(-1, k)
        if self.lora_down is not None:
            q, s, act = ops.w4a4_quant_lora_down(x2, self.smooth, self.lora_down, torch.float32)
        else:
            (q, s), act = ops.w4a4_quant(x2, self.smooth, torch.float32), None
        y = ops.w4a4_linear(q, self.weight_rows32, s, self.weight_scale, self.bias, x.dtype, 64, act,
                            self.lora_up if act is not None else None)
        return y.reshape(*x.shape[:-1], y.shape[-1])


def load_int8_linear(src, prefix: str, name: str, d_out: int, d_in: int, device="cuda", bias_dtype=None) -> Int8Linear:
    get = _source(src)
    w = get(prefix + name + ".weight_int8", (d_out, d_in), torch.int8).to(device)
    bias = None
    if bias_dtype is not None:
        bias = get(prefix + name + ".bias", (d_out,), bias_dtype).to(device)
    return Int8Linear(ops.repack_weight(w),
                      get(prefix + name + ".weight_quant_scale", (d_out,), torch.float32).to(device),
                      get(prefix + name + ".input_quant_scale", (1,), torch.float32).to(device),
                      get(prefix + name + ".pre_quant_scale", (d_in,), torch.float32).to(device), bias)


def load_fp8_linear(src, prefix: str, name: str, d_out: int, d_in: int, dtype=torch.bfloat16, device="cuda",
                    keep_master: bool = False) -> FP8Linear:
    """The 16-bit weight is quantised on the device as the reference does at load time: scale = max|w|/448
    (invokeGetFP8WeightScale), codes = e4m3(w * (1/scale)) (invokeCudaD2DScaleCpyConvert).  keep_master keeps the
    16-bit weight on the host (the reference's `*_weight_h`) so that LoRA deltas can be merged and removed later."""
    get = _source(src)
    w_host = get(prefix + name + ".weight", (d_out, d_in), dtype)
    w = w_host.to(device)
    scale = ops.fp8_amax_scale(w)
    codes = ops.fp8_scale_cast(w, scale)
    return FP8Linear(ops.repack_weight(codes), scale,
                     get(prefix + name + "_input_scale", (1,), torch.float32).to(device),
                     get(prefix + name + ".bias", (d_out,), dtype).to(device),
                     w_host.detach().cpu().clone() if keep_master else None)


def load_w4a4_linear(src, prefix: str, d_out: int, d_in: int, lora_rank: int = 32, has_bias: bool = False,
                     dtype=torch.bfloat16, device="cuda") -> W4A4Linear:
    get = _source(src)
    packed = get(prefix + "packed_weight", (d_out, d_in // 2), torch.int8).to(device)
    lin = W4A4Linear(ops.repack_weight(packed.view(torch.uint8)),
                     get(prefix + "weight_scale", (d_out, d_in // 64), torch.float32).to(device),
                     get(prefix + "smooth", (d_in,), torch.float32).to(device))
    if lora_rank:
        lin.lora_up = get(prefix + "lora_up", (d_out, lora_rank), dtype).to(device)
        lin.lora_down = get(prefix + "lora_down", (lora_rank, d_in), dtype).to(device)
    if has_bias:
        lin.bias = get(prefix + "bias", (d_out,), dtype).to(device)
    return lin


# ---- int4 <-> int8 host helpers of the weight tooling (offline, CPU tensors, as in the reference) ------------------
def pack_int8_tensor_to_packed_int4(weight: torch.Tensor) -> torch.Tensor:
    """int8 values in [-8, 7] -> two per byte along the last dim, element 2j in the low nibble
    (pack_int8_tensor_to_packed_int4, src/lyradiff/layers/gemm_utils/WeightOnlyQuantOps.cc:286-321)."""
    if weight.is_cuda or weight.dtype != torch.int8 or not weight.is_contiguous() or weight.numel() == 0:
        raise ValueError("weight must be a non-empty contiguous CPU int8 tensor")
    if weight.shape[-1] % 2:
        raise ValueError("the last dimension must be even")
    if int(weight.min()) < -8 or int(weight.max()) > 7:
        raise ValueError("Value in unpacked tensor not in int4 range")
    w = weight.to(torch.int16)
    return ((w[..., 0::2] & 0xF) | ((w[..., 1::2] & 0xF) << 4)).to(torch.uint8).view(torch.int8).contiguous()


def unpack_int4_packed_tensor_to_int8(weight: torch.Tensor) -> torch.Tensor:
    """Inverse, sign-extending (unpack_int4_packed_tensor_to_int8, WeightOnlyQuantOps.cc:256-284)."""
    if weight.is_cuda or weight.dtype != torch.int8 or not weight.is_contiguous() or weight.numel() == 0:
        raise ValueError("weight must be a non-empty contiguous CPU int8 packed tensor")
    b = weight.view(torch.uint8).to(torch.int16)
    lo, hi = b & 0xF, b >> 4
    lo, hi = torch.where(lo > 7, lo - 16, lo), torch.where(hi > 7, hi - 16, hi)
    return torch.stack((lo, hi), dim=-1).reshape(*weight.shape[:-1], weight.shape[-1] * 2).to(torch.int8)


def symmetric_quantize_last_axis_of_batched_matrix(weight: torch.Tensor, bits: int = 8):
    """Per-column symmetric weight-only quantisation of a CPU [K, N] (or [E, K, N]) fp16/bf16/fp32 weight
    (symmetric_quantize, src/lyradiff/kernels/cutlass_kernels/cutlass_preprocessors.cpp:532-631, exposed as
    lyrallms::symmetric_quantize_last_axis_of_batched_matrix, WeightOnlyQuantOps.cc:120-215): scale = max|w| / 2^(bits-1)
    per column, q = clip(round-half-away(w / scale)).  Returns (unprocessed codes int8 -- int4 packed two per byte
    along N, low nibble first --, scales in the weight's dtype); prepare the codes for the GEMM with
    ops.repack_weight_only on the device."""
    if weight.is_cuda or weight.dim() not in (2, 3) or bits not in (4, 8):
        raise ValueError("weight must be a CPU tensor of 2 or 3 dimensions, bits 4 or 8")
    w = weight.float()
    half = float(1 << (bits - 1))
    col = w.abs().amax(dim=-2) * (1.0 / half)
    r = w / col.unsqueeze(-2)
    r = torch.sign(r) * torch.floor(r.abs() + 0.5)
    q = torch.nan_to_num(r, nan=0.0).clamp(-half, half - 1).to(torch.int8)
    if bits == 4:
        q = pack_int8_tensor_to_packed_int4(q.contiguous())
    return q.contiguous(), col.to(weight.dtype)
