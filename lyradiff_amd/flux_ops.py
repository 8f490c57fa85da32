"""Block-level FLUX ops with the interface of the reference's torch custom classes.

`FluxTransformerBlockOp` / `FluxSingleTransformerBlockOp` mirror the classes the reference registers in
src/lyradiff/th_op/pybind.cc:66-96 (constructor arguments, initialize, forward, reload_model_from_state_dict,
load_lora_by_name, clear_lora: th_op/flux_transformer_block/FluxTransformerBlockOp.cc:6-107 and
th_op/flux_single_transformer_block/FluxSingleTransformerBlockOp.cc:6-98), so that the reference's Python wrappers
(lyradiff/lyradiff_model/lyradiff_flux_transformer_model_v2.py:67-168) can hold one of these instead of a
`torch.classes.lyradiff.*` object.  Every quantized linear, every adaLN / gate / residual step and every activation
quantisation runs on this library's HIP kernels (flux_fp8.py), as do the per-head RMSNorm of q and k and the rotary
embedding behind the QKV projection (lq_rmsnorm_rope); the softmax attention itself is not part of the quantized-linear
path and is PyTorch's (`flux_attention_core`).

Supported quant levels: FP8_W8A8, FP8_W8A8_FULL, INT4_W4A4 and INT4_W4A4_FULL (W4A4 linears with their low-rank branch,
th_op/flux_transformer_block/FluxTransformerBlockOp.h:165-182).  Any other level raises at construction.
"""
from __future__ import annotations

from enum import Enum
from typing import Mapping, Optional, Sequence

import torch

from . import flux_fp8 as F
from . import flux_int4 as I4
from . import ops
from . import weights as W


class LyraQuantLevel(Enum):
    """lyradiff/lyradiff_model/lyradiff_utils.py:4-13."""
    NONE = 0
    FP8_W8A8 = 1
    FP8_W8A8_FULL = 2
    FP8_WEIGHT_ONLY = 3
    INT8_SMOOTH_QUANT_LEVEL1 = 4
    INT8_SMOOTH_QUANT_LEVEL2 = 5
    INT8_SMOOTH_QUANT_LEVEL3 = 6
    INT4_W4A4 = 7
    INT4_W4A4_FULL = 8


_DTYPES = {"fp16": torch.float16, "bf16": torch.bfloat16}


def flux_attention_core(qkv: torch.Tensor, norm_q: torch.Tensor, norm_k: torch.Tensor, rope_emb: torch.Tensor, heads: int,
                        context_qkv: Optional[torch.Tensor] = None, norm_added_q: Optional[torch.Tensor] = None,
                        norm_added_k: Optional[torch.Tensor] = None):
    """The part of FluxAttentionFP8Processor::forward (FluxAttentionFP8Processor.cc:232-291) and
    FluxSingleAttentionFP8Processor::forward (FluxSingleAttentionFP8Processor.cc:183-213) between the QKV and the output
    projections: q/k RMSNorm per head, rotary embedding and the [text, image] concatenation in one HIP kernel
    (ops.rmsnorm_rope = invokeFusedRmsNormCatAndRope), then softmax attention (PyTorch) on its [B, S, 3, H, Dh] output.
    With `context_qkv` (image [B, S, D], text [B, Sc, D]) is returned; without it a single [B, S, D] tensor."""
    b, s, d3 = qkv.shape
    d = d3 // 3
    sc = 0 if context_qkv is None else context_qkv.shape[1]
    added = None if context_qkv is None else torch.cat([norm_added_q, norm_added_k])
    cat = ops.rmsnorm_rope(qkv.contiguous(), torch.cat([norm_q, norm_k]), rope_emb.contiguous(), heads,
                           None if context_qkv is None else context_qkv.contiguous(), added)
    q, k, v = (cat[:, :, i].transpose(1, 2) for i in range(3))  # [B, H, Sc + S, Dh] views
    o = torch.nn.functional.scaled_dot_product_attention(q, k, v)
    o = o.transpose(1, 2).reshape(b, sc + s, d)
    if context_qkv is None:
        return o
    return o[:, sc:], o[:, :sc]


class _BlockOpBase:
    def __init__(self, inference_dtype: str, embedding_dim: int, embedding_head_num: int, embedding_head_dim: int,
                 mlp_scale: int, quant_level: int):
        if inference_dtype not in _DTYPES:
            raise ValueError("wrong inference_dtype")  # the reference throws on anything but fp32 / fp16 / bf16
        level = LyraQuantLevel(int(quant_level))
        if level not in (LyraQuantLevel.FP8_W8A8, LyraQuantLevel.FP8_W8A8_FULL, LyraQuantLevel.INT4_W4A4,
                         LyraQuantLevel.INT4_W4A4_FULL):
            raise NotImplementedError(f"quant level {level.name}: only the FP8 and INT4 blocks are built on this library")
        self.int4 = level in (LyraQuantLevel.INT4_W4A4, LyraQuantLevel.INT4_W4A4_FULL)
        if embedding_dim != embedding_head_num * embedding_head_dim:
            raise ValueError("embedding_dim must equal embedding_head_num * embedding_head_dim")
        self.inference_dtype = inference_dtype
        self.dtype = _DTYPES[inference_dtype]
        self.dim, self.heads, self.head_dim, self.mlp_scale = embedding_dim, embedding_head_num, embedding_head_dim, mlp_scale
        self.quant_level = level
        self.weights = None
        self.device = "cuda"

    def initialize(self, lyradiff_context=None) -> None:
        """The reference creates its stream, cuBLAS wrapper and allocator here; nothing of the kind is needed."""

    def _check(self, name: str, t: torch.Tensor) -> None:  # CHECK_TH_CUDA, CHECK_CONTIGUOUS, dtype TORCH_CHECK
        if not t.is_cuda:
            raise RuntimeError(f"{name} must be a CUDA tensor")
        if not t.is_contiguous():
            raise RuntimeError(f"{name} must be contiguous")
        if t.dtype != self.dtype:
            raise RuntimeError(f"{name} dtype should be {self.dtype}")

    def _loaded(self):
        if self.weights is None:
            raise RuntimeError("reload_model_from_state_dict has not been called")
        return self.weights

    def _fp8_linears(self):
        raise NotImplementedError

    def load_lora_by_name(self, lora_name: Sequence[str], lora_weights: torch.Tensor, lora_strength: float) -> None:
        """Merges `lora_strength * lora_weights` into the named linear's 16-bit master copy and re-quantises it
        (FP8LoraWeight::load_lora, IFLoraWeight.h:79-128).  `lora_name` is the path the reference walks through its
        lora_layer_map / lora_weight_map (IFLoraWeight.h:146-168): ["attn", "to_qkv"], ["attn", "to_out.0"],
        ["ff", "net.0.proj"], ["norm1", "linear"], ["proj_mlp"], ...  An unknown name raises (the reference prints a
        message and goes on)."""
        key = ".".join(lora_name)
        if self.int4:  # the reference's INT4 block weights register no LoRA targets (FluxTransformerInt4BlockWeight.cc:41-45)
            raise KeyError(f"no LoRA target named {key}: the INT4 blocks carry their low-rank branch in the checkpoint")
        lin = self._fp8_linears().get(key)
        if lin is None or not isinstance(lin, W.FP8Linear):
            raise KeyError(f"no FP8 linear named {key} in this block")
        lin.load_lora(lora_weights.to(self.device), float(lora_strength))

    def clear_lora(self) -> None:
        self._loaded()
        if not self.int4:
            for lin in self._fp8_linears().values():
                if isinstance(lin, W.FP8Linear):
                    lin.clear_lora()


class FluxTransformerBlockOp(_BlockOpBase):
    """Double-stream FLUX block (FluxTransformerFP8Block.cc:159-262)."""

    def reload_model_from_state_dict(self, prefix: str, weights: Mapping[str, torch.Tensor], device: str = "cpu") -> None:
        """Keys as FluxTransformerFP8BlockWeight::loadWeightsFromCache / FluxAttentionFP8ProcessorWeight::loadWeightsFromCache
        read them (FluxAttentionFP8ProcessorWeight.cc:194-260): the linears' `.weight`, `.bias`, `_input_scale`, and
        `attn.norm_q.weight`, `attn.norm_k.weight`, `attn.norm_added_q.weight`, `attn.norm_added_k.weight`.  `device` names
        where the tensors of `weights` live, as in the reference; they end up on the GPU either way."""
        self._load(prefix, weights)

    def reload_model_from_bin(self, model_path: str, model_dtype: str) -> None:
        """FluxTransformerBlockOp::reload_model_from_bin (th_op/flux_transformer_block/FluxTransformerBlockOp.h:239-258):
        `model_path` is the prefix of the block's raw .bin files (model_path + "attn.to_qkv.weight.bin", ...), with the
        same tensor names as the state dict; `model_dtype` is the element type the 16-bit tensors were written in."""
        self._load(model_path, W.BinFiles("", model_dtype))

    def _load(self, prefix: str, src) -> None:
        if self.int4:
            self.weights = I4.load_flux_double_block_int4(src, prefix, self.dim, self.quant_level is LyraQuantLevel.INT4_W4A4_FULL,
                                                          self.dtype, self.device)
        else:
            self.weights = F.load_flux_double_block_fp8(src, prefix, self.dim, self.dtype, self.device, keep_master=True,
                                                        full=self.quant_level is LyraQuantLevel.FP8_W8A8_FULL)
        get = W._source(src)
        self.norms = [get(prefix + f"attn.{n}.weight", (self.head_dim,), self.dtype).to(self.device)
                      for n in ("norm_q", "norm_k", "norm_added_q", "norm_added_k")]

    def _fp8_linears(self):
        w = self._loaded()
        return {"norm1.linear": w.norm1, "norm1_context.linear": w.norm1_context, "attn.to_qkv": w.to_qkv,
                "attn.to_added_qkv": w.to_added_qkv, "attn.to_out.0": w.to_out, "attn.to_add_out": w.to_add_out,
                "ff.net.0.proj": w.ff.gelu_proj, "ff.net.2": w.ff.ff_linear,
                "ff_context.net.0.proj": w.ff_context.gelu_proj, "ff_context.net.2": w.ff_context.ff_linear}

    def forward(self, hidden_states: torch.Tensor, encoder_hidden_states: torch.Tensor, rope_emb: torch.Tensor,
                temb_emb: torch.Tensor):
        """Returns [hidden_states_out, encoder_hidden_states_out] (FluxTransformerBlockOp.h:186-235)."""
        w = self._loaded()
        for n, t in (("hidden_states", hidden_states), ("encoder_hidden_states", encoder_hidden_states),
                     ("rope_emb", rope_emb), ("temb_emb", temb_emb)):
            self._check(n, t)
        nq, nk, naq, nak = self.norms
        core = lambda qkv, cqkv: flux_attention_core(qkv, nq, nk, rope_emb, self.heads, cqkv, naq, nak)
        block = I4.flux_double_block_int4 if self.int4 else F.flux_double_block_fp8
        out, ctx = block(hidden_states, encoder_hidden_states, temb_emb, w, core)
        return [out, ctx]


class FluxSingleTransformerBlockOp(_BlockOpBase):
    """Single-stream FLUX block (FluxSingleTransformerFP8Block.cc:163-291)."""

    def reload_model_from_state_dict(self, prefix: str, weights: Mapping[str, torch.Tensor], device: str = "cpu") -> None:
        self._load(prefix, weights)

    def reload_model_from_bin(self, model_path: str, model_dtype: str) -> None:
        """FluxSingleTransformerBlockOp::reload_model_from_bin: raw .bin files named model_path + tensor name + ".bin"."""
        self._load(model_path, W.BinFiles("", model_dtype))

    def _load(self, prefix: str, src) -> None:
        if self.int4:
            self.weights = I4.load_flux_single_block_int4(src, prefix, self.dim, self.mlp_scale,
                                                          self.quant_level is LyraQuantLevel.INT4_W4A4_FULL, self.dtype, self.device)
        else:
            self.weights = F.load_flux_single_block_fp8(src, prefix, self.dim, self.mlp_scale, self.dtype, self.device,
                                                        keep_master=True, full=self.quant_level is LyraQuantLevel.FP8_W8A8_FULL)
        get = W._source(src)
        self.norms = [get(prefix + f"attn.{n}.weight", (self.head_dim,), self.dtype).to(self.device) for n in ("norm_q", "norm_k")]

    def _fp8_linears(self):
        w = self._loaded()
        return {"norm.linear": w.norm, "attn.to_qkv": w.to_qkv, "proj_mlp": w.mlp.proj_mlp, "proj_out": w.mlp.proj_out}

    def forward(self, hidden_states: torch.Tensor, rope_emb: torch.Tensor, temb_emb: torch.Tensor) -> torch.Tensor:
        w = self._loaded()
        for n, t in (("hidden_states", hidden_states), ("rope_emb", rope_emb), ("temb_emb", temb_emb)):
            self._check(n, t)
        nq, nk = self.norms
        block = I4.flux_single_block_int4 if self.int4 else F.flux_single_block_fp8
        return block(hidden_states, temb_emb, w, lambda qkv: flux_attention_core(qkv, nq, nk, rope_emb, self.heads))
