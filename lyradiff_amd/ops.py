"""Tensor-level Python wrapper over the C ABI (PyTorch-ROCm supplies device memory and streams).

Checks follow the reference's torch binding conventions (CHECK_TH_CUDA / CHECK_CONTIGUOUS /
dtype TORCH_CHECK, src/lyradiff/th_op/th_utils.h:14-33): inputs must be contiguous device
tensors of the stated dtype; outputs are allocated with torch.empty on the input's device;
work is enqueued on the current stream.  lyradiff_amd/torch_ops.py registers the same functions as
torch.ops.lyradiff.* custom operators.
"""
from __future__ import annotations

import ctypes as C

import torch

from . import lib as _l

_DT = {torch.float32: _l.LQ_F32, torch.float16: _l.LQ_F16, torch.bfloat16: _l.LQ_BF16, torch.int32: _l.LQ_I32}


def _chk(t: torch.Tensor, name: str, dtypes=None) -> torch.Tensor:
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor")
    if not t.is_cuda:
        raise ValueError(f"{name} must be a CUDA(HIP) tensor")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    if dtypes is not None and t.dtype not in dtypes:
        raise TypeError(f"{name} has dtype {t.dtype}, expected one of {dtypes}")
    return t


def _ptr(t):
    return None if t is None else t.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream():
    """Handle of the current HIP stream of the current device.  The private accessors skip the Stream object and the
    device-index normalisation of torch.cuda.current_stream() (2.8 -> 0.4 us per call); without them the public path is used."""
    if _raw_stream is not None and _raw_device is not None:
        return _raw_stream(_raw_device())
    return torch.cuda.current_stream().cuda_stream


_FLOATS = (torch.float32, torch.float16, torch.bfloat16)


# ---- INT8 SmoothQuant ---------------------------------------------------------------------------

def col_absmax(x, out=None):
    """Per-column max |x| over all rows, accumulated into `out` (fp32 [K]; allocated and zeroed when None)."""
    _chk(x, "x", _FLOATS)
    k = x.shape[-1]
    if out is None:
        out = torch.zeros(k, dtype=torch.float32, device=x.device)
    _chk(out, "out", (torch.float32,))
    _l.check(_l.load().lq_col_absmax(_ptr(out), _ptr(x), _DT[x.dtype], x.numel() // k if k else 0, k, _stream()), "lq_col_absmax")
    return out


def smooth_vector(act_absmax, weight_absmax, alpha: float = 0.5):
    """SmoothQuant s[k] = act^alpha / weight^(1-alpha); returns (pre_quant_scale = 1/s, s)."""
    _chk(act_absmax, "act_absmax", (torch.float32,))
    _chk(weight_absmax, "weight_absmax", (torch.float32,))
    k = act_absmax.numel()
    if weight_absmax.numel() != k:
        raise ValueError("act_absmax and weight_absmax must have the same length")
    pre, s = torch.empty_like(act_absmax), torch.empty_like(act_absmax)
    _l.check(_l.load().lq_smooth_vector(_ptr(pre), _ptr(s), _ptr(act_absmax), _ptr(weight_absmax), float(alpha), k, _stream()),
             "lq_smooth_vector")
    return pre, s


def sq_quant(x, pre_quant_scale, input_quant_scale, per_token: bool = False):
    """invokeSqInputQuant: x [..., K] -> int8 [..., K] with a static (or given per-token) scale."""
    _chk(x, "x", _FLOATS)
    _chk(input_quant_scale, "input_quant_scale", (torch.float32,))
    if pre_quant_scale is not None:
        _chk(pre_quant_scale, "pre_quant_scale", (torch.float32,))
        if pre_quant_scale.numel() != x.shape[-1]:
            raise ValueError("pre_quant_scale must have K elements")
    k = x.shape[-1]
    rows = x.numel() // k if k else 0
    if per_token and input_quant_scale.numel() != rows:
        raise ValueError("per-token input_quant_scale must have one element per row")
    q = torch.empty(x.shape, dtype=torch.int8, device=x.device)
    _l.check(_l.load().lq_sq_input_quant(_ptr(q), _ptr(x), _DT[x.dtype], _ptr(pre_quant_scale),
                                         _ptr(input_quant_scale), int(per_token), rows, k, _stream()),
             "lq_sq_input_quant")
    return q


def sq_quant_dynamic(x, pre_quant_scale=None):
    """Dynamic per-token SmoothQuant: returns (q int8 [..., K], scale fp32 [rows])."""
    _chk(x, "x", _FLOATS)
    if pre_quant_scale is not None:
        _chk(pre_quant_scale, "pre_quant_scale", (torch.float32,))
        if pre_quant_scale.numel() != x.shape[-1]:
            raise ValueError("pre_quant_scale must have K elements")
    k = x.shape[-1]
    rows = x.numel() // k if k else 0
    q = torch.empty(x.shape, dtype=torch.int8, device=x.device)
    s = torch.empty(rows, dtype=torch.float32, device=x.device)
    _l.check(_l.load().lq_sq_dynamic_quant(_ptr(q), _ptr(s), _ptr(x), _DT[x.dtype], _ptr(pre_quant_scale),
                                           rows, k, _stream()), "lq_sq_dynamic_quant")
    return q, s


def sq_dequant(acc, input_quant_scale, weight_quant_scale, per_token: bool = False, out_dtype=torch.float16):
    """invokeSqOutputDequant: int32 [M,N] -> T [M,N]."""
    _chk(acc, "acc", (torch.int32,))
    _chk(input_quant_scale, "input_quant_scale", (torch.float32,))
    _chk(weight_quant_scale, "weight_quant_scale", (torch.float32,))
    n = acc.shape[-1]
    rows = acc.numel() // n if n else 0
    if weight_quant_scale.numel() != n:
        raise ValueError("weight_quant_scale must have N elements")
    if input_quant_scale.numel() < (rows if per_token else 1):
        raise ValueError("input_quant_scale must have one element per row when per_token, at least one otherwise")
    if out_dtype not in _FLOATS:
        raise TypeError("out_dtype must be float16, bfloat16 or float32")
    y = torch.empty(acc.shape, dtype=out_dtype, device=acc.device)
    _l.check(_l.load().lq_sq_output_dequant(_ptr(y), _DT[out_dtype], _ptr(acc), _ptr(input_quant_scale),
                                            _ptr(weight_quant_scale), int(per_token), rows, n, _stream()),
             "lq_sq_output_dequant")
    return y


def int8_weight_quant(w, pre_quant_scale=None):
    """invokeGetINT8WeightScale: w [N,K] -> (q int8 [N,K] row-major, scale fp32 [N])."""
    _chk(w, "w", _FLOATS)
    if pre_quant_scale is not None:
        _chk(pre_quant_scale, "pre_quant_scale", (torch.float32,))
    if w.dim() != 2:
        raise ValueError("w must be a matrix [N, K]")
    n, k = w.shape
    if pre_quant_scale is not None and pre_quant_scale.numel() != k:
        raise ValueError("pre_quant_scale must have K elements")
    q = torch.empty((n, k), dtype=torch.int8, device=w.device)
    s = torch.empty(n, dtype=torch.float32, device=w.device)
    _l.check(_l.load().lq_int8_weight_quant(_ptr(s), _ptr(q), _ptr(w), _DT[w.dtype], _ptr(pre_quant_scale), n, k,
                                            _stream()), "lq_int8_weight_quant")
    return q, s


def geglu_int8(hidden, bias, pre_quant_scale, input_quant_scale):
    """invokeFusedAddBiasGegluInt8O: hidden [..., 2D] -> int8 [..., D], static scale."""
    _chk(hidden, "hidden", _FLOATS)
    _chk(input_quant_scale, "input_quant_scale", (torch.float32,))
    if bias is not None:
        _chk(bias, "bias", (hidden.dtype,))
    if pre_quant_scale is not None:
        _chk(pre_quant_scale, "pre_quant_scale", (torch.float32,))
    d = hidden.shape[-1] // 2
    rows = hidden.numel() // (2 * d) if d else 0
    q = torch.empty(hidden.shape[:-1] + (d,), dtype=torch.int8, device=hidden.device)
    _l.check(_l.load().lq_geglu_int8(_ptr(q), _ptr(hidden), _ptr(bias), _DT[hidden.dtype], _ptr(pre_quant_scale),
                                     _ptr(input_quant_scale), rows, d, _stream()), "lq_geglu_int8")
    return q


def geglu_int8_dynamic(hidden, bias=None, pre_quant_scale=None):
    _chk(hidden, "hidden", _FLOATS)
    if bias is not None:
        _chk(bias, "bias", (hidden.dtype,))
    if pre_quant_scale is not None:
        _chk(pre_quant_scale, "pre_quant_scale", (torch.float32,))
    d = hidden.shape[-1] // 2
    rows = hidden.numel() // (2 * d) if d else 0
    q = torch.empty(hidden.shape[:-1] + (d,), dtype=torch.int8, device=hidden.device)
    s = torch.empty(rows, dtype=torch.float32, device=hidden.device)
    _l.check(_l.load().lq_geglu_int8_dynamic(_ptr(q), _ptr(s), _ptr(hidden), _ptr(bias), _DT[hidden.dtype],
                                             _ptr(pre_quant_scale), rows, d, _stream()), "lq_geglu_int8_dynamic")
    return q, s


def layernorm_int8(x, gamma, beta, pre_quant_scale=None, input_quant_scale=None, residual=None, bias=None, eps: float = 1e-6):
    """invokeLayerNormInt8O / invokeFusedResidualBiasLayerNormInt8O: LayerNorm over the last dim fused with the
    INT8 quantisation.  input_quant_scale given: static scale, returns (q, None, h); None: dynamic per-token
    scale, returns (q, scale[rows], h).  h = x + residual (+ bias) in x's dtype, or None without a residual."""
    _chk(x, "x", (torch.float16, torch.bfloat16))
    _chk(gamma, "gamma", (x.dtype,))
    _chk(beta, "beta", (x.dtype,))
    for name, t in (("residual", residual), ("bias", bias)):
        if t is not None:
            _chk(t, name, (x.dtype,))
    if pre_quant_scale is not None:
        _chk(pre_quant_scale, "pre_quant_scale", (torch.float32,))
    if input_quant_scale is not None:
        _chk(input_quant_scale, "input_quant_scale", (torch.float32,))
    dim = x.shape[-1]
    rows = x.numel() // dim if dim else 0
    q = torch.empty(x.shape, dtype=torch.int8, device=x.device)
    s = torch.empty(rows, dtype=torch.float32, device=x.device) if input_quant_scale is None else None
    h = torch.empty_like(x) if residual is not None else None
    _l.check(_l.load().lq_layernorm_int8(_ptr(q), _ptr(s), _ptr(h), _ptr(x), _ptr(residual), _ptr(bias), _ptr(gamma), _ptr(beta),
                                         _DT[x.dtype], _ptr(pre_quant_scale), _ptr(input_quant_scale), rows, dim, float(eps),
                                         _stream()), "lq_layernorm_int8")
    return q, s, h


def _codes_like(x, panels: bool):
    """Destination of the e4m3 codes of x [B, S, D]: the same shape, or k-panels [D/64, B*S, 64] (see fp8_quant_panels)."""
    if not panels:
        return torch.empty(x.shape, dtype=torch.uint8, device=x.device)
    if x.shape[-1] % 64 != 0:
        raise ValueError("codes in k-panels need a last dimension that is a multiple of 64")
    return torch.empty((x.shape[-1] // 64, x.numel() // x.shape[-1], 64), dtype=torch.uint8, device=x.device)


def layernorm_mod_fp8(x, scale, shift, input_scale, eps: float = 1e-6, panels: bool = False):
    """invokeLayerNormWithShiftAndScale + FP8 cast: x [B, S, D], scale/shift [B, D], static input_scale [1];
    returns e4m3 codes (uint8) of shape x, or with panels=True as k-panels [D/64, B*S, 64]."""
    _chk(x, "x", (torch.float16, torch.bfloat16))
    _chk(scale, "scale", (x.dtype,))
    _chk(shift, "shift", (x.dtype,))
    _chk(input_scale, "input_scale", (torch.float32,))
    if x.dim() != 3 or tuple(scale.shape) != (x.shape[0], x.shape[2]) or scale.shape != shift.shape:
        raise ValueError("x must be [B,S,D] and scale, shift [B,D]")
    q = _codes_like(x, panels)
    fn = _l.load().lq_layernorm_mod_fp8_panels if panels else _l.load().lq_layernorm_mod_fp8
    _l.check(fn(_ptr(q), _ptr(x), _ptr(scale), _ptr(shift), _DT[x.dtype], _ptr(input_scale),
                x.shape[0], x.shape[1], x.shape[2], float(eps), _stream()), "lq_layernorm_mod_fp8")
    return q


def layernorm_mod_fp8_dual(x, scale, shift, input_scale_a, input_scale_b, eps: float = 1e-6, panels: bool = False):
    """layernorm_mod_fp8 for two consumers of the normalised tensor: returns (codes_a, codes_b)."""
    _chk(x, "x", (torch.float16, torch.bfloat16))
    _chk(scale, "scale", (x.dtype,))
    _chk(shift, "shift", (x.dtype,))
    _chk(input_scale_a, "input_scale_a", (torch.float32,))
    _chk(input_scale_b, "input_scale_b", (torch.float32,))
    if x.dim() != 3 or tuple(scale.shape) != (x.shape[0], x.shape[2]) or scale.shape != shift.shape:
        raise ValueError("x must be [B,S,D] and scale, shift [B,D]")
    qa, qb = _codes_like(x, panels), _codes_like(x, panels)
    fn = _l.load().lq_layernorm_mod_fp8_dual_panels if panels else _l.load().lq_layernorm_mod_fp8_dual
    _l.check(fn(_ptr(qa), _ptr(input_scale_a), _ptr(qb), _ptr(input_scale_b), _ptr(x), _ptr(scale), _ptr(shift), _DT[x.dtype],
                x.shape[0], x.shape[1], x.shape[2], float(eps), _stream()), "lq_layernorm_mod_fp8_dual")
    return qa, qb


def gate_residual_layernorm_mod_fp8(attn, gate, x, scale, shift, input_scale, eps: float = 1e-6, hidden_out=None,
                                    panels: bool = False):
    """invokeFusedGateAndResidual + invokeLayerNormWithShiftAndScale + FP8 cast in one pass:
    hidden = x + gate*attn (each op rounded to the tensor dtype), codes = e4m3(adaLN(hidden) / input_scale).
    attn, x [B,S,D]; gate, scale, shift [B,D].  Returns (codes, hidden); hidden_out may be x itself."""
    _chk(x, "x", (torch.float16, torch.bfloat16))
    for name, t in (("attn", attn), ("gate", gate), ("scale", scale), ("shift", shift)):
        _chk(t, name, (x.dtype,))
    _chk(input_scale, "input_scale", (torch.float32,))
    if x.dim() != 3 or attn.shape != x.shape or any(tuple(t.shape) != (x.shape[0], x.shape[2]) for t in (gate, scale, shift)):
        raise ValueError("attn, x must be [B,S,D] and gate, scale, shift [B,D]")
    if hidden_out is None:
        hidden_out = torch.empty_like(x)
    _chk(hidden_out, "hidden_out", (x.dtype,))
    q = _codes_like(x, panels)
    fn = _l.load().lq_gate_residual_layernorm_mod_fp8_panels if panels else _l.load().lq_gate_residual_layernorm_mod_fp8
    _l.check(fn(_ptr(q), _ptr(hidden_out), _ptr(attn), _ptr(gate), _ptr(x), _ptr(scale), _ptr(shift), _DT[x.dtype],
                _ptr(input_scale), x.shape[0], x.shape[1], x.shape[2], float(eps), _stream()),
             "lq_gate_residual_layernorm_mod_fp8")
    return q, hidden_out


def gate_residual_layernorm_mod(x, scale, shift, attn=None, gate=None, eps: float = 1e-6, hidden_out=None):
    """adaLN (1+scale)*LN(h)+shift as a 16-bit tensor, h = x or, with attn and gate, x + gate*attn (also returned).
    x, attn [B,S,D]; gate, scale, shift [B,D].  Returns norm, or (norm, hidden) when gated."""
    _chk(x, "x", (torch.float16, torch.bfloat16))
    _chk(scale, "scale", (x.dtype,))
    _chk(shift, "shift", (x.dtype,))
    if x.dim() != 3 or tuple(scale.shape) != (x.shape[0], x.shape[2]) or scale.shape != shift.shape:
        raise ValueError("x must be [B,S,D] and scale, shift [B,D]")
    if (attn is None) != (gate is None):
        raise ValueError("attn and gate go together")
    out = torch.empty_like(x)
    if attn is not None:
        _chk(attn, "attn", (x.dtype,))
        _chk(gate, "gate", (x.dtype,))
        if attn.shape != x.shape or gate.shape != scale.shape:
            raise ValueError("attn must be [B,S,D] and gate [B,D]")
        if hidden_out is None:
            hidden_out = torch.empty_like(x)
        _chk(hidden_out, "hidden_out", (x.dtype,))
    _l.check(_l.load().lq_gate_residual_layernorm_mod(_ptr(out), _ptr(hidden_out) if attn is not None else None, _ptr(attn),
                                                      _ptr(gate), _ptr(x), _ptr(scale), _ptr(shift), _DT[x.dtype], x.shape[0],
                                                      x.shape[1], x.shape[2], float(eps), _stream()),
             "lq_gate_residual_layernorm_mod")
    return (out, hidden_out) if attn is not None else out


# ---- FP8 -------------------------------------------------------------------------------------------

def fp8_amax_scale(x, scale=None):
    """invokeGetFP8WeightScale: scale = max(scale, max|x|/448); allocates a zeroed scale if None."""
    _chk(x, "x", _FLOATS)
    if scale is None:
        scale = torch.zeros(1, dtype=torch.float32, device=x.device)
    _chk(scale, "scale", (torch.float32,))
    _l.check(_l.load().lq_fp8_amax_scale(_ptr(scale), _ptr(x), _DT[x.dtype], x.numel(), _stream()),
             "lq_fp8_amax_scale")
    return scale


def fp8_scale_cast(x, scale, invert: bool = True):
    """invokeCudaD2DScaleCpyConvert to e4m3; returns a uint8 tensor of e4m3fn codes."""
    _chk(x, "x", _FLOATS)
    _chk(scale, "scale", (torch.float32,))
    q = torch.empty(x.shape, dtype=torch.uint8, device=x.device)
    _l.check(_l.load().lq_fp8_scale_cast(_ptr(q), _ptr(x), _DT[x.dtype], _ptr(scale), int(invert), x.numel(),
                                         _stream()), "lq_fp8_scale_cast")
    return q


def fp8_quant(x):
    """Dynamic per-tensor activation quant: returns (e4m3 codes uint8, scale fp32 [1])."""
    _chk(x, "x", _FLOATS)
    q = torch.empty(x.shape, dtype=torch.uint8, device=x.device)
    s = torch.empty(1, dtype=torch.float32, device=x.device)
    _l.check(_l.load().lq_fp8_amax_cast(_ptr(q), _ptr(s), _ptr(x), _DT[x.dtype], x.numel(), _stream()),
             "lq_fp8_amax_cast")
    return q, s


def fp8_amax_cast_status() -> bool:
    """True when something went wrong in a dynamic fp8 quantisation on the current device since the last call: a one-launch
    fp8_quant timed out at its exchange (its scale is NaN), or overlapping fp8_quant_static calls corrupted the ticket
    counters (fp8_quant_static_reset repairs them); lyradiff_amd.lib.load().lq_last_error() says which.  Copies 8 bytes from
    the device: synchronise the quantising streams first."""
    rc = _l.load().lq_fp8_amax_cast_status()
    if rc < 0:
        _l.check(rc, "lq_fp8_amax_cast_status")
    return rc >= 1


def fp8_quant_release_stream(stream=None) -> int:
    """Gives back the exchange slot the one-launch fp8_quant holds for `stream` (default: the current stream); call it before a
    stream that quantised is destroyed.  Returns the freed slot or -1."""
    st = _stream() if stream is None else stream.cuda_stream
    return int(_l.load().lq_fp8_amax_cast_release_slot(st))


def fp8_quant_static_reset() -> None:
    """Puts the ticket counters of fp8_quant_static back to zero on the current stream (after calls overlapped)."""
    _l.check(_l.load().lq_fp8_amax_cast_static_reset(_stream()), "lq_fp8_amax_cast_static_reset")


def fp8_quant_timeline(x):
    """fp8_quant's one launch with device time stamps: returns (codes, scale, stamps int64 [workgroups, 4] in units of 10 ns:
    started, loads back, released from the exchange, stores acknowledged)."""
    _chk(x, "x", _FLOATS)
    q = torch.empty(x.shape, dtype=torch.uint8, device=x.device)
    s = torch.empty(1, dtype=torch.float32, device=x.device)
    stamps = torch.zeros((512, 4), dtype=torch.int64, device=x.device)
    _l.check(_l.load().lq_fp8_amax_cast_timeline(_ptr(q), _ptr(s), _ptr(x), _DT[x.dtype], x.numel(), _ptr(stamps), _stream()),
             "lq_fp8_amax_cast_timeline")
    return q, s, stamps[stamps[:, 0] != 0]


def fp8_quant_static(x, q_out, scale_out):
    """fp8_quant into caller-owned outputs through lq_fp8_amax_cast_static: two launches, no barrier, no allocation
    (scratch in a static device array shared by every call on the GPU: do not overlap calls)."""
    _chk(x, "x", _FLOATS)
    _chk(q_out, "q_out", (torch.uint8,))
    _chk(scale_out, "scale_out", (torch.float32,))
    if q_out.numel() != x.numel() or scale_out.numel() < 1:
        raise ValueError("q_out must have as many elements as x, scale_out at least one")
    _l.check(_l.load().lq_fp8_amax_cast_static(_ptr(q_out), _ptr(scale_out), _ptr(x), _DT[x.dtype], x.numel(), _stream()),
             "lq_fp8_amax_cast_static")
    return q_out, scale_out


# ---- W4A4 ------------------------------------------------------------------------------------------

def w4a4_quant(x, smooth=None, scale_dtype=torch.float32, group: int = 64):
    """Group-64 INT4 quantisation: returns (words int32 [M, K/8], scales [M, K/64])."""
    _chk(x, "x", _FLOATS)
    if smooth is not None:
        _chk(smooth, "smooth", (torch.float32,))
    m, k = x.shape
    q = torch.empty((m, k // 8), dtype=torch.int32, device=x.device)
    s = torch.empty((m, k // group), dtype=scale_dtype, device=x.device)
    _l.check(_l.load().lq_w4a4_quantize(_ptr(q), _ptr(s), _DT[scale_dtype], _ptr(x), _DT[x.dtype], _ptr(smooth),
                                        m, k, group, _stream()), "lq_w4a4_quantize")
    return q, s


# ---- weight repack ---------------------------------------------------------------------------------

def repack_weight(w_bytes, out=None):
    """[N, row_bytes] byte matrix (int8 / e4m3 codes / packed nibbles) -> rows32 layout, same size.
    `out` (same shape and dtype, not w_bytes itself) receives the result when given."""
    _chk(w_bytes, "w", (torch.int8, torch.uint8))
    n, rb = w_bytes.shape
    if out is None:
        out = torch.empty_like(w_bytes)
    _chk(out, "out", (w_bytes.dtype,))
    if out.shape != w_bytes.shape:
        raise ValueError("out must have the shape of w")
    _l.check(_l.load().lq_repack_rows32(_ptr(out), _ptr(w_bytes), n, rb, _stream()), "lq_repack_rows32")
    return out


def unpack_weight(packed):
    _chk(packed, "packed", (torch.int8, torch.uint8))
    n, rb = packed.shape
    out = torch.empty_like(packed)
    _l.check(_l.load().lq_unpack_rows32(_ptr(out), _ptr(packed), n, rb, _stream()), "lq_unpack_rows32")
    return out


# ---- GEMMs -----------------------------------------------------------------------------------------

def int8_linear(a_q, w_rows32, alpha_col, alpha_row, bias=None, out_dtype=torch.float16):
    """runGemmInt8 + fused bias: a_q int8 [M,K], w_rows32 int8 [N,K] (rows32), returns [M,N]."""
    _chk(a_q, "a_q", (torch.int8,))
    _chk(w_rows32, "w_rows32", (torch.int8,))
    m, k = a_q.shape
    n = w_rows32.shape[0]
    if w_rows32.shape[1] != k:
        raise ValueError("K mismatch between activation and weight")
    per_token = 0
    if out_dtype != torch.int32:
        _chk(alpha_col, "alpha_col", (torch.float32,))
        _chk(alpha_row, "alpha_row", (torch.float32,))
        if alpha_col.numel() != n:
            raise ValueError("alpha_col must have N elements")
        if alpha_row.numel() not in (1, m):
            raise ValueError("alpha_row must have 1 or M elements")
        per_token = int(alpha_row.numel() == m and m != 1)
    if bias is not None:
        _chk(bias, "bias", (out_dtype,))
    c = torch.empty((m, n), dtype=out_dtype, device=a_q.device)
    _l.check(_l.load().lq_gemm_int8(_ptr(c), _DT[out_dtype], _ptr(a_q), _ptr(w_rows32), _ptr(alpha_col),
                                    _ptr(alpha_row), per_token, _ptr(bias), m, n, k, _stream()), "lq_gemm_int8")
    return c


def fp8_linear(a_q, w_rows32, a_scale, b_scale, bias=None, gelu: bool = False, residual=None, beta: float = 0.0,
               out_dtype=torch.bfloat16, out_scale=None, out_fp8_scale=None, want_output: bool = True):
    """FP8 GemmWithResidualAndBias: a_q uint8 e4m3 [M,K], w_rows32 uint8 e4m3 [N,K] (rows32).
    out_scale (fp32 [1], zeroed by the caller): also accumulates max|C|/448, the dynamic e4m3 scale of the output.
    out_fp8_scale (fp32 [1], static): also returns the e4m3 codes of C with that scale -> (C, codes); with
    want_output=False the 16-bit C is not written at all and only the codes are returned."""
    _chk(a_q, "a_q", (torch.uint8,))
    _chk(w_rows32, "w_rows32", (torch.uint8,))
    _chk(a_scale, "a_scale", (torch.float32,))
    _chk(b_scale, "b_scale", (torch.float32,))
    m, k = a_q.shape
    n = w_rows32.shape[0]
    if w_rows32.shape[1] != k:
        raise ValueError("K mismatch between activation and weight")
    if bias is not None:
        _chk(bias, "bias", (out_dtype,))
    if residual is not None:
        _chk(residual, "residual", (out_dtype,))
    for name, t in (("out_scale", out_scale), ("out_fp8_scale", out_fp8_scale)):
        if t is not None:
            _chk(t, name, (torch.float32,))
    if not want_output and out_fp8_scale is None:
        raise ValueError("want_output=False needs out_fp8_scale")
    c = torch.empty((m, n), dtype=out_dtype, device=a_q.device) if want_output else None
    c8 = torch.empty((m, n), dtype=torch.uint8, device=a_q.device) if out_fp8_scale is not None else None
    _l.check(_l.load().lq_gemm_fp8_ex(_ptr(c), _DT[out_dtype], _ptr(a_q), _ptr(w_rows32), _ptr(a_scale), _ptr(b_scale),
                                      _ptr(bias), int(gelu), _ptr(residual), float(beta), m, n, k, _ptr(out_scale), _ptr(c8),
                                      _ptr(out_fp8_scale), _stream()), "lq_gemm_fp8")
    if out_fp8_scale is None:
        return c
    return (c, c8) if want_output else c8


def fp8_linear_max(a_q, w_rows32, a_scale, b_scale, bias, out_max, out_dtype=torch.bfloat16):
    """fp8_linear without activation that also joins its largest output into out_max (fp32 [1], zeroed by the caller; stays
    >= 0): what fp8_gelu_quant needs to quantise gelu(C) in one pass."""
    _chk(a_q, "a_q", (torch.uint8,))
    _chk(w_rows32, "w_rows32", (torch.uint8,))
    _chk(a_scale, "a_scale", (torch.float32,))
    _chk(b_scale, "b_scale", (torch.float32,))
    _chk(out_max, "out_max", (torch.float32,))
    m, k = a_q.shape
    n = w_rows32.shape[0]
    if w_rows32.shape[1] != k:
        raise ValueError("K mismatch between activation and weight")
    if bias is not None:
        _chk(bias, "bias", (out_dtype,))
    c = torch.empty((m, n), dtype=out_dtype, device=a_q.device)
    _l.check(_l.load().lq_gemm_fp8_max(_ptr(c), _DT[out_dtype], _ptr(a_q), _ptr(w_rows32), _ptr(a_scale), _ptr(b_scale),
                                       _ptr(bias), m, n, k, _ptr(out_max), _stream()), "lq_gemm_fp8_max")
    return c


def fp8_gelu_quant(y, y_max, want_h: bool = False, clear_max=None):
    """h = T(gelu_tanh(y)), codes = e4m3(h / scale), scale = max|h| / 448 in one pass over y; y_max (fp32 [1]) >= max(y, 0) as
    fp8_linear_max leaves it.  Returns (codes uint8, scale fp32 [1]) and h when want_h.  clear_max (fp32 [1], another tensor
    than y_max) is set to 0 by the same launch: the slot of the next fp8_linear_max."""
    _chk(y, "y", _FLOATS)
    _chk(y_max, "y_max", (torch.float32,))
    if clear_max is not None:
        _chk(clear_max, "clear_max", (torch.float32,))
    q = torch.empty(y.shape, dtype=torch.uint8, device=y.device)
    s = torch.empty(1, dtype=torch.float32, device=y.device)
    h = torch.empty_like(y) if want_h else None
    _l.check(_l.load().lq_fp8_gelu_cast(_ptr(q), _ptr(s), _ptr(h), _ptr(y), _DT[y.dtype], y.numel(), _ptr(y_max), _ptr(clear_max), _stream()),
             "lq_fp8_gelu_cast")
    return (q, s, h) if want_h else (q, s)


# ---- activations in k-panels ------------------------------------------------------------------------------------------
# A quantised activation [M, K] stored as [K/64, M, 64] (k-panels): the 64 bytes a GEMM k-tile takes from each row are then
# contiguous over the rows, so the GEMM's transfers fetch whole 128-byte cache lines (a row-major operand gives half a line
# per row and every line is requested from L2 twice).  The quantisers write the layout directly; the GEMM results are the
# bits of the row-major calls.  K % 64 == 0.

def fp8_panels_to_rows(q_panels):
    """[K/64, M, 64] k-panels -> the row-major [M, K] tensor (a copy; for checks and for consumers of the plain layout)."""
    kp, m, w = q_panels.shape
    return q_panels.permute(1, 0, 2).reshape(m, kp * w).contiguous()


def _panel_block(out, m: int, n: int, col_offset: int) -> int:
    """Address of columns [col_offset, col_offset + n) inside k-panels out [W/64, M, 64]: a block of columns is a run of whole
    panels, so writing into a wider destination is a pointer offset."""
    _chk(out, "out", (torch.uint8,))
    if out.dim() != 3 or out.shape[1] != m or out.shape[2] != 64 or col_offset < 0 or col_offset % 64 != 0 or n % 64 != 0 or \
            col_offset + n > out.shape[0] * 64:
        raise ValueError("out must be k-panels [W/64, M, 64] with col_offset and N multiples of 64 and col_offset + N <= W")
    return out.data_ptr() + (col_offset // 64) * m * 64


def fp8_scale_cast_panels(x, scale, invert: bool = True, out=None, col_offset: int = 0):
    """fp8_scale_cast (a given scale: the reference's static input scale) of a 2-D x [M, K] into k-panels uint8 [K/64, M, 64],
    or into columns [col_offset, col_offset + K) of wider k-panels `out` [W/64, M, 64]."""
    _chk(x, "x", _FLOATS)
    _chk(scale, "scale", (torch.float32,))
    if x.dim() != 2 or x.shape[1] % 64 != 0:
        raise ValueError("fp8_scale_cast_panels: x must be [M, K] with K % 64 == 0")
    m, k = x.shape
    if out is None:
        out = torch.empty((k // 64, m, 64), dtype=torch.uint8, device=x.device)
    _l.check(_l.load().lq_fp8_scale_cast_panels(_panel_block(out, m, k, col_offset), _ptr(x), _DT[x.dtype], _ptr(scale), int(invert), m, k,
                                                _stream()), "lq_fp8_scale_cast_panels")
    return out


def fp8_quant_panels(x):
    """fp8_quant of a 2-D x [M, K] with the codes written as k-panels: returns (uint8 [K/64, M, 64], scale fp32 [1])."""
    _chk(x, "x", _FLOATS)
    if x.dim() != 2 or x.shape[1] % 64 != 0:
        raise ValueError("fp8_quant_panels: x must be [M, K] with K % 64 == 0")
    m, k = x.shape
    q = torch.empty((k // 64, m, 64), dtype=torch.uint8, device=x.device)
    s = torch.empty(1, dtype=torch.float32, device=x.device)
    _l.check(_l.load().lq_fp8_amax_cast_panels(_ptr(q), _ptr(s), _ptr(x), _DT[x.dtype], m, k, _stream()), "lq_fp8_amax_cast_panels")
    return q, s


def fp8_gelu_quant_panels(y, y_max, clear_max=None):
    """fp8_gelu_quant of a 2-D y [M, K] with the codes written as k-panels [K/64, M, 64]."""
    _chk(y, "y", _FLOATS)
    _chk(y_max, "y_max", (torch.float32,))
    if clear_max is not None:
        _chk(clear_max, "clear_max", (torch.float32,))
    if y.dim() != 2 or y.shape[1] % 64 != 0:
        raise ValueError("fp8_gelu_quant_panels: y must be [M, K] with K % 64 == 0")
    m, k = y.shape
    q = torch.empty((k // 64, m, 64), dtype=torch.uint8, device=y.device)
    s = torch.empty(1, dtype=torch.float32, device=y.device)
    _l.check(_l.load().lq_fp8_gelu_cast_panels(_ptr(q), _ptr(s), _ptr(y), _DT[y.dtype], m, k, _ptr(y_max), _ptr(clear_max), _stream()),
             "lq_fp8_gelu_cast_panels")
    return q, s


def fp8_linear_panels(a_panels, w_rows32, a_scale, b_scale, bias, out_max=None, out_dtype=torch.bfloat16):
    """fp8_linear (scales and bias, no activation) on an activation in k-panels [K/64, M, 64]; with out_max (fp32 [1]) also
    fp8_linear_max.  Same bits as the row-major calls."""
    _chk(a_panels, "a_panels", (torch.uint8,))
    _chk(w_rows32, "w_rows32", (torch.uint8,))
    _chk(a_scale, "a_scale", (torch.float32,))
    _chk(b_scale, "b_scale", (torch.float32,))
    if out_max is not None:
        _chk(out_max, "out_max", (torch.float32,))
    if a_panels.dim() != 3 or a_panels.shape[2] != 64:
        raise ValueError("fp8_linear_panels: a_panels must be [K/64, M, 64]")
    kp, m, _ = a_panels.shape
    k = kp * 64
    n = w_rows32.shape[0]
    if w_rows32.shape[1] != k:
        raise ValueError("K mismatch between activation and weight")
    if bias is not None:
        _chk(bias, "bias", (out_dtype,))
    c = torch.empty((m, n), dtype=out_dtype, device=a_panels.device)
    _l.check(_l.load().lq_gemm_fp8_panels(_ptr(c), _DT[out_dtype], _ptr(a_panels), _ptr(w_rows32), _ptr(a_scale), _ptr(b_scale),
                                          _ptr(bias), m, n, k, _ptr(out_max), _stream()), "lq_gemm_fp8_panels")
    return c


def sq_quant_dynamic_panels(x, pre_quant_scale=None):
    """sq_quant_dynamic of a 2-D x [M, K] with the codes written as k-panels: returns (int8 [K/64, M, 64], scale fp32 [M])."""
    _chk(x, "x", _FLOATS)
    if x.dim() != 2 or x.shape[1] % 64 != 0:
        raise ValueError("sq_quant_dynamic_panels: x must be [M, K] with K % 64 == 0")
    m, k = x.shape
    if pre_quant_scale is not None:
        _chk(pre_quant_scale, "pre_quant_scale", (torch.float32,))
        if pre_quant_scale.numel() != k:
            raise ValueError("pre_quant_scale must have K elements")
    q = torch.empty((k // 64, m, 64), dtype=torch.int8, device=x.device)
    s = torch.empty(m, dtype=torch.float32, device=x.device)
    _l.check(_l.load().lq_sq_dynamic_quant_panels(_ptr(q), _ptr(s), _ptr(x), _DT[x.dtype], _ptr(pre_quant_scale), m, k, _stream()),
             "lq_sq_dynamic_quant_panels")
    return q, s


def int8_linear_panels(a_panels, w_rows32, alpha_col, alpha_row, bias=None, out_dtype=torch.float16):
    """int8_linear on an activation in k-panels [K/64, M, 64].  Same bits as the row-major call."""
    _chk(a_panels, "a_panels", (torch.int8,))
    _chk(w_rows32, "w_rows32", (torch.int8,))
    if a_panels.dim() != 3 or a_panels.shape[2] != 64:
        raise ValueError("int8_linear_panels: a_panels must be [K/64, M, 64]")
    kp, m, _ = a_panels.shape
    k = kp * 64
    n = w_rows32.shape[0]
    if w_rows32.shape[1] != k:
        raise ValueError("K mismatch between activation and weight")
    per_token = 0
    if out_dtype != torch.int32:
        _chk(alpha_col, "alpha_col", (torch.float32,))
        _chk(alpha_row, "alpha_row", (torch.float32,))
        if alpha_col.numel() != n:
            raise ValueError("alpha_col must have N elements")
        if alpha_row.numel() not in (1, m):
            raise ValueError("alpha_row must have 1 or M elements")
        per_token = int(alpha_row.numel() == m and m != 1)
    if bias is not None:
        _chk(bias, "bias", (out_dtype,))
    c = torch.empty((m, n), dtype=out_dtype, device=a_panels.device)
    _l.check(_l.load().lq_gemm_int8_panels(_ptr(c), _DT[out_dtype], _ptr(a_panels), _ptr(w_rows32), _ptr(alpha_col),
                                           _ptr(alpha_row), per_token, _ptr(bias), m, n, k, _stream()), "lq_gemm_int8_panels")
    return c


def fp8_linear_gated(a_q, w_rows32, a_scale, b_scale, bias, gate, residual, rows_per_gate: int, out=None):
    """FP8 GEMM + invokeFusedGateAndResidual: out = residual + gate[row // rows_per_gate] * (A.W^T*sa*sb + bias), with
    the roundings of the unfused sequence.  gate [ceil(M/rows_per_gate), N], residual [M, N]; out may be residual."""
    _chk(a_q, "a_q", (torch.uint8,))
    _chk(w_rows32, "w_rows32", (torch.uint8,))
    _chk(a_scale, "a_scale", (torch.float32,))
    _chk(b_scale, "b_scale", (torch.float32,))
    _chk(residual, "residual", _FLOATS)
    _chk(gate, "gate", (residual.dtype,))
    if bias is not None:
        _chk(bias, "bias", (residual.dtype,))
    m, k = a_q.shape
    n = w_rows32.shape[0]
    if w_rows32.shape[1] != k:
        raise ValueError("K mismatch between activation and weight")
    if residual.numel() != m * n or rows_per_gate <= 0 or gate.numel() != ((m + rows_per_gate - 1) // rows_per_gate) * n:
        raise ValueError("residual must be [M,N] and gate [ceil(M/rows_per_gate), N]")
    if out is None:
        out = torch.empty((m, n), dtype=residual.dtype, device=a_q.device)
    _chk(out, "out", (residual.dtype,))
    _l.check(_l.load().lq_gemm_fp8_gated(_ptr(out), _DT[residual.dtype], _ptr(a_q), _ptr(w_rows32), _ptr(a_scale), _ptr(b_scale),
                                         _ptr(bias), _ptr(gate), int(rows_per_gate), _ptr(residual), m, n, k, _stream()),
             "lq_gemm_fp8_gated")
    return out


def fp8_linear_codes(a_q, w_rows32, a_scale, b_scale, bias, out_fp8_scale, gelu: int = 0, round_dtype=torch.bfloat16,
                     out=None, col_offset: int = 0):
    """FP8 GEMM that writes only e4m3 codes (static scale out_fp8_scale) of its optionally GELU'd output, into columns
    [col_offset, col_offset+N) of `out` (uint8 [M, W], allocated [M, N] when None).  gelu: 0 none, 1 on the fp32 value,
    2 on the value rounded to round_dtype first."""
    _chk(a_q, "a_q", (torch.uint8,))
    _chk(w_rows32, "w_rows32", (torch.uint8,))
    _chk(a_scale, "a_scale", (torch.float32,))
    _chk(b_scale, "b_scale", (torch.float32,))
    _chk(out_fp8_scale, "out_fp8_scale", (torch.float32,))
    if bias is not None:
        _chk(bias, "bias", (round_dtype,))
    m, k = a_q.shape
    n = w_rows32.shape[0]
    if w_rows32.shape[1] != k:
        raise ValueError("K mismatch between activation and weight")
    if out is None:
        out = torch.empty((m, n), dtype=torch.uint8, device=a_q.device)
    _chk(out, "out", (torch.uint8,))
    if out.dim() != 2 or out.shape[0] != m or col_offset < 0 or col_offset + n > out.shape[1]:
        raise ValueError("out must be [M, W] with col_offset + N <= W")
    _l.check(_l.load().lq_gemm_fp8_codes(out.data_ptr() + col_offset, out.shape[1], _ptr(out_fp8_scale), _DT[round_dtype],
                                         _ptr(a_q), _ptr(w_rows32), _ptr(a_scale), _ptr(b_scale), _ptr(bias), int(gelu), m, n, k,
                                         _stream()), "lq_gemm_fp8_codes")
    return out


def fp8_linear_gated_panels(a_panels, w_rows32, a_scale, b_scale, bias, gate, residual, rows_per_gate: int, out=None):
    """fp8_linear_gated on an activation in k-panels [K/64, M, 64].  Same bits as the row-major call."""
    _chk(a_panels, "a_panels", (torch.uint8,))
    _chk(w_rows32, "w_rows32", (torch.uint8,))
    _chk(a_scale, "a_scale", (torch.float32,))
    _chk(b_scale, "b_scale", (torch.float32,))
    _chk(residual, "residual", _FLOATS)
    _chk(gate, "gate", (residual.dtype,))
    if bias is not None:
        _chk(bias, "bias", (residual.dtype,))
    if a_panels.dim() != 3 or a_panels.shape[2] != 64:
        raise ValueError("a_panels must be [K/64, M, 64]")
    kp, m, _ = a_panels.shape
    k, n = kp * 64, w_rows32.shape[0]
    if w_rows32.shape[1] != k:
        raise ValueError("K mismatch between activation and weight")
    if residual.numel() != m * n or rows_per_gate <= 0 or gate.numel() != ((m + rows_per_gate - 1) // rows_per_gate) * n:
        raise ValueError("residual must be [M,N] and gate [ceil(M/rows_per_gate), N]")
    if out is None:
        out = torch.empty((m, n), dtype=residual.dtype, device=a_panels.device)
    _chk(out, "out", (residual.dtype,))
    _l.check(_l.load().lq_gemm_fp8_gated_panels(_ptr(out), _DT[residual.dtype], _ptr(a_panels), _ptr(w_rows32), _ptr(a_scale),
                                                _ptr(b_scale), _ptr(bias), _ptr(gate), int(rows_per_gate), _ptr(residual), m, n, k,
                                                _stream()), "lq_gemm_fp8_gated_panels")
    return out


def fp8_linear_codes_panels(a_panels, w_rows32, a_scale, b_scale, bias, out_fp8_scale, gelu: int = 0, round_dtype=torch.bfloat16,
                            out=None, col_offset: int = 0):
    """fp8_linear_codes with both the activation and the codes it writes as k-panels: a_panels [K/64, M, 64] -> codes
    [N/64, M, 64], or columns [col_offset, col_offset + N) of wider k-panels `out` [W/64, M, 64].  Same codes as the row-major
    call."""
    _chk(a_panels, "a_panels", (torch.uint8,))
    _chk(w_rows32, "w_rows32", (torch.uint8,))
    _chk(a_scale, "a_scale", (torch.float32,))
    _chk(b_scale, "b_scale", (torch.float32,))
    _chk(out_fp8_scale, "out_fp8_scale", (torch.float32,))
    if bias is not None:
        _chk(bias, "bias", (round_dtype,))
    if a_panels.dim() != 3 or a_panels.shape[2] != 64:
        raise ValueError("a_panels must be [K/64, M, 64]")
    kp, m, _ = a_panels.shape
    k, n = kp * 64, w_rows32.shape[0]
    if w_rows32.shape[1] != k:
        raise ValueError("K mismatch between activation and weight")
    if n % 64 != 0:
        raise ValueError("codes in k-panels need N % 64 == 0")
    if out is None:
        out = torch.empty((n // 64, m, 64), dtype=torch.uint8, device=a_panels.device)
    _l.check(_l.load().lq_gemm_fp8_codes_panels(_panel_block(out, m, n, col_offset), _ptr(out_fp8_scale), _DT[round_dtype], _ptr(a_panels),
                                                _ptr(w_rows32), _ptr(a_scale), _ptr(b_scale), _ptr(bias), int(gelu), m, n, k, _stream()),
             "lq_gemm_fp8_codes_panels")
    return out


def fp8_scale_cast_into(x, scale, out, col_offset: int = 0, invert: bool = True):
    """invokeCudaD2DScaleCpyConvert of x [M, C] into columns [col_offset, col_offset+C) of out (uint8 [M, W])."""
    _chk(x, "x", _FLOATS)
    _chk(scale, "scale", (torch.float32,))
    _chk(out, "out", (torch.uint8,))
    if x.dim() != 2 or out.dim() != 2 or out.shape[0] != x.shape[0] or col_offset < 0 or col_offset + x.shape[1] > out.shape[1]:
        raise ValueError("x must be [M, C] and out [M, W] with col_offset + C <= W")
    _l.check(_l.load().lq_fp8_scale_cast_2d(out.data_ptr() + col_offset, out.shape[1], _ptr(x), x.shape[1], _DT[x.dtype],
                                            _ptr(scale), int(invert), x.shape[0], x.shape[1], _stream()), "lq_fp8_scale_cast_2d")
    return out


def repack_weight_only(q_kn, kind: str):
    """One-time preparation of a weight-only weight.  q_kn: int8 [K, N] signed codes, or for kind "int4" int8
    [K, N/2] with column 2j in the low nibble (the reference's unprocessed_quantized_weight).  Returns the uint8
    tensor [N, K] / [N, K/2] that weight_only_linear reads."""
    _chk(q_kn, "q_kn", (torch.int8,))
    k = q_kn.shape[0]
    n = q_kn.shape[1] * (2 if kind == "int4" else 1)
    out = torch.empty((n, k // 2 if kind == "int4" else k), dtype=torch.uint8, device=q_kn.device)
    _l.check(_l.load().lq_repack_weight_only(_ptr(out), _ptr(q_kn), _KINDS[kind], k, n, _stream()), "lq_repack_weight_only")
    return out


def weight_only_linear(x, w_prepared, scales, bias=None, kind: str = "int8"):
    """W8A16 / W4A16 linear: x [M, K] fp16/bf16, w_prepared from repack_weight_only, scales and bias [N] of x.dtype."""
    _chk(x, "x", (torch.float16, torch.bfloat16))
    _chk(w_prepared, "w_prepared", (torch.uint8,))
    _chk(scales, "scales", (x.dtype,))
    if bias is not None:
        _chk(bias, "bias", (x.dtype,))
    m, k = x.shape
    n = w_prepared.shape[0]
    if w_prepared.shape[1] != (k // 2 if kind == "int4" else k) or scales.numel() != n:
        raise ValueError("shape mismatch between x, w_prepared and scales")
    c = torch.empty((m, n), dtype=x.dtype, device=x.device)
    _l.check(_l.load().lq_gemm_weight_only(_ptr(c), _ptr(x), _DT[x.dtype], _ptr(w_prepared), _KINDS[kind], _ptr(scales),
                                           _ptr(bias), m, n, k, _stream()), "lq_gemm_weight_only")
    return c


def weight_only_linear_grouped(x, w_prepared, scales, zeros=None, bias=None, kind: str = "int8", group_size: int = 128):
    """W8A16 / W4A16 linear with group-wise scales [K / group_size, N] and optional zero points of the same shape (the
    reference's FINEGRAINED_SCALE_ONLY / FINEGRAINED_SCALE_AND_ZEROS): every weight is dequantised in x.dtype,
    w = q * scale (+ zero), before it is multiplied."""
    _chk(x, "x", (torch.float16, torch.bfloat16))
    _chk(w_prepared, "w_prepared", (torch.uint8,))
    _chk(scales, "scales", (x.dtype,))
    for name, t in (("zeros", zeros), ("bias", bias)):
        if t is not None:
            _chk(t, name, (x.dtype,))
    m, k = x.shape
    n = w_prepared.shape[0]
    if group_size not in (64, 128) or k % group_size:
        raise ValueError("group_size must be 64 or 128 and divide K")
    if w_prepared.shape[1] != (k // 2 if kind == "int4" else k) or tuple(scales.shape) != (k // group_size, n) or \
            (zeros is not None and zeros.shape != scales.shape) or (bias is not None and bias.numel() != n):
        raise ValueError("shape mismatch between x, w_prepared, scales [K/group, N], zeros and bias")
    c = torch.empty((m, n), dtype=x.dtype, device=x.device)
    _l.check(_l.load().lq_gemm_weight_only_grouped(_ptr(c), _ptr(x), _DT[x.dtype], _ptr(w_prepared), _KINDS[kind], _ptr(scales),
                                                   _ptr(zeros), _ptr(bias), m, n, k, int(group_size), _stream()),
             "lq_gemm_weight_only_grouped")
    return c


def load_lora(weight, lora, alpha: float):
    """invokeLoadLora: weight += lora * alpha in the tensors' dtype, in place; returns weight."""
    _chk(weight, "weight", _FLOATS)
    _chk(lora, "lora", (weight.dtype,))
    if lora.numel() != weight.numel():
        raise ValueError("lora and weight must have the same number of elements")
    _l.check(_l.load().lq_load_lora(_ptr(weight), _ptr(lora), _DT[weight.dtype], weight.numel(), float(alpha), _stream()),
             "lq_load_lora")
    return weight


def w4a4_linear(a_words, w_rows32, sA, sB, bias=None, out_dtype=torch.bfloat16, group: int = 64, lora_act=None, lora_up=None,
                gelu: int = 0, addend=None, gate=None, residual=None, rows_per_gate: int = 1, out_fp8_scale=None,
                out_fp8=None, col_offset: int = 0, want_output: bool = True, out=None):
    """W4A4 GEMM: a_words int32 [M,K/8], w_rows32 uint8 [N,K/2] (rows32), scales [M,G] / [N,G].
    lora_act [M,R] and lora_up [N,R] (fp16 or bf16, R a multiple of 16) add the low-rank branch.
    Epilogue options, in this order: gelu (1: on fp32, 2: on the T-rounded value), addend [M,N] (T(T(y)+addend)),
    gate + residual (T(T(T(y)*gate[row // rows_per_gate]) + residual)), out_fp8_scale (e4m3 codes of the result, into
    columns [col_offset, col_offset+N) of out_fp8 when given; want_output=False skips the 16-bit output)."""
    _chk(a_words, "a_words", (torch.int32,))
    _chk(w_rows32, "w_rows32", (torch.uint8, torch.int8))
    _chk(sA, "sA", (torch.float32, torch.float16))
    _chk(sB, "sB", (sA.dtype,))
    m = a_words.shape[0]
    k = a_words.shape[1] * 8
    n = w_rows32.shape[0]
    if w_rows32.shape[1] * 2 != k:
        raise ValueError("K mismatch between activation and weight")
    if bias is not None:
        _chk(bias, "bias", (out_dtype,))
    rank, lora_dt = 0, _l.LQ_BF16
    if (lora_act is None) != (lora_up is None):
        raise ValueError("the low-rank branch needs both lora_act and lora_up")
    if lora_act is not None:
        _chk(lora_act, "lora_act", (torch.float16, torch.bfloat16))
        _chk(lora_up, "lora_up", (lora_act.dtype,))
        rank = lora_act.shape[1]
        if lora_act.shape[0] != m or tuple(lora_up.shape) != (n, rank):
            raise ValueError("lora_act must be [M,R] and lora_up [N,R]")
        lora_dt = _DT[lora_act.dtype]
    epi = None
    c8 = None
    if gelu or addend is not None or gate is not None or out_fp8_scale is not None:
        for name, t in (("addend", addend), ("gate", gate), ("residual", residual)):
            if t is not None:
                _chk(t, name, (out_dtype,))
        if (gate is None) != (residual is None):
            raise ValueError("gate and residual go together")
        if gate is not None and (residual.numel() != m * n or rows_per_gate <= 0 or
                                 gate.numel() != ((m + rows_per_gate - 1) // rows_per_gate) * n):
            raise ValueError("residual must be [M,N] and gate [ceil(M/rows_per_gate), N]")
        if addend is not None and addend.numel() != m * n:
            raise ValueError("addend must be [M,N]")
        epi = _l.Epilogue(int(gelu), _ptr(addend), _ptr(gate), int(rows_per_gate), _ptr(residual), None, 0, None)
        if out_fp8_scale is not None:
            _chk(out_fp8_scale, "out_fp8_scale", (torch.float32,))
            c8 = out_fp8 if out_fp8 is not None else torch.empty((m, n), dtype=torch.uint8, device=a_words.device)
            _chk(c8, "out_fp8", (torch.uint8,))
            if c8.dim() != 2 or c8.shape[0] != m or col_offset < 0 or col_offset + n > c8.shape[1]:
                raise ValueError("out_fp8 must be [M, W] with col_offset + N <= W")
            epi.C_fp8, epi.ldc_fp8, epi.C_fp8_scale = c8.data_ptr() + col_offset, c8.shape[1], _ptr(out_fp8_scale)
    if not want_output and c8 is None:
        raise ValueError("want_output=False needs out_fp8_scale")
    c = (out if out is not None else torch.empty((m, n), dtype=out_dtype, device=a_words.device)) if want_output else None
    if c is not None:
        _chk(c, "out", (out_dtype,))
    _l.check(_l.load().lq_gemm_w4a4_ex(_ptr(c), _DT[out_dtype], _ptr(a_words), _ptr(w_rows32), _ptr(sA), _ptr(sB),
                                       _DT[sA.dtype], _ptr(bias), _ptr(lora_act), _ptr(lora_up), lora_dt, rank, m, n, k,
                                       group, C.byref(epi) if epi is not None else None, _stream()), "lq_gemm_w4a4_ex")
    if c8 is None:
        return c
    return (c, c8) if want_output else c8


def lora_down(x, lora_down_w, out_dtype=None):
    """Low-rank down projection out[M,R] = x[M,K] . lora_down_w[R,K]^T (fp32 accumulation), R = 32 or 64."""
    _chk(x, "x", (torch.float16, torch.bfloat16))
    _chk(lora_down_w, "lora_down_w", (x.dtype,))
    m, k = x.shape
    rank = lora_down_w.shape[0]
    if lora_down_w.shape[1] != k:
        raise ValueError("K mismatch between x and lora_down_w")
    out_dtype = out_dtype or x.dtype
    out = torch.empty((m, rank), dtype=out_dtype, device=x.device)
    _l.check(_l.load().lq_lora_down(_ptr(out), _DT[out_dtype], _ptr(x), _ptr(lora_down_w), _DT[x.dtype], m, k, rank, _stream()),
             "lq_lora_down")
    return out


def w4a4_quant_lora_down(x, smooth, lora_down_w, scale_dtype=torch.float32, out_dtype=None, group: int = 64):
    """w4a4_quant and lora_down from one read of x (invokeFusedQuantizeAndLoraDownSimple, kernels/w4a4_gemm/w4a4_gemm.h:6-16):
    returns (words int32 [M, K/8], scales [M, K/64], lora_act [M, R])."""
    _chk(x, "x", (torch.float16, torch.bfloat16))
    _chk(lora_down_w, "lora_down_w", (x.dtype,))
    if smooth is not None:
        _chk(smooth, "smooth", (torch.float32,))
    m, k = x.shape
    rank = lora_down_w.shape[0]
    if lora_down_w.shape[1] != k:
        raise ValueError("K mismatch between x and lora_down_w")
    out_dtype = out_dtype or x.dtype
    q = torch.empty((m, k // 8), dtype=torch.int32, device=x.device)
    s = torch.empty((m, k // group), dtype=scale_dtype, device=x.device)
    act = torch.empty((m, rank), dtype=out_dtype, device=x.device)
    _l.check(_l.load().lq_w4a4_quantize_lora_down(_ptr(q), _ptr(s), _DT[scale_dtype], _ptr(act), _DT[out_dtype], _ptr(x),
                                                  _DT[x.dtype], _ptr(smooth), _ptr(lora_down_w), m, k, rank, group, _stream()),
             "lq_w4a4_quantize_lora_down")
    return q, s, act


def rmsnorm_rope(qkv, norm_qk, rope, heads: int, context_qkv=None, norm_added_qk=None, eps: float = 1e-6):
    """invokeFusedRmsNormCatAndRope / invokeFusedRmsNormAndRope: qkv [B, S, 3*H*Dh] (context_qkv [B, Sc, 3*H*Dh], text tokens,
    placed first) -> [B, Sc + S, 3, H, Dh] with q and k RMS-normalised per head, scaled by norm_qk / norm_added_qk ([2*Dh]: q
    weights then k weights) and rotated by the 2x2 matrices of rope [B or 1, Sc + S, Dh/2, 2, 2]; v copied."""
    _chk(qkv, "qkv", (torch.float16, torch.bfloat16))
    b, s, d3 = qkv.shape
    if d3 % (3 * heads):
        raise ValueError("the last dimension of qkv must be 3 * heads * head_dim")
    dh = d3 // (3 * heads)
    sc = 0
    for name, t in (("norm_qk", norm_qk), ("rope", rope), ("context_qkv", context_qkv), ("norm_added_qk", norm_added_qk)):
        if t is not None:
            _chk(t, name, (qkv.dtype,))
    if context_qkv is not None:
        if norm_added_qk is None or context_qkv.shape[0] != b or context_qkv.shape[2] != d3:
            raise ValueError("context_qkv needs norm_added_qk and the batch and width of qkv")
        sc = context_qkv.shape[1]
    if norm_qk.numel() != 2 * dh or (norm_added_qk is not None and norm_added_qk.numel() != 2 * dh):
        raise ValueError("norm weights must hold 2 * head_dim elements (q then k)")
    per_batch = (sc + s) * dh * 2
    if rope.numel() not in (per_batch, b * per_batch):
        raise ValueError("rope must be [B or 1, Sc + S, head_dim / 2, 2, 2]")
    out = torch.empty((b, sc + s, 3, heads, dh), dtype=qkv.dtype, device=qkv.device)
    _l.check(_l.load().lq_rmsnorm_rope(_ptr(out), _ptr(qkv), _ptr(context_qkv), _ptr(norm_qk), _ptr(norm_added_qk), _ptr(rope),
                                       per_batch if rope.numel() != per_batch else 0, _DT[qkv.dtype], b, s, sc, heads, dh, eps,
                                       _stream()), "lq_rmsnorm_rope")
    return out


_KINDS = {"int8": _l.LQ_W_INT8, "fp8": _l.LQ_W_FP8, "int4": _l.LQ_W_INT4}


def gemm_set_tactic(kind: str, tactic: int = -1) -> None:
    """Forces the tile configuration of the `kind` GEMM ("int8", "fp8", "int4"); -1 restores the
    built-in table (the role of the tactic argument of CutlassInt8GemmRunner<T>::gemm,
    src/lyradiff/kernels/cutlass_kernels/int8_gemm/int8_gemm.h:24-39)."""
    _l.check(_l.load().lq_gemm_set_tactic(_KINDS[kind], int(tactic)), "lq_gemm_set_tactic")


class gemm_thread_tactic:
    """`with gemm_thread_tactic(t):` -- the GEMM calls of this thread inside the block use tile configuration t (the per-call
    gemmConfig argument of the reference's runners, kernels/cutlass_kernels/int8_gemm/int8_gemm.h:24-36)."""

    def __init__(self, tactic: int):
        self.tactic = int(tactic)

    def __enter__(self):
        _l.check(_l.load().lq_gemm_set_thread_tactic(self.tactic), "lq_gemm_set_thread_tactic")
        return self

    def __exit__(self, *exc):
        _l.load().lq_gemm_set_thread_tactic(-1)
        return False


def gemm_tactics_dumps() -> bytes:
    """The per-shape tactic cache as bytes (GemmPluginProfiler::serialize, layers/gemm_utils/GemmProfiler.cc:26-38)."""
    lib = _l.load()
    size = int(lib.lq_gemm_tactics_serialized_size())
    buf = C.create_string_buffer(size + 64)  # room for entries another thread adds in between
    written = C.c_size_t(0)
    _l.check(lib.lq_gemm_tactics_serialize(buf, size + 64, C.byref(written)), "lq_gemm_tactics_serialize")
    return buf.raw[: written.value]


def gemm_tactics_loads(data: bytes) -> None:
    """Adds a table made by gemm_tactics_dumps to the cache (GemmPluginProfiler::deserialize, GemmProfiler.cc:40-65)."""
    _l.check(_l.load().lq_gemm_tactics_deserialize(C.c_char_p(bytes(data)), len(data)), "lq_gemm_tactics_deserialize")


def gemm_tactic_count(kind: str) -> int:
    return int(_l.load().lq_gemm_tactic_count(_KINDS[kind]))


def gemm_profile(kind: str, m: int, n: int, k: int, device=None):
    """Times every tile configuration of the `kind` GEMM on (m, n, k) and caches the fastest for later
    calls of that shape (GemmPluginProfiler::profileTactics, src/lyradiff/layers/gemm_utils/
    GemmProfiler.cc:78-127).  Set-up-time only: allocates a temporary buffer and blocks until timed.
    Returns (tactic, microseconds per call)."""
    import ctypes as C

    lib = _l.load()
    nbytes = int(lib.lq_gemm_profile_workspace(_KINDS[kind], m, n, k))
    if nbytes == 0:
        raise ValueError(f"bad profile request kind={kind} m={m} n={n} k={k}")
    ws = torch.empty(nbytes, dtype=torch.uint8, device=device or "cuda")
    best, us = C.c_int(-1), C.c_float(0.0)
    _l.check(lib.lq_gemm_profile(_KINDS[kind], m, n, k, ws.data_ptr(), nbytes, C.byref(best), C.byref(us), _stream()),
             "lq_gemm_profile")
    return best.value, us.value


def shader_clock_probe(microseconds: int, probes: int = 8, stream=None):
    """Enqueues lq_shader_clock_probe on `stream` (a torch stream; default: the current one) and returns the int64 tensor
    [probes, 2] it will fill with (shader clock ticks, 100 MHz ticks); after synchronising,
    0.1 * t[:, 0] / t[:, 1] is the clock in GHz the compute units ran at during the window."""
    out = torch.zeros((probes, 2), dtype=torch.int64, device="cuda")
    st = _stream() if stream is None else stream.cuda_stream
    _l.check(_l.load().lq_shader_clock_probe(_ptr(out), int(probes), int(microseconds), st), "lq_shader_clock_probe")
    return out


_PROBE_SINK = {}


def mfma_fp8_probe(codes, iters: int) -> float:
    """Enqueues lq_mfma_fp8_probe (one workgroup per CU, 16 x iters FP8 MFMAs of 32x32x64 per wavefront on register
    operands drawn from the uint8 e4m3 tensor `codes`, or on zeros when codes is None) and returns the FLOP of the launch."""
    dev = torch.cuda.current_device()
    sink = _PROBE_SINK.get(dev)
    if sink is None:
        sink = _PROBE_SINK[dev] = torch.zeros(1, dtype=torch.float32, device="cuda")
    wgs = C.c_int(0)
    _l.check(_l.load().lq_mfma_fp8_probe(_ptr(sink), None if codes is None else _ptr(codes), 0 if codes is None else codes.numel(),
                                         int(iters), C.byref(wgs), _stream()), "lq_mfma_fp8_probe")
    return 2.0 * 32 * 32 * 64 * 16 * iters * 4 * wgs.value


def gemm_shape_tactic(kind: str, m: int, n: int, k: int, tactic=None) -> int:
    """Reads (tactic=None) or writes the per-shape tactic cache; -1 removes an entry / means no entry."""
    lib = _l.load()
    if tactic is not None:
        _l.check(lib.lq_gemm_set_shape_tactic(_KINDS[kind], m, n, k, int(tactic)), "lq_gemm_set_shape_tactic")
    return int(lib.lq_gemm_get_shape_tactic(_KINDS[kind], m, n, k))

