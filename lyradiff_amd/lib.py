"""ctypes binding of liblyraquant.so (the C ABI declared in include/lyraquant.h).

The library is the product; this module only loads it and declares argument types.  There is
no CPU fallback: if the shared library is missing, import of the ops fails with a clear error.
"""
from __future__ import annotations

import ctypes as C
import os

PKG = os.path.dirname(os.path.abspath(__file__))


def _paths():
    """(C-ABI library, torch custom-class library).  LYRA_LIB_PATH is the variable the reference's Python wrapper hands to
    torch.classes.load_library (lyradiff/__init__.py:4-5): here it names libth_lyradiff.so, and liblyraquant.so is taken
    from the same directory (the class library links it by $ORIGIN); a LYRA_LIB_PATH that names liblyraquant.so itself is
    accepted too.  LYRA_LIB_PATH_AMD names liblyraquant.so directly and wins (a machine that also carries the reference's
    CUDA build).  Without either, the in-tree build."""
    ref = os.environ.get("LYRA_LIB_PATH")
    th = os.path.join(PKG, "libth_lyradiff.so")
    abi = os.path.join(PKG, "liblyraquant.so")
    if ref:
        if os.path.basename(ref).startswith("liblyraquant"):
            abi, th = ref, os.path.join(os.path.dirname(ref), "libth_lyradiff.so")
        else:
            th, abi = ref, os.path.join(os.path.dirname(os.path.abspath(ref)), "liblyraquant.so")
    return os.environ.get("LYRA_LIB_PATH_AMD") or abi, th


LIB_PATH, TH_LIB_PATH = _paths()
_th_loaded = False


def load_torch_classes():
    """torch.classes.load_library on libth_lyradiff.so: registers torch.classes.lyradiff.FluxTransformerBlockOp,
    FluxSingleTransformerBlockOp and LyraDiffCommonContext (th_op/th_lyradiff.cpp).  Fails loudly when the library is missing."""
    global _th_loaded
    if not _th_loaded:
        import torch

        if not os.path.exists(TH_LIB_PATH):
            raise ImportError(f"{TH_LIB_PATH} not found: run `python -m lyradiff_amd.build` (there is no Python fallback behind "
                              "torch.classes.lyradiff)")
        torch.classes.load_library(TH_LIB_PATH)
        _th_loaded = True
    return TH_LIB_PATH


LQ_F32, LQ_F16, LQ_BF16, LQ_I32 = 0, 1, 2, 3
LQ_W_INT8, LQ_W_FP8, LQ_W_INT4 = 0, 1, 2

# every symbol include/lyraquant.h declares: name -> (restype, argtypes)
_P, _I, _Z, _F = C.c_void_p, C.c_int, C.c_size_t, C.c_float
SYMBOLS = {
    "lq_last_error": (C.c_char_p, []),
    "lq_version": (_I, []),
    "lq_sq_input_quant": (_I, [_P, _P, _I, _P, _P, _I, _Z, _Z, _P]),
    "lq_sq_dynamic_quant": (_I, [_P, _P, _P, _I, _P, _Z, _Z, _P]),
    "lq_sq_output_dequant": (_I, [_P, _I, _P, _P, _P, _I, _Z, _Z, _P]),
    "lq_int8_weight_quant": (_I, [_P, _P, _P, _I, _P, _Z, _Z, _P]),
    "lq_geglu_int8": (_I, [_P, _P, _P, _I, _P, _P, _Z, _Z, _P]),
    "lq_geglu_int8_dynamic": (_I, [_P, _P, _P, _P, _I, _P, _Z, _Z, _P]),
    "lq_fp8_amax_scale": (_I, [_P, _P, _I, _Z, _P]),
    "lq_fp8_scale_cast": (_I, [_P, _P, _I, _P, _I, _Z, _P]),
    "lq_fp8_amax_cast": (_I, [_P, _P, _P, _I, _Z, _P]),
    "lq_fp8_amax_cast_status": (_I, []),
    "lq_fp8_amax_cast_slot": (_I, [_P]),
    "lq_fp8_amax_cast_release_slot": (_I, [_P]),
    "lq_fp8_amax_cast_static_reset": (_I, [_P]),
    "lq_fp8_amax_cast_static": (_I, [_P, _P, _P, _I, _Z, _P]),
    "lq_fp8_amax_cast_static_max_elems": (_Z, []),
    "lq_w4a4_quantize": (_I, [_P, _P, _I, _P, _I, _P, _I, _I, _I, _P]),
    "lq_weight_row_bytes": (_Z, [_I, _Z]),
    "lq_repack_rows32": (_I, [_P, _P, _Z, _Z, _P]),
    "lq_unpack_rows32": (_I, [_P, _P, _Z, _Z, _P]),
    "lq_gemm_int8": (_I, [_P, _I, _P, _P, _P, _P, _I, _P, _I, _I, _I, _P]),
    "lq_gemm_fp8": (_I, [_P, _I, _P, _P, _P, _P, _P, _I, _P, _F, _I, _I, _I, _P]),
    "lq_gemm_fp8_ex": (_I, [_P, _I, _P, _P, _P, _P, _P, _I, _P, _F, _I, _I, _I, _P, _P, _P, _P]),
    "lq_gemm_fp8_gated": (_I, [_P, _I, _P, _P, _P, _P, _P, _P, _Z, _P, _I, _I, _I, _P]),
    "lq_gemm_fp8_codes": (_I, [_P, _Z, _P, _I, _P, _P, _P, _P, _P, _I, _I, _I, _I, _P]),
    "lq_fp8_scale_cast_2d": (_I, [_P, _Z, _P, _Z, _I, _P, _I, _Z, _Z, _P]),
    "lq_gemm_w4a4": (_I, [_P, _I, _P, _P, _P, _P, _I, _P, _I, _I, _I, _I, _P]),
    "lq_gemm_weight_only": (_I, [_P, _P, _I, _P, _I, _P, _P, _I, _I, _I, _P]),
    "lq_gemm_weight_only_grouped": (_I, [_P, _P, _I, _P, _I, _P, _P, _P, _I, _I, _I, _I, _P]),
    "lq_repack_weight_only": (_I, [_P, _P, _I, _Z, _Z, _P]),
    "lq_col_absmax": (_I, [_P, _P, _I, _Z, _Z, _P]),
    "lq_smooth_vector": (_I, [_P, _P, _P, _P, _F, _Z, _P]),
    "lq_layernorm_int8": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _I, _P, _P, _Z, _Z, _F, _P]),
    "lq_layernorm_mod_fp8": (_I, [_P, _P, _P, _P, _I, _P, _Z, _Z, _Z, _F, _P]),
    "lq_layernorm_mod_fp8_dual": (_I, [_P, _P, _P, _P, _P, _P, _P, _I, _Z, _Z, _Z, _F, _P]),
    "lq_gate_residual_layernorm_mod_fp8": (_I, [_P, _P, _P, _P, _P, _P, _P, _I, _P, _Z, _Z, _Z, _F, _P]),
    "lq_gate_residual_layernorm_mod": (_I, [_P, _P, _P, _P, _P, _P, _P, _I, _Z, _Z, _Z, _F, _P]),
    "lq_gemm_w4a4_ex": (_I, [_P, _I, _P, _P, _P, _P, _I, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P, _P]),
    "lq_gemm_w4a4_lora": (_I, [_P, _I, _P, _P, _P, _P, _I, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P]),
    "lq_fp8_amax_cast_timeline": (_I, [_P, _P, _P, _I, _Z, _P, _P]),
    "lq_gemm_fp8_max": (_I, [_P, _I, _P, _P, _P, _P, _P, _I, _I, _I, _P, _P]),
    "lq_fp8_gelu_cast": (_I, [_P, _P, _P, _P, _I, _Z, _P, _P, _P]),
    "lq_fp8_amax_cast_panels": (_I, [_P, _P, _P, _I, _Z, _Z, _P]),
    "lq_layernorm_mod_fp8_panels": (_I, [_P, _P, _P, _P, _I, _P, _Z, _Z, _Z, _F, _P]),
    "lq_layernorm_mod_fp8_dual_panels": (_I, [_P, _P, _P, _P, _P, _P, _P, _I, _Z, _Z, _Z, _F, _P]),
    "lq_gate_residual_layernorm_mod_fp8_panels": (_I, [_P, _P, _P, _P, _P, _P, _P, _I, _P, _Z, _Z, _Z, _F, _P]),
    "lq_gemm_fp8_gated_panels": (_I, [_P, _I, _P, _P, _P, _P, _P, _P, _Z, _P, _I, _I, _I, _P]),
    "lq_gemm_fp8_codes_panels": (_I, [_P, _P, _I, _P, _P, _P, _P, _P, _I, _I, _I, _I, _P]),
    "lq_fp8_scale_cast_panels": (_I, [_P, _P, _I, _P, _I, _Z, _Z, _P]),
    "lq_sq_dynamic_quant_panels": (_I, [_P, _P, _P, _I, _P, _Z, _Z, _P]),
    "lq_gemm_int8_panels": (_I, [_P, _I, _P, _P, _P, _P, _I, _P, _I, _I, _I, _P]),
    "lq_fp8_gelu_cast_panels": (_I, [_P, _P, _P, _I, _Z, _Z, _P, _P, _P]),
    "lq_gemm_fp8_panels": (_I, [_P, _I, _P, _P, _P, _P, _P, _I, _I, _I, _P, _P]),
    "lq_lora_down": (_I, [_P, _I, _P, _P, _I, _I, _I, _I, _P]),
    "lq_w4a4_quantize_lora_down": (_I, [_P, _P, _I, _P, _I, _P, _I, _P, _P, _I, _I, _I, _I, _P]),
    "lq_rmsnorm_rope": (_I, [_P, _P, _P, _P, _P, _P, _Z, _I, _I, _I, _I, _I, _I, _F, _P]),
    "lq_cast_f32": (_I, [_P, _I, _P, _Z, _P]),
    "lq_load_lora": (_I, [_P, _P, _I, _Z, _F, _P]),
    "lq_gemm_set_tactic": (_I, [_I, _I]),
    "lq_gemm_set_thread_tactic": (_I, [_I]),
    "lq_gemm_tactics_serialized_size": (_Z, []),
    "lq_gemm_tactics_serialize": (_I, [_P, _Z, _P]),
    "lq_gemm_tactics_deserialize": (_I, [_P, _Z]),
    "lq_gemm_tactic_count": (_I, [_I]),
    "lq_gemm_set_shape_tactic": (_I, [_I, _I, _I, _I, _I]),
    "lq_gemm_get_shape_tactic": (_I, [_I, _I, _I, _I]),
    "lq_gemm_profile_workspace": (_Z, [_I, _I, _I, _I]),
    "lq_gemm_profile": (_I, [_I, _I, _I, _I, _P, _Z, C.POINTER(_I), C.POINTER(_F), _P]),
    "lq_shader_clock_probe": (_I, [_P, _I, C.c_uint, _P]),
    "lq_mfma_fp8_probe": (_I, [_P, _P, C.c_size_t, _I, _P, _P]),
}



class Epilogue(C.Structure):
    """lq_epilogue_t of include/lyraquant.h."""
    _fields_ = [("gelu", _I), ("addend", _P), ("gate", _P), ("rows_per_gate", _Z), ("residual", _P), ("C_fp8", _P),
                ("ldc_fp8", _Z), ("C_fp8_scale", _P)]


_lib = None


class LyraQuantError(RuntimeError):
    """Raised when an lq_* call returns a negative status (message from lq_last_error())."""


def load() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} not found: build it with `python -m lyradiff_amd.build` "
                "(hipcc, gfx950). There is no CPU fallback for the quantized-linear path.")
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def check(status: int, what: str) -> None:
    if status != 0:
        msg = load().lq_last_error().decode("utf-8", "replace")
        raise LyraQuantError(f"[lyradiff Error][{what}] status {status}: {msg}")
