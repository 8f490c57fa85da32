"""ctypes loader for the scalar C oracle (TEST INFRASTRUCTURE, NOT PRODUCT CODE).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this."""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_DIR = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_DIR, "liboracle_c.so")


def build(force: bool = False) -> str:
    src = os.path.join(_DIR, "oracle_c.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _DIR, "-B", "liboracle_c.so"], stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = C.CDLL(_SO)
        fp, ip, u8, u16, u32, i8, i32 = (C.c_void_p,) * 7
        L.oc_rne_sat_s8.restype = C.c_int8
        L.oc_rne_sat_s8.argtypes = [C.c_float]
        L.oc_bf16_to_f32.restype = C.c_float
        L.oc_bf16_to_f32.argtypes = [C.c_uint16]
        L.oc_f32_to_bf16.restype = C.c_uint16
        L.oc_f32_to_bf16.argtypes = [C.c_float]
        L.oc_f16_to_f32.restype = C.c_float
        L.oc_f16_to_f32.argtypes = [C.c_uint16]
        L.oc_f32_to_f16.restype = C.c_uint16
        L.oc_f32_to_f16.argtypes = [C.c_float]
        L.oc_tanh_f32.restype = C.c_float
        L.oc_tanh_f32.argtypes = [C.c_float]
        L.oc_e4m3_decode.restype = C.c_float
        L.oc_e4m3_decode.argtypes = [C.c_uint8]
        L.oc_e4m3_encode.restype = C.c_uint8
        L.oc_e4m3_encode.argtypes = [C.c_float]
        L.oc_fp8_scale.restype = C.c_float
        L.oc_fp8_scale.argtypes = [fp, C.c_size_t]
        L.oc_fp8_scale_cast.restype = None
        L.oc_fp8_scale_cast.argtypes = [u8, fp, C.c_float, C.c_int, C.c_size_t]
        L.oc_sq_input_quant.restype = None
        L.oc_sq_input_quant.argtypes = [i8, fp, fp, fp, C.c_int, C.c_int, C.c_int]
        L.oc_sq_dynamic_quant.restype = None
        L.oc_sq_dynamic_quant.argtypes = [i8, fp, fp, fp, C.c_int, C.c_int]
        L.oc_gemm_i8.restype = None
        L.oc_gemm_i8.argtypes = [i32, i8, i8, C.c_int, C.c_int, C.c_int]
        L.oc_int8_epilogue.restype = None
        L.oc_int8_epilogue.argtypes = [fp, i32, fp, fp, C.c_int, fp, C.c_int, C.c_int]
        L.oc_w4a4_quant.restype = None
        L.oc_w4a4_quant.argtypes = [u32, fp, fp, fp, C.c_int, C.c_int, C.c_int, C.c_int]
        L.oc_w4a4_gemm.restype = None
        L.oc_w4a4_gemm.argtypes = [fp, i32, u32, u32, fp, fp, fp] + [C.c_int] * 4
        _lib = L
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _f32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


def sq_input_quant(x, pre, scale, per_token):
    x, pre, scale = _f32(x), _f32(pre), _f32(scale)
    m, k = x.shape
    q = np.empty((m, k), np.int8)
    lib().oc_sq_input_quant(_p(q), _p(x), _p(pre), _p(scale), int(per_token), m, k)
    return q


def sq_dynamic_quant(x, pre):
    x, pre = _f32(x), _f32(pre)
    m, k = x.shape
    q = np.empty((m, k), np.int8)
    s = np.empty((m,), np.float32)
    lib().oc_sq_dynamic_quant(_p(q), _p(s), _p(x), _p(pre), m, k)
    return q, s


def gemm_i8(a, w):
    a = np.ascontiguousarray(a, np.int8)
    w = np.ascontiguousarray(w, np.int8)
    m, k = a.shape
    n = w.shape[0]
    acc = np.empty((m, n), np.int32)
    lib().oc_gemm_i8(_p(acc), _p(a), _p(w), m, n, k)
    return acc


def int8_epilogue(acc, alpha_col, alpha_row, bias=None):
    acc = np.ascontiguousarray(acc, np.int32)
    m, n = acc.shape
    ac, ar, b = _f32(alpha_col), _f32(np.reshape(alpha_row, -1)), _f32(bias)
    y = np.empty((m, n), np.float32)
    lib().oc_int8_epilogue(_p(y), _p(acc), _p(ac), _p(ar), int(ar.size > 1), _p(b), m, n)
    return y


def fp8_scale_cast(x, scale, invert=True):
    x = _f32(x)
    q = np.empty(x.shape, np.uint8)
    lib().oc_fp8_scale_cast(_p(q), _p(x), float(scale), int(invert), x.size)
    return q


def fp8_scale(x):
    x = _f32(x)
    return np.float32(lib().oc_fp8_scale(_p(x), x.size))


def w4a4_quant(x, smooth, group=64, f16_scale=False):
    x, smooth = _f32(x), _f32(smooth)
    m, k = x.shape
    words = np.empty((m, k // 8), np.uint32)
    scales = np.empty((m, k // group), np.float32)
    lib().oc_w4a4_quant(_p(words), _p(scales), _p(x), _p(smooth), m, k, group, int(f16_scale))
    return words, scales


def w4a4_gemm(qa, qb, sA, sB, bias=None, group=64, want_p=False):
    """fp32 result of the ascending-g fmaf chain (before the cast to bf16) and, optionally,
    the exact per-group int32 sums [M,N,G]."""
    qa = np.ascontiguousarray(qa, np.uint32)
    qb = np.ascontiguousarray(qb, np.uint32)
    m, k8 = qa.shape
    n = qb.shape[0]
    k = k8 * 8
    sA, sB, bias = _f32(sA), _f32(sB), _f32(bias)
    y = np.empty((m, n), np.float32)
    p = np.empty((m, n, k // group), np.int32) if want_p else None
    lib().oc_w4a4_gemm(_p(y), _p(p), _p(qa), _p(qb), _p(sA), _p(sB), _p(bias), m, n, k, group)
    return (y, p) if want_p else y
