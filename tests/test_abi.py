"""The C-ABI library loads, exports every symbol include/lyraquant.h declares, and rejects bad
arguments before touching the GPU (no compute calls here: this file runs on a CPU-only box)."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    txt = open(os.path.join(ROOT, "include", "lyraquant.h")).read()
    txt = re.sub(r"/\*.*?\*/", "", txt, flags=re.S)
    return sorted(set(re.findall(r"\b(lq_[a-z0-9_]+)\s*\(", txt)))


@pytest.fixture(scope="module")
def lib():
    from lyradiff_amd import lib as L

    if not os.path.exists(L.LIB_PATH):
        from lyradiff_amd import build

        build.build()
    return L.load()


def test_every_declared_symbol_is_exported(lib):
    from lyradiff_amd import lib as L

    names = declared_symbols()
    assert len(names) >= 19
    for n in names:
        assert hasattr(lib, n), f"{n} declared in lyraquant.h but not exported"
    assert set(names) == set(L.SYMBOLS), "ctypes table and header disagree"
    assert lib.lq_version() >= 100


def test_argument_errors_do_not_reach_the_gpu(lib):
    from lyradiff_amd import lib as L

    one = C.c_void_p(16)  # a non-null, 16-byte aligned dummy "pointer"; rejected calls never dereference it
    assert lib.lq_sq_input_quant(None, one, L.LQ_F16, None, one, 0, 4, 8, None) == -1
    assert b"null" in lib.lq_last_error()
    assert lib.lq_gemm_int8(one, L.LQ_F16, one, one, one, one, 1, None, 16, 33, 64, None) == -2
    assert b"n % 32" in lib.lq_last_error()
    assert lib.lq_gemm_fp8(one, L.LQ_BF16, one, one, one, one, None, 0, None, 0.0, 16, 64, 100, None) == -2
    assert lib.lq_gemm_w4a4(one, L.LQ_BF16, one, one, one, one, L.LQ_F32, None, 16, 64, 128, 32, None) == -2
    assert b"group" in lib.lq_last_error()
    assert lib.lq_w4a4_quantize(one, one, L.LQ_F32, one, L.LQ_BF16, None, 4, 100, 64, None) == -2
    assert lib.lq_w4a4_quantize(one, one, L.LQ_I32, one, L.LQ_BF16, None, 4, 128, 64, None) == -4
    assert lib.lq_repack_rows32(one, one, 64, 64, None) == -1  # in place
    assert lib.lq_repack_rows32(one, C.c_void_p(32), 33, 64, None) == -2
    assert lib.lq_geglu_int8(one, one, None, L.LQ_F16, None, one, 4, 12, None) == -2
    assert lib.lq_gemm_int8(one, 9, one, one, one, one, 0, None, 16, 32, 64, None) == -4
    # empty problems are no-ops
    assert lib.lq_sq_dynamic_quant(one, one, one, L.LQ_F16, None, 0, 64, None) == 0
    assert lib.lq_gemm_int8(one, L.LQ_F16, one, one, one, one, 0, None, 0, 32, 64, None) == 0
    assert lib.lq_weight_row_bytes(L.LQ_W_INT4, 3072) == 1536 and lib.lq_weight_row_bytes(L.LQ_W_FP8, 3072) == 3072


def test_wrapper_rejects_host_tensors():
    import torch

    from lyradiff_amd import ops

    with pytest.raises(ValueError):
        ops.sq_quant_dynamic(torch.zeros(4, 8, dtype=torch.float16), None)
    with pytest.raises(TypeError):
        ops.sq_quant_dynamic("x", None)


def test_shape_tactic_cache(lib):
    """The per-shape tactic cache is host logic: exact shape first, then m rounded up to a power of two."""
    from lyradiff_amd import lib as L

    k8, k4 = L.LQ_W_INT8, L.LQ_W_INT4
    assert lib.lq_gemm_tactic_count(k8) == 8 and lib.lq_gemm_tactic_count(L.LQ_W_FP8) == 8 and lib.lq_gemm_tactic_count(k4) == 3
    assert lib.lq_gemm_tactic_count(7) < 0
    assert lib.lq_gemm_get_shape_tactic(k8, 4096, 640, 2560) == -1
    assert lib.lq_gemm_set_shape_tactic(k8, 4096, 640, 2560, 2) == 0
    assert lib.lq_gemm_get_shape_tactic(k8, 4096, 640, 2560) == 2
    assert lib.lq_gemm_get_shape_tactic(k8, 3000, 640, 2560) == 2      # 3000 -> bucket 4096
    assert lib.lq_gemm_get_shape_tactic(k8, 2048, 640, 2560) == -1     # another bucket
    assert lib.lq_gemm_get_shape_tactic(k4, 4096, 640, 2560) == -1     # another GEMM
    assert lib.lq_gemm_set_shape_tactic(k8, 3000, 640, 2560, 4) == 0   # an exact entry wins over the bucket
    assert lib.lq_gemm_get_shape_tactic(k8, 3000, 640, 2560) == 4
    assert lib.lq_gemm_set_shape_tactic(k8, 4096, 640, 2560, lib.lq_gemm_tactic_count(k8)) == -1  # tactic out of range
    assert b"tactic" in lib.lq_last_error()
    assert lib.lq_gemm_set_shape_tactic(k8, 3000, 640, 2560, -1) == 0 and lib.lq_gemm_set_shape_tactic(k8, 4096, 640, 2560, -1) == 0
    assert lib.lq_gemm_get_shape_tactic(k8, 3000, 640, 2560) == -1
    # profiler argument checks (no GPU work is started)
    assert lib.lq_gemm_profile_workspace(k8, 1024, 1280, 1280) >= 1024 * 1280 * 2 + 1024 * 1280 * 2
    assert lib.lq_gemm_profile(k8, 1024, 1280, 1280, None, 0, None, None, None) == -1
    assert b"workspace" in lib.lq_last_error()


def test_tactic_cache_round_trips_through_bytes(lib):
    """lq_gemm_tactics_serialize / deserialize (the reference's GemmPluginProfiler::serialize / deserialize,
    layers/gemm_utils/GemmProfiler.cc:26-65): the table survives a round trip, a damaged or foreign table is refused whole."""
    import struct

    from lyradiff_amd import lib as L
    from lyradiff_amd import ops

    k8, kf = L.LQ_W_INT8, L.LQ_W_FP8
    shapes = [(k8, 4608, 12288, 3072, 7), (kf, 4608, 3072, 12288, 6), (kf, 6912, 9216, 3072, 4)]
    try:
        for kind, m, n, k, t in shapes:
            assert lib.lq_gemm_set_shape_tactic(kind, m, n, k, t) == 0
        blob = ops.gemm_tactics_dumps()
        assert blob[:4] == b"LQT1" and len(blob) == lib.lq_gemm_tactics_serialized_size() and (len(blob) - 8) % 20 == 0
        count = struct.unpack("<i", blob[4:8])[0]
        entries = {struct.unpack("<5i", blob[8 + 20 * i: 28 + 20 * i]) for i in range(count)}
        assert set(shapes) <= entries
        for kind, m, n, k, _ in shapes:
            assert lib.lq_gemm_set_shape_tactic(kind, m, n, k, -1) == 0 and lib.lq_gemm_get_shape_tactic(kind, m, n, k) == -1
        ops.gemm_tactics_loads(blob)
        for kind, m, n, k, t in shapes:
            assert lib.lq_gemm_get_shape_tactic(kind, m, n, k) == t
        # refused: wrong magic, truncated, a tactic number the kind does not have, a bad kind; nothing of a refused table is kept
        bad_tactic = blob[:8] + struct.pack("<5i", k8, 64, 64, 64, 99) + blob[28:]
        bad_kind = blob[:8] + struct.pack("<5i", 42, 64, 64, 64, 0) + blob[28:]
        for bad in (b"XXXX" + blob[4:], blob[:-4], bad_tactic, bad_kind, b""):
            with pytest.raises(Exception):
                ops.gemm_tactics_loads(bad)
        assert lib.lq_gemm_get_shape_tactic(k8, 64, 64, 64) == -1
        small = (C := __import__("ctypes")).create_string_buffer(4)
        assert lib.lq_gemm_tactics_serialize(small, 4, None) == -1 and b"needed" in lib.lq_last_error()
    finally:
        for kind, m, n, k, _ in shapes:
            lib.lq_gemm_set_shape_tactic(kind, m, n, k, -1)
