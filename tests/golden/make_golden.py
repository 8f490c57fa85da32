"""Writes tests/golden/quant_golden.npz: small known-answer vectors for the quantized-linear path.

The lyraDiff reference ships no tests, golden vectors or fixtures for this path (its tests/
directory does not exist), so these vectors are derived here from first principles with exact
rational / integer arithmetic (fractions.Fraction, Python ints) and do NOT import the oracle:
they pin the oracle (tests/test_oracle_pins.py) and, through it, the HIP kernels.

    python tests/golden/make_golden.py
"""
from __future__ import annotations

import os
import struct
from fractions import Fraction

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def f32(x: float) -> float:
    return struct.unpack("f", struct.pack("f", x))[0]


def round_half_even(fr: Fraction) -> int:
    fl = fr.numerator // fr.denominator
    rem = fr - fl
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1):
        return fl + 1
    return fl


def rne_sat(fr: Fraction, lo: int, hi: int) -> int:
    return max(lo, min(hi, round_half_even(fr)))


def e4m3_value(code: int) -> Fraction | None:
    e, m = (code >> 3) & 0xF, code & 7
    if (code & 0x7F) == 0x7F:
        return None  # NaN
    v = Fraction(m, 8) * Fraction(1, 64) if e == 0 else (1 + Fraction(m, 8)) * Fraction(2) ** (e - 7)
    return -v if code & 0x80 else v


def e4m3_encode_exact(x: Fraction) -> int:
    """Nearest e4m3 value, ties to the even code, saturating at +-448 (brute force over 127 codes)."""
    sign = 0x80 if x < 0 else 0
    a = min(abs(x), Fraction(448))
    best, best_d = 0, None
    for c in range(0x7F):
        d = abs(e4m3_value(c) - a)
        if best_d is None or d < best_d or (d == best_d and c % 2 == 0 and best % 2 == 1):
            best, best_d = c, d
    return best | sign


def main():
    out = {}
    # 1. float_to_int8_rn: all half-integers and neighbours in [-131, 131]
    xs = [Fraction(n, 4) for n in range(-131 * 4, 131 * 4 + 1)]
    out["s8_in"] = np.array([float(x) for x in xs], np.float32)
    out["s8_out"] = np.array([rne_sat(x, -128, 127) for x in xs], np.int8)
    # 2. e4m3: decode table and exact encode of a grid of rationals (every 1/64 up to 2, then coarser)
    dec = np.array([float(e4m3_value(c)) if e4m3_value(c) is not None else np.nan for c in range(256)], np.float32)
    out["e4m3_decode"] = dec
    grid = [Fraction(n, 1024) for n in range(0, 2048)] + [Fraction(n, 16) for n in range(32, 8000, 7)] + [Fraction(10 ** 6)]
    grid = grid + [-g for g in grid]
    out["e4m3_in"] = np.array([float(g) for g in grid], np.float32)
    out["e4m3_out"] = np.array([e4m3_encode_exact(Fraction(f32(float(g)))) for g in grid], np.uint8)
    # 3. per-token INT8 quant of a tiny hand-checkable matrix: exact rationals, scale = amax/127 in fp32
    x = np.array([[1.0, -2.0, 0.5, 4.0, -0.25, 3.0, 0.0, 2.5],
                  [0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0],
                  [-127.0, 63.5, 1.0, -1.0, 126.0, 0.5, -0.5, 64.0]], np.float32)
    pre = np.array([1.0, 0.5, 2.0, 1.0, 4.0, 1.0, 1.0, 2.0], np.float32)
    q = np.zeros_like(x, dtype=np.int8)
    s = np.zeros(3, np.float32)
    for i in range(3):
        t = [Fraction(f32(float(x[i, j]) * float(pre[j]))) for j in range(8)]  # products are exact in fp32 here
        amax = max(abs(v) for v in t)
        if amax <= Fraction(1, 2 ** 24):
            s[i] = 1.0
            continue
        si = float(np.float32(float(amax)) / np.float32(127.0))  # one IEEE fp32 division
        s[i] = si
        for j in range(8):
            quo = Fraction(float(np.float32(float(t[j])) / np.float32(si)))  # IEEE fp32 division, then exact rounding
            q[i, j] = rne_sat(quo, -128, 127)
    out["sq_x"], out["sq_pre"], out["sq_q"], out["sq_scale"] = x, pre, q, s
    # 4. INT8 GEMM 4x8x16 with hand-checkable accumulators (Python ints)
    rng = np.random.RandomState(7)
    a = rng.randint(-128, 128, size=(4, 16)).astype(np.int8)
    w = rng.randint(-127, 128, size=(8, 16)).astype(np.int8)
    acc = np.array([[sum(int(a[i, k]) * int(w[j, k]) for k in range(16)) for j in range(8)] for i in range(4)], np.int32)
    out["gemm_a"], out["gemm_w"], out["gemm_acc"] = a, w, acc
    # 5. W4A4 packing: element i of a word sits in bits [4i, 4i+3], two's complement
    qv = np.array([[((i * 5 + r * 3) % 16) - 8 for i in range(64)] for r in range(8)], np.int8)
    words = np.zeros((8, 8), np.uint32)
    for r in range(8):
        for i in range(64):
            words[r, i // 8] |= np.uint32((int(qv[r, i]) & 0xF) << (4 * (i % 8)))
    out["w4_q"], out["w4_words"] = qv, words
    # the first word of row 0 spelled out: values -8,-3,2,7,-4,1,6,-5 -> nibbles 8,D,2,7,C,1,6,B -> 0xB61C72D8
    assert int(words[0, 0]) == 0xB61C72D8, hex(int(words[0, 0]))
    # 6. W4A4 group quant of one row with a power-of-two amax so that every quotient is exact
    xr = np.array([[0.25 * ((i % 15) - 7) for i in range(64)]], np.float32)  # amax = 1.75, scale = 1.75/7 = 0.25
    out["w4_x"], out["w4_scale"] = xr, np.array([[0.25]], np.float32)
    out["w4_xq"] = np.array([[(i % 15) - 7 for i in range(64)]], np.int8)
    # 7. rows32 repack: byte (n, k) -> index ((n//32 * K/16 + k//16) * 32 + n%32) * 16 + k%16
    n, kb = 64, 48
    src = np.arange(n * kb, dtype=np.uint32).reshape(n, kb)
    dst = np.zeros(n * kb, np.uint32)
    for r in range(n):
        for c in range(kb):
            dst[((r // 32 * (kb // 16) + c // 16) * 32 + r % 32) * 16 + c % 16] = src[r, c]
    out["rows32_src"], out["rows32_dst"] = (src % 251).astype(np.uint8), (dst % 251).astype(np.uint8)
    np.savez_compressed(os.path.join(HERE, "quant_golden.npz"), **out)
    print("wrote", os.path.join(HERE, "quant_golden.npz"), {k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main()
