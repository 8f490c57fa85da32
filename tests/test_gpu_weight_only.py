"""GPU parity of the weight-only (W8A16 / W4A16) GEMM and its weight preparation, through the C ABI.

The preparation is a bijection of integer codes: compared bit for bit with the oracle's restatement of the layout.
The GEMM accumulates exact products (a 16-bit float times a small integer) in fp32 in an order of its own; it is
compared with the fp64 evaluation of the contract within 1e-2 relative / 2 fp16 ULP, plus a few fp32 ULPs of the sum of
the |terms| where the terms cancel."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from tests.helpers import TORCH_DT, assert_close_tol, rng_t, to_np_f32

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops(dev):
    from lyradiff_amd import ops as _ops

    return _ops


def _pack_n(q_kn):
    """[K, N] int8 codes in [-8, 7] -> [K, N/2] bytes, column 2j in the low nibble."""
    q = q_kn.astype(np.int16)
    return ((q[:, 0::2] & 0xF) | ((q[:, 1::2] & 0xF) << 4)).astype(np.uint8).view(np.int8)


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("k,n", [(64, 32), (192, 160), (3072, 1280)])
def test_repack_weight_only_layout(ops, dev, bits, k, n):
    rng = np.random.default_rng(k + n + bits)
    half = 1 << (bits - 1)
    q = rng.integers(-half, half, (k, n)).astype(np.int8)
    src = torch.from_numpy(q if bits == 8 else _pack_n(q)).to(dev)
    got = ops.repack_weight_only(src, "int8" if bits == 8 else "int4").cpu().numpy()
    want = O.repack_rows32(O.weight_only_prepared(q, bits))
    assert got.size == want.size and np.array_equal(got.reshape(-1), want.reshape(-1))


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("m,n,k,with_bias", [(256, 128, 64, True), (300, 160, 192, False), (1, 32, 128, True),
                                             (1024, 1280, 1280, True), (777, 3072, 512, True)])
def test_weight_only_gemm(ops, dev, dt, bits, m, n, k, with_bias):
    from lyradiff_amd.weights import symmetric_quantize_last_axis_of_batched_matrix as squant

    g = rng_t(m + n + k + bits)
    t = TORCH_DT[dt]
    w = (0.05 * torch.randn(k, n, generator=g)).to(t)
    x = torch.randn(m, k, generator=g).to(t)
    bias = (0.2 * torch.randn(n, generator=g)).to(t) if with_bias else None
    codes, scales = squant(w, bits)
    q_ref, s_ref = O.weight_only_quantize(to_np_f32(w), bits, dt)
    unpacked = codes.numpy() if bits == 8 else None
    if bits == 4:  # unpack along N for the comparison
        b = codes.numpy().view(np.uint8).astype(np.int16)
        lo, hi = b & 0xF, b >> 4
        unpacked = np.stack([np.where(lo > 7, lo - 16, lo), np.where(hi > 7, hi - 16, hi)], axis=-1).reshape(k, n).astype(np.int8)
    assert np.array_equal(unpacked, q_ref) and np.array_equal(to_np_f32(scales), s_ref)
    kind = "int8" if bits == 8 else "int4"
    wp = ops.repack_weight_only(codes.to(dev), kind)
    y = ops.weight_only_linear(x.to(dev), wp, scales.to(dev), bias.to(dev) if with_bias else None, kind)
    ref = O.weight_only_gemm_f64(to_np_f32(x), q_ref, s_ref, to_np_f32(bias) if with_bias else None, dt)
    floor = 4e-6 * (np.abs(to_np_f32(x)).astype(np.float64) @ np.abs(q_ref.astype(np.float64))) * s_ref.astype(np.float64)[None, :]
    if dt == "bf16":  # the output's own rounding: one bf16 ULP is 8 fp16 ULPs
        floor = floor + 2.0 ** -8 * np.abs(ref.astype(np.float64))
    assert_close_tol(to_np_f32(y), ref, f"weight-only {kind} {dt}", abs_floor=floor)


def _grouped_case(k, n, bits, group, dt, with_zeros, seed):
    """Random codes with group-wise scales of varied magnitude and (optionally) zero points, all values of T."""
    rng = np.random.default_rng(seed)
    half = 1 << (bits - 1)
    q = rng.integers(-half, half, (k, n)).astype(np.int8)
    t = TORCH_DT[dt]
    scales = torch.from_numpy((0.002 + 0.02 * rng.random((k // group, n))).astype(np.float32)).to(t)
    zeros = torch.from_numpy((0.05 * rng.standard_normal((k // group, n))).astype(np.float32)).to(t) if with_zeros else None
    return q, scales, zeros


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("with_zeros", [False, True])
@pytest.mark.parametrize("group", [64, 128])
def test_weight_only_grouped_dequantised_weights(ops, dev, dt, bits, with_zeros, group):
    """With the identity as activation every output is one dequantised weight (all other products are exact zeros), so the
    kernel's per-element arithmetic is visible: bit-exact against the reference's rounding sequence for fp16 (multiply, then
    add) and for the scale-only forms; for bf16 with zero points the kernel rounds the fp32 fused multiply-add to bf16, which
    differs from the single rounding by one bf16 step when the fp32 result falls on a bf16 midpoint (counted, < 1e-3)."""
    k, n = 256, 160
    q, scales, zeros = _grouped_case(k, n, bits, group, dt, with_zeros, 100 * bits + group + with_zeros)
    kind = "int8" if bits == 8 else "int4"
    wp = ops.repack_weight_only(torch.from_numpy(q if bits == 8 else _pack_n(q)).to(dev), kind)
    eye = torch.eye(k, dtype=TORCH_DT[dt]).to(dev)
    got = to_np_f32(ops.weight_only_linear_grouped(eye, wp, scales.to(dev), None if zeros is None else zeros.to(dev), None, kind, group))
    want = O.weight_only_dequant_grouped(q, to_np_f32(scales), None if zeros is None else to_np_f32(zeros), group, dt)
    if dt == "bf16" and with_zeros:
        diff = got != want
        assert diff.mean() < 1e-3 and np.all(np.abs(got - want)[diff] <= 2.0 ** -7 * np.abs(want)[diff])
    else:
        assert np.array_equal(got, want)


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("bits,with_zeros,group", [(8, False, 128), (8, True, 64), (4, True, 128), (4, False, 64)])
@pytest.mark.parametrize("m,n,k,with_bias", [(256, 128, 128, True), (300, 160, 384, False), (1, 32, 128, True),
                                             (1024, 1280, 1280, True), (777, 3072, 512, True)])
def test_weight_only_gemm_grouped(ops, dev, dt, bits, with_zeros, group, m, n, k, with_bias):
    g = rng_t(m + n + k + bits + group)
    t = TORCH_DT[dt]
    q, scales, zeros = _grouped_case(k, n, bits, group, dt, with_zeros, m + n + k)
    x = torch.randn(m, k, generator=g).to(t)
    bias = (0.2 * torch.randn(n, generator=g)).to(t) if with_bias else None
    kind = "int8" if bits == 8 else "int4"
    wp = ops.repack_weight_only(torch.from_numpy(q if bits == 8 else _pack_n(q)).to(dev), kind)
    y = ops.weight_only_linear_grouped(x.to(dev), wp, scales.to(dev), None if zeros is None else zeros.to(dev),
                                       None if bias is None else bias.to(dev), kind, group)
    zs = None if zeros is None else to_np_f32(zeros)
    ref = O.weight_only_gemm_grouped_f64(to_np_f32(x), q, to_np_f32(scales), zs, None if bias is None else to_np_f32(bias), group, dt)
    w = np.abs(O.weight_only_dequant_grouped(q, to_np_f32(scales), zs, group, dt)).astype(np.float64)
    ax = np.abs(to_np_f32(x)).astype(np.float64)
    floor = 4e-6 * (ax @ w)
    if dt == "bf16":  # the output's own rounding, and a weight that is one bf16 step off where the fp32 fma double-rounds
        floor = floor + 2.0 ** -8 * np.abs(ref.astype(np.float64)) + (2.0 ** -7 * ax.max(axis=1)[:, None] * w.max(axis=0)[None, :] if with_zeros else 0.0)
    assert_close_tol(to_np_f32(y), ref, f"weight-only grouped {kind} {dt} g{group} zeros={with_zeros}", abs_floor=floor)


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("bits,grouped,group", [(8, 0, 0), (4, 0, 0), (8, 1, 64), (4, 1, 128), (8, 2, 128), (4, 2, 64)])
@pytest.mark.parametrize("m,n,k", [(4096, 3072, 256), (4000, 3104, 384)])
def test_weight_only_gemm_256x256_tiles(ops, dev, dt, bits, grouped, group, m, n, k):
    """The 256x256 eight-wavefront three-stage kernels (picked from 192 such tiles up): per-channel, group-wise scale-only and
    scale + zero-point forms, int8 and int4, n a multiple of 256 and not, ragged m; against the fp64 contract, and bit for bit
    against the 256x128 configuration (same k order) forced through the thread tactic."""
    g = rng_t(m + n + k + bits + group)
    t = TORCH_DT[dt]
    kind = "int8" if bits == 8 else "int4"
    x = torch.randn(m, k, generator=g).to(t)
    bias = (0.2 * torch.randn(n, generator=g)).to(t)
    assert ((m + 255) // 256) * ((n + 255) // 256) >= 192
    if grouped == 0:
        rng = np.random.default_rng(m + bits)
        half = 1 << (bits - 1)
        q = rng.integers(-half, half, (k, n)).astype(np.int8)
        scales = torch.from_numpy((0.002 + 0.02 * rng.random(n)).astype(np.float32)).to(t)
        run = lambda wp: ops.weight_only_linear(x.to(dev), wp, scales.to(dev), bias.to(dev), kind)
        ref = O.weight_only_gemm_f64(to_np_f32(x), q, to_np_f32(scales), to_np_f32(bias), dt)
        w = np.abs(q.astype(np.float64)) * to_np_f32(scales).astype(np.float64)[None, :]
    else:
        q, scales, zeros = _grouped_case(k, n, bits, group, dt, grouped == 2, m + n + k)
        run = lambda wp: ops.weight_only_linear_grouped(x.to(dev), wp, scales.to(dev), None if zeros is None else zeros.to(dev),
                                                        bias.to(dev), kind, group)
        zs = None if zeros is None else to_np_f32(zeros)
        ref = O.weight_only_gemm_grouped_f64(to_np_f32(x), q, to_np_f32(scales), zs, to_np_f32(bias), group, dt)
        w = np.abs(O.weight_only_dequant_grouped(q, to_np_f32(scales), zs, group, dt)).astype(np.float64)
    wp = ops.repack_weight_only(torch.from_numpy(q if bits == 8 else _pack_n(q)).to(dev), kind)
    y = run(wp)  # built-in rule: 256x256
    with ops.gemm_thread_tactic(0):
        y0 = run(wp)
    with ops.gemm_thread_tactic(1):
        y1 = run(wp)
    assert torch.equal(y, y0), "the built-in rule did not pick the 256x256 configuration"
    assert torch.equal(y0, y1), "256x256 and 256x128 configurations differ"
    ax = np.abs(to_np_f32(x)).astype(np.float64)
    floor = 4e-6 * (ax @ w)
    if dt == "bf16":
        floor = floor + 2.0 ** -8 * np.abs(ref.astype(np.float64)) + (2.0 ** -7 * ax.max(axis=1)[:, None] * w.max(axis=0)[None, :] if grouped == 2 else 0.0)
    assert_close_tol(to_np_f32(y), ref, f"weight-only 256x256 {kind} {dt} grouped={grouped} g{group}", abs_floor=floor)
    with pytest.raises(Exception, match="unknown tile configuration"):
        with ops.gemm_thread_tactic(5):
            run(wp)


def test_weight_only_grouped_argument_checks(ops, dev):
    from lyradiff_amd.lib import LyraQuantError

    x = torch.zeros(8, 128, dtype=torch.float16, device=dev)
    w = torch.zeros(32, 128, dtype=torch.uint8, device=dev)
    with pytest.raises(ValueError, match="group_size"):
        ops.weight_only_linear_grouped(x, w, torch.ones(4, 32, dtype=torch.float16, device=dev), group_size=32)
    with pytest.raises(ValueError, match="shape mismatch"):
        ops.weight_only_linear_grouped(x, w, torch.ones(2, 32, dtype=torch.float16, device=dev), group_size=128)
    lib = __import__("lyradiff_amd.lib", fromlist=["load"]).load()
    s = torch.ones(1, 32, dtype=torch.float16, device=dev)
    c = torch.empty(8, 32, dtype=torch.float16, device=dev)
    rc = lib.lq_gemm_weight_only_grouped(c.data_ptr(), x.data_ptr(), 1, w.data_ptr(), 0, s.data_ptr(), None, None, 8, 32, 128, 96, None)
    assert rc < 0 and b"group_size must be 64 or 128" in lib.lq_last_error()
    assert LyraQuantError is not None


def test_weight_only_argument_checks(ops, dev):
    from lyradiff_amd.lib import LyraQuantError

    x = torch.zeros(8, 96, dtype=torch.float16, device=dev)  # k = 96 is not a multiple of 64
    w = torch.zeros(32, 96, dtype=torch.uint8, device=dev)
    s = torch.ones(32, dtype=torch.float16, device=dev)
    with pytest.raises(LyraQuantError, match="k %% 64|k % 64"):
        ops.weight_only_linear(x, w, s)
    with pytest.raises(TypeError):
        ops.weight_only_linear(x.float(), w, s)
