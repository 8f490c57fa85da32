"""GPU parity of the quantized GEMMs against the CPU oracle, through the C ABI.

int32 accumulators bit-exact; fp16/bf16/fp32 outputs of the INT8 and W4A4 paths bit-exact against
the oracle's fp32 formula (same operation order, no contraction); FP8 outputs within the stated
tolerance (1e-2 relative or 2 fp16 ULP) of an fp64 evaluation."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from oracle import oracle_c as OC
from tests.helpers import (TORCH_DT, assert_close_tol, check_fp8_against_instruction_model, check_fp8_gemm, rng_t,
                           to_np_f32)

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops(dev):
    from lyradiff_amd import ops as _ops

    return _ops


INT8_SHAPES = [(1024, 1280, 1280), (4096, 5120, 640), (4096, 640, 2560), (77, 96, 64), (300, 1280, 192),
               (1, 32, 64), (513, 3072, 3072)]


@pytest.mark.parametrize("m,n,k", INT8_SHAPES)
def test_int8_gemm_int32_exact(ops, dev, m, n, k):
    g = rng_t(m * 7 + n + k)
    a = torch.randint(-128, 128, (m, k), generator=g, dtype=torch.int8)
    w = torch.randint(-127, 128, (n, k), generator=g, dtype=torch.int8)
    wp = ops.repack_weight(w.to(dev))
    acc = ops.int8_linear(a.to(dev), wp, None, None, None, torch.int32)
    assert np.array_equal(acc.cpu().numpy(), O.gemm_i8_acc(a.numpy(), w.numpy()))


@pytest.mark.parametrize("dt", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("per_token", [True, False])
@pytest.mark.parametrize("with_bias", [True, False])
def test_int8_gemm_epilogue(ops, dev, dt, per_token, with_bias):
    m, n, k = 1024, 1280, 1280
    g = rng_t(42)
    a = torch.randint(-127, 128, (m, k), generator=g, dtype=torch.int8)
    w = torch.randint(-127, 128, (n, k), generator=g, dtype=torch.int8)
    ac = (torch.rand(n, generator=g) * 9e-3 + 1e-3).float()
    ar = (torch.rand(m if per_token else 1, generator=g) * 0.05 + 0.01).float()
    bias = (torch.randn(n, generator=g) * 0.02).to(TORCH_DT[dt]) if with_bias else None
    y = ops.int8_linear(a.to(dev), ops.repack_weight(w.to(dev)), ac.to(dev), ar.to(dev),
                        bias.to(dev) if with_bias else None, TORCH_DT[dt])
    acc = O.gemm_i8_acc(a.numpy(), w.numpy())
    ref = O.int8_epilogue(acc, ac.numpy(), ar.numpy(), to_np_f32(bias) if with_bias else None, dt)
    got = to_np_f32(y)
    assert_close_tol(got, ref, "int8 epilogue")
    assert np.array_equal(got, ref), "fused epilogue should reproduce the oracle's fp32 formula bit for bit"


FP8_SHAPES = [(512, 3072, 3072), (100, 256, 128), (33, 64, 64), (256, 12288, 3072), (640, 3072, 12288)]
FP8_SHARE = {}  # share of outputs outside the stated tolerance per case, printed by the last test of this group


def _fp8_operands(m, n, k, seed, nonneg=False):
    g = rng_t(seed)
    x = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(n, k, generator=g) * 0.02).bfloat16()
    if nonneg:
        x, w = x.abs(), w.abs()
    qa, sa = O.fp8_amax_cast(to_np_f32(x))
    qb, sb = O.fp8_amax_cast(to_np_f32(w))
    return qa, sa, qb, sb


def _fp8_run(ops, dev, qa, sa, qb, sb, bias, gelu, res, beta, out_dt):
    return ops.fp8_linear(torch.from_numpy(qa).to(dev), ops.repack_weight(torch.from_numpy(qb).to(dev)),
                          torch.tensor([sa], dtype=torch.float32, device=dev), torch.tensor([sb], dtype=torch.float32, device=dev),
                          None if bias is None else bias.to(dev), gelu, None if res is None else res.to(dev), beta, out_dt)


@pytest.mark.parametrize("m,n,k", FP8_SHAPES)
@pytest.mark.parametrize("dt", ["bf16", "f16"])
def test_fp8_gemm(ops, dev, m, n, k, dt):
    """Contract C = T((sa*sb) * sum_k a*b + bias) (utils/cublasMMWrapper.cc:1104-1274) in fp64, stated tolerance; the few
    outputs that cancel to near zero must stay inside the matrix instruction's own error bound, and their share is
    asserted small.  A band of rows is also compared with the instruction-level model, which nearly all outputs must
    reproduce bit for bit."""
    qa, sa, qb, sb = _fp8_operands(m, n, k, m + n + k)
    bias = (torch.randn(n, generator=rng_t(5)) * 0.1).to(TORCH_DT[dt])
    y = to_np_f32(_fp8_run(ops, dev, qa, sa, qb, sb, bias, False, None, 0.0, TORCH_DT[dt]))
    ref = O.fp8_gemm(qa, qb, sa, sb, to_np_f32(bias), False, None, 0.0, dt)
    FP8_SHARE[(m, n, k, dt)] = check_fp8_gemm(y, ref, qa, qb, sa, sb, dt, "fp8 gemm")
    rows = np.unique(np.linspace(0, m - 1, 6).astype(int))
    check_fp8_against_instruction_model(y[rows], qa[rows], qb, sa, sb, to_np_f32(bias), dt, "fp8 gemm vs instruction model")


@pytest.mark.parametrize("m,n,k", [(512, 3072, 3072), (256, 1024, 12288)])
def test_fp8_gemm_without_cancellation_meets_the_stated_tolerance_everywhere(ops, dev, m, n, k):
    """All operands non-negative: nothing cancels, so the stated tolerance must hold for every output with no allowance
    (the instruction's truncation costs at most 7 * 2^-13 of a group's largest product, i.e. < 1e-3 relative)."""
    qa, sa, qb, sb = _fp8_operands(m, n, k, 11 + k, nonneg=True)
    for dt in ("bf16", "f32"):
        y = to_np_f32(_fp8_run(ops, dev, qa, sa, qb, sb, None, False, None, 0.0, TORCH_DT[dt]))
        ref = O.fp8_gemm(qa, qb, sa, sb, None, False, None, 0.0, dt)
        assert_close_tol(y, ref, f"fp8 gemm, non-negative operands, {dt}")
    # in fp32 the deviation is visible and one-sided (truncation toward zero): below the exact sum, by less than 2^-10 of it
    exact = O.e4m3_decode(qa).astype(np.float64) @ O.e4m3_decode(qb).astype(np.float64).T * float(np.float32(sa) * np.float32(sb))
    rel = (y.astype(np.float64) - exact) / exact
    assert rel.max() <= 2.0 ** -22 and rel.min() >= -2.0 ** -10


def test_fp8_gemm_fp32_output_against_the_instruction_model(ops, dev):
    """fp32 output, unit scales: the raw accumulators.  They follow the instruction model to within a few fp32 units (the
    model's last stage is approximate), far inside the truncation error itself -- a missing product would be 2^10 times larger."""
    m, n, k = 96, 256, 3072
    qa, sa, qb, sb = _fp8_operands(m, n, k, 99)
    y = to_np_f32(_fp8_run(ops, dev, qa, 1.0, qb, 1.0, None, False, None, 0.0, torch.float32)).astype(np.float64)
    a, b = O.e4m3_decode(qa), O.e4m3_decode(qb)
    model = O.fp8_mfma_dot_model(a, b).astype(np.float64)
    exact = a.astype(np.float64) @ b.astype(np.float64).T
    bound = O.fp8_mfma_step_bound(a, b)
    assert (np.abs(y - exact) <= bound).all()
    assert (np.abs(y - model) <= 2e-3 * bound).all(), float((np.abs(y - model) / bound).max())
    assert (y == model).mean() >= 0.9
    # the model is not the exact sum: the hardware's truncation is really there, and the model predicts it
    assert (np.abs(model - exact) > 50 * np.abs(y - model).max()).mean() > 0.5


def test_fp8_matrix_instruction_single_step(ops, dev):
    """One v_mfma_f32_32x32x64_f8f6f4 per output (K = 64, unit scales, fp32 out) on the crafted and adversarial operands of
    tests/golden/record_mfma_fp8.py: the hardware must return what was recorded in tests/golden/mfma_fp8_recorded.npz,
    stay inside the error bound the GEMM tests allow (7 truncated products of 2^-13 per group of 8), and follow the
    instruction model (exactly on the crafted cases, almost everywhere at a 2^16 exponent spread)."""
    import importlib.util
    import os

    here = os.path.dirname(os.path.abspath(__file__))
    spec = importlib.util.spec_from_file_location("record_mfma_fp8", os.path.join(here, "golden", "record_mfma_fp8.py"))
    rec = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(rec)
    R = np.load(os.path.join(here, "golden", "mfma_fp8_recorded.npz"))
    worst = 0.0
    for name, (a, b) in rec.cases().items():
        y = to_np_f32(_fp8_run(ops, dev, O.e4m3_encode(a), 1.0, O.e4m3_encode(b), 1.0, None, False, None, 0.0, torch.float32))
        assert np.array_equal(y, R[name + "__y"]), f"{name}: differs from the recorded hardware output"
        exact = a.astype(np.float64) @ b.astype(np.float64).T
        bound = O.fp8_mfma_step_bound(a, b)
        err = np.abs(y.astype(np.float64) - exact)
        assert (err <= bound).all(), name
        worst = max(worst, float((err / np.maximum(bound, 1e-300)).max()))
        model = O.fp8_mfma_dot_model(a, b)
        if name.startswith("rand8") or name == "rand4_k128":
            assert (model == y).mean() >= 0.97 and (np.abs(model.astype(np.float64) - y) <= 1e-3 * bound).all(), name
        else:
            assert np.array_equal(model, y), name
    # the bound is not slack by orders of magnitude: some case uses a good part of it
    assert worst >= 0.25


def test_fp8_gemm_gelu_residual(ops, dev):
    m, n, k = 384, 512, 256
    g = rng_t(3)
    qa, sa, qb, sb = _fp8_operands(m, n, k, 3)
    bias = (torch.randn(n, generator=g) * 0.1).bfloat16()
    res = torch.randn(m, n, generator=g).bfloat16()
    y = to_np_f32(_fp8_run(ops, dev, qa, sa, qb, sb, bias, True, None, 0.0, torch.bfloat16))
    # + hardware exp2/rcp in the GELU (about 1e-6 absolute)
    FP8_SHARE[(m, n, k, "bf16+gelu")] = check_fp8_gemm(y, O.fp8_gemm(qa, qb, sa, sb, to_np_f32(bias), True, None, 0.0, "bf16"),
                                                       qa, qb, sa, sb, "bf16", "gelu", extra_abs=2e-6)
    y2 = to_np_f32(_fp8_run(ops, dev, qa, sa, qb, sb, bias, False, res, 0.5, torch.bfloat16))
    FP8_SHARE[(m, n, k, "bf16+residual")] = check_fp8_gemm(
        y2, O.fp8_gemm(qa, qb, sa, sb, to_np_f32(bias), False, to_np_f32(res), 0.5, "bf16"), qa, qb, sa, sb, "bf16", "residual")


def test_fp8_share_of_outputs_outside_the_stated_tolerance_is_reported():
    for key, share in sorted(FP8_SHARE.items(), key=str):
        print(f"fp8 gemm {key}: {share:.3e} of the outputs outside 1e-2 rel / 2 fp16 ULP (all inside the instruction bound)")
    assert all(v <= 3e-3 for v in FP8_SHARE.values())


W4_SHAPES = [(256, 256, 256), (130, 96, 128), (512, 1024, 3072)]


@pytest.mark.parametrize("m,n,k", W4_SHAPES)
@pytest.mark.parametrize("sdt", ["f32", "f16"])
def test_w4a4_gemm(ops, dev, m, n, k, sdt):
    g = rng_t(m + n + k)
    x = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(n, k, generator=g) * 0.02).bfloat16()
    bias = (torch.randn(n, generator=g) * 0.1).bfloat16()
    qa, sA = O.w4a4_quant(to_np_f32(x), None, 64, sdt)
    qb, sB = O.w4a4_quant(to_np_f32(w), None, 64, sdt)
    wp = ops.repack_weight(torch.from_numpy(qb.view(np.uint8).reshape(n, k // 2)).to(dev))
    sdt_t = TORCH_DT[sdt]
    y = ops.w4a4_linear(torch.from_numpy(qa.view(np.int32)).to(dev), wp, torch.from_numpy(sA).to(sdt_t).to(dev),
                        torch.from_numpy(sB).to(sdt_t).to(dev), bias.to(dev), torch.bfloat16)
    ref32 = OC.w4a4_gemm(qa, qb, sA, sB, to_np_f32(bias))  # ascending-g fmaf chain, fp32
    ref = O.round_to(ref32, "bf16")
    got = to_np_f32(y)
    assert_close_tol(got, ref, "w4a4 gemm")
    assert np.array_equal(got, ref), "group accumulation order should match the oracle bit for bit"
    # fp32 output exposes the accumulation itself
    y32 = ops.w4a4_linear(torch.from_numpy(qa.view(np.int32)).to(dev), wp, torch.from_numpy(sA).to(sdt_t).to(dev),
                          torch.from_numpy(sB).to(sdt_t).to(dev), None, torch.float32)
    assert np.array_equal(y32.cpu().numpy(), OC.w4a4_gemm(qa, qb, sA, sB, None))


# ---- every tile configuration, forced one by one, against the same oracle -------------------------------------------
N_TACTICS = {"int8": 8, "fp8": 8, "int4": 3}


@pytest.fixture
def tactic_guard(ops):
    yield
    for kind in N_TACTICS:
        ops.gemm_set_tactic(kind, -1)


@pytest.mark.parametrize("tactic", range(N_TACTICS["int8"]))
@pytest.mark.parametrize("k", [704, 768])  # 704: a multiple of 64 only, the 128-byte k-tile configuration falls back
def test_int8_gemm_every_tactic(ops, dev, tactic, k, tactic_guard):
    m, n = 333, 416  # ragged M, N a multiple of 32 only
    g = rng_t(900 + tactic)
    a = torch.randint(-128, 128, (m, k), generator=g, dtype=torch.int8)
    w = torch.randint(-127, 128, (n, k), generator=g, dtype=torch.int8)
    ac = (torch.rand(n, generator=g) * 9e-3 + 1e-3).float()
    ar = (torch.rand(m, generator=g) * 0.05 + 0.01).float()
    bias = (torch.randn(n, generator=g) * 0.02).half()
    ops.gemm_set_tactic("int8", tactic)
    wp = ops.repack_weight(w.to(dev))
    acc = ops.int8_linear(a.to(dev), wp, None, None, None, torch.int32)
    y = ops.int8_linear(a.to(dev), wp, ac.to(dev), ar.to(dev), bias.to(dev), torch.float16)
    ref_acc = O.gemm_i8_acc(a.numpy(), w.numpy())
    assert np.array_equal(acc.cpu().numpy(), ref_acc)
    assert np.array_equal(to_np_f32(y), O.int8_epilogue(ref_acc, ac.numpy(), ar.numpy(), to_np_f32(bias), "f16"))


@pytest.mark.parametrize("tactic", range(N_TACTICS["int8"]))
@pytest.mark.parametrize("k", [64, 128, 192, 320])
def test_int8_gemm_fewer_k_tiles_than_pipeline_stages(ops, dev, tactic, k, tactic_guard):
    """One to five k-tiles: the pipelines of three and four stages start, re-fetch past the end and drain correctly
    when the loop is shorter than they are deep (exact int32 sums)."""
    m, n = 300, 288
    g = rng_t(1700 + 10 * tactic + k)
    a = torch.randint(-128, 128, (m, k), generator=g, dtype=torch.int8)
    w = torch.randint(-127, 128, (n, k), generator=g, dtype=torch.int8)
    ops.gemm_set_tactic("int8", tactic)
    acc = ops.int8_linear(a.to(dev), ops.repack_weight(w.to(dev)), None, None, None, torch.int32)
    assert np.array_equal(acc.cpu().numpy(), O.gemm_i8_acc(a.numpy(), w.numpy()))


@pytest.mark.parametrize("tactic", range(N_TACTICS["fp8"]))
@pytest.mark.parametrize("k", [704, 768])
def test_fp8_gemm_every_tactic(ops, dev, tactic, k, tactic_guard):
    m, n = 333, 416
    g = rng_t(950 + tactic)
    qa, sa = O.fp8_amax_cast(to_np_f32(torch.randn(m, k, generator=g).bfloat16()))
    qb, sb = O.fp8_amax_cast(to_np_f32((torch.randn(n, k, generator=g) * 0.02).bfloat16()))
    bias = (torch.randn(n, generator=g) * 0.1).bfloat16()
    ops.gemm_set_tactic("fp8", tactic)
    y = ops.fp8_linear(torch.from_numpy(qa).to(dev), ops.repack_weight(torch.from_numpy(qb).to(dev)),
                       torch.tensor([sa], dtype=torch.float32, device=dev), torch.tensor([sb], dtype=torch.float32, device=dev),
                       bias.to(dev), False, None, 0.0, torch.bfloat16)
    y = to_np_f32(y)
    check_fp8_gemm(y, O.fp8_gemm(qa, qb, sa, sb, to_np_f32(bias), False, None, 0.0, "bf16"), qa, qb, sa, sb, "bf16", "fp8 tactic")
    rows = np.arange(0, m, 37)  # every tactic walks k in the same order, so each reproduces the instruction model
    check_fp8_against_instruction_model(y[rows], qa[rows], qb, sa, sb, to_np_f32(bias), "bf16", f"fp8 tactic {tactic}")


@pytest.mark.parametrize("kind", ["int8", "fp8"])
@pytest.mark.parametrize("m,n,k", [(512, 1024, 256),     # 8 tiles: fewer than CUs, one round, four k-tiles (two per buffer parity)
                                   (4608, 12288, 128),   # 864 tiles: three rounds on 256 CUs and 96 left over, cut into 192 halves
                                   (4864, 14336, 384),   # 1064 tiles: four rounds and 40 left over (80 halves)
                                   (6912, 9216, 256),    # 972 tiles: 204 left over, more than half a round: whole tiles
                                   (4608, 12288 + 256, 128)])  # 882 tiles: 114 left over, not a multiple of 8: whole tiles
def test_persistent_gemm(ops, dev, kind, m, n, k, tactic_guard):
    """Tactic 7, the persistent one-wavefront-per-SIMD kernel: every tile count class (fewer tiles than CUs, leftover tiles
    cut into halves, leftover tiles kept whole) gives the bits of tactic 4, whose results the other tests pin to the oracle (all
    tactics walk k in the same order); one 256-row band of the big outputs is compared with the oracle directly."""
    g = rng_t(m + n + k)
    rows = slice(m - 256, m)  # the last band: a half tile where the last round is split
    if kind == "int8":
        a = torch.randint(-128, 128, (m, k), generator=g, dtype=torch.int8)
        w = torch.randint(-127, 128, (n, k), generator=g, dtype=torch.int8)
        ac = (torch.rand(n, generator=g) * 9e-3 + 1e-3).float()
        ar = (torch.rand(m, generator=g) * 0.05 + 0.01).float()
        bias = (torch.randn(n, generator=g) * 0.02).half()
        wp = ops.repack_weight(w.to(dev))
        run = lambda: ops.int8_linear(a.to(dev), wp, ac.to(dev), ar.to(dev), bias.to(dev), torch.float16)
        ref = O.int8_epilogue(O.gemm_i8_acc(a[rows].numpy(), w.numpy()), ac.numpy(), ar[rows].numpy(), to_np_f32(bias), "f16")
    else:
        qa, sa = O.fp8_amax_cast(to_np_f32(torch.randn(m, k, generator=g).bfloat16()))
        qb, sb = O.fp8_amax_cast(to_np_f32((torch.randn(n, k, generator=g) * 0.02).bfloat16()))
        bias = (torch.randn(n, generator=g) * 0.1).bfloat16()
        wp = ops.repack_weight(torch.from_numpy(qb).to(dev))
        sad, sbd = torch.tensor([sa], dtype=torch.float32, device=dev), torch.tensor([sb], dtype=torch.float32, device=dev)
        run = lambda: ops.fp8_linear(torch.from_numpy(qa).to(dev), wp, sad, sbd, bias.to(dev), False, None, 0.0, torch.bfloat16)
        ref = None
    ops.gemm_set_tactic(kind, 4)
    want = run()
    ops.gemm_set_tactic(kind, 7)
    got = run()
    again = run()
    assert torch.equal(got, want) and torch.equal(again, want)
    if kind == "int8":
        assert np.array_equal(to_np_f32(got[rows]), ref)
    else:
        y = to_np_f32(got[rows])
        check_fp8_gemm(y, O.fp8_gemm(qa[rows], qb, sa, sb, to_np_f32(bias), False, None, 0.0, "bf16"), qa[rows], qb, sa, sb, "bf16", "fp8 persistent")
    ops.gemm_set_tactic(kind, -1)
    if k > 1024:
        assert torch.equal(run(), want)  # the built-in table takes the same kernel for these shapes


@pytest.mark.parametrize("tactic", range(N_TACTICS["int4"]))
@pytest.mark.parametrize("sdt", ["f32", "f16"])
def test_w4a4_gemm_every_tactic(ops, dev, tactic, sdt, tactic_guard):
    m, n, k = 333, 416, 640
    g = rng_t(1000 + tactic)
    x = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(n, k, generator=g) * 0.02).bfloat16()
    qa, sA = O.w4a4_quant(to_np_f32(x), None, 64, sdt)
    qb, sB = O.w4a4_quant(to_np_f32(w), None, 64, sdt)
    sdt_t = TORCH_DT[sdt]
    ops.gemm_set_tactic("int4", tactic)
    for kk in (k, 128):  # 128: a single k-tile
        y32 = ops.w4a4_linear(torch.from_numpy(np.ascontiguousarray(qa[:, :kk // 8]).view(np.int32)).to(dev),
                              ops.repack_weight(torch.from_numpy(np.ascontiguousarray(qb[:, :kk // 8]).view(np.uint8).reshape(n, kk // 2)).to(dev)),
                              torch.from_numpy(np.ascontiguousarray(sA[:, :kk // 64])).to(sdt_t).to(dev),
                              torch.from_numpy(np.ascontiguousarray(sB[:, :kk // 64])).to(sdt_t).to(dev), None, torch.float32)
        ref = OC.w4a4_gemm(np.ascontiguousarray(qa[:, :kk // 8]), np.ascontiguousarray(qb[:, :kk // 8]),
                           np.ascontiguousarray(sA[:, :kk // 64]), np.ascontiguousarray(sB[:, :kk // 64]), None)
        assert np.array_equal(y32.cpu().numpy(), ref), f"k={kk}"


def test_matrix_pipe_probe_runs_and_reports_its_work(ops, dev):
    """lq_mfma_fp8_probe: measurement aid; the launch completes and the FLOP count follows the CU count."""
    import torch

    codes = torch.randint(0, 120, (1 << 16,), dtype=torch.uint8, device=dev)
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    for c in (codes, None):
        flop = ops.mfma_fp8_probe(c, 8)
        torch.cuda.synchronize()
        assert flop == 2.0 * 32 * 32 * 64 * 16 * 8 * 4 * cus
    with pytest.raises(Exception):
        ops.mfma_fp8_probe(codes, 0)


def test_profiler_fills_the_shape_cache(ops, dev, tactic_guard):
    """lq_gemm_profile picks a valid configuration, later calls of that shape use it, results stay exact."""
    m, n, k = 1000, 1280, 1280
    try:
        for kind in ("int8", "fp8", "int4"):
            assert ops.gemm_shape_tactic(kind, m, n, k) == -1
            best, us = ops.gemm_profile(kind, m, n, k, dev)
            assert 0 <= best < ops.gemm_tactic_count(kind) and 0.5 < us < 5000.0, (kind, best, us)
            assert ops.gemm_shape_tactic(kind, m, n, k) == best
        g = rng_t(77)
        a = torch.randint(-128, 128, (m, k), generator=g, dtype=torch.int8)
        w = torch.randint(-127, 128, (n, k), generator=g, dtype=torch.int8)
        acc = ops.int8_linear(a.to(dev), ops.repack_weight(w.to(dev)), None, None, None, torch.int32)
        assert np.array_equal(acc.cpu().numpy(), O.gemm_i8_acc(a.numpy(), w.numpy()))
    finally:
        for kind in ("int8", "fp8", "int4"):
            ops.gemm_shape_tactic(kind, m, n, k, -1)


# ---- W4A4 low-rank branch ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dt", ["bf16", "f16"])
# rows per workgroup follow m: 8 (m = 5, 70, 300), 18 (4608), 27 (6912), 32 with a ragged last workgroup (9000)
@pytest.mark.parametrize("m,k,rank", [(300, 3072, 32), (4608, 3072, 32), (70, 256, 64), (5, 64, 32), (6912, 3072, 32), (9000, 1024, 64)])
def test_lora_down(ops, dev, dt, m, k, rank):
    g = rng_t(m + k + rank)
    x = torch.randn(m, k, generator=g).to(TORCH_DT[dt])
    down = (torch.randn(rank, k, generator=g) * 0.05).to(TORCH_DT[dt])
    ref = O.lora_down_f64(to_np_f32(x), to_np_f32(down))
    mag = np.abs(to_np_f32(x)).astype(np.float64) @ np.abs(to_np_f32(down)).astype(np.float64).T
    y32 = ops.lora_down(x.to(dev), down.to(dev), torch.float32).cpu().numpy()
    assert np.all(np.abs(y32 - ref) <= 2.0 ** -20 * mag + 1e-30), "fp32 accumulation error beyond a few ULP of the term magnitudes"
    y = ops.lora_down(x.to(dev), down.to(dev))
    assert_close_tol(to_np_f32(y), O.round_to(ref.astype(np.float32), dt), "lora down", abs_floor=2.0 ** -20 * mag)
    assert torch.equal(ops.lora_down(x.to(dev), down.to(dev)), y), "no atomics: repeated calls agree bit for bit"


# One pass over x for both halves of invokeFusedQuantizeAndLoraDownSimple (kernels/w4a4_gemm/w4a4_gemm.h:6-16): words and scales are
# the bits of the stand-alone quantiser (and so of the oracle), the low-rank result meets the stand-alone kernel's error bound.
# Rows per workgroup follow m: 4 (m = 5, 70, 300), 18 (4608), 27 (6912), 32 with a ragged last workgroup (9000); k = 128 gives
# seven of the eight wavefronts no slice at all, k = 1152 an uneven share; the last two cases take the two-kernel route inside the
# call (rank 64; k not a multiple of 128).
@pytest.mark.parametrize("dt,sdt", [("bf16", "f32"), ("f16", "f32"), ("bf16", "f16")])
@pytest.mark.parametrize("m,k,rank", [(300, 3072, 32), (4608, 3072, 32), (70, 128, 32), (5, 1152, 32), (6912, 3072, 32), (9000, 1024, 32),
                                      (1024, 12288, 32), (70, 256, 64), (33, 192, 32)])
def test_w4a4_quant_and_lora_down_in_one_pass(ops, dev, dt, sdt, m, k, rank):
    g = rng_t(m + k + rank + 1)
    x = (torch.randn(m, k, generator=g) * (1.0 + 4.0 * torch.rand(m, 1, generator=g))).to(TORCH_DT[dt])
    x[m // 2, : min(k, 192)] = 0  # all-zero groups
    smooth = (0.25 + 2.0 * torch.rand(k, generator=g)).float()
    down = (torch.randn(rank, k, generator=g) * 0.05).to(TORCH_DT[dt])
    sdtype = torch.float32 if sdt == "f32" else torch.float16
    xd, sd, dd = x.to(dev), smooth.to(dev), down.to(dev)
    q, s, act32 = ops.w4a4_quant_lora_down(xd, sd, dd, sdtype, torch.float32)
    q0, s0 = ops.w4a4_quant(xd, sd, sdtype)
    assert torch.equal(q, q0) and torch.equal(s.view(torch.int16 if sdt == "f16" else torch.int32),
                                              s0.view(torch.int16 if sdt == "f16" else torch.int32)), "words and scales: the stand-alone quantiser's bits"
    if m * k <= 300 * 3072:  # and the oracle's, where it finishes quickly
        qo, so = O.w4a4_quant(to_np_f32(x), smooth.numpy(), 64, sdt)
        assert np.array_equal(q.cpu().numpy().view(np.uint32), qo)
        assert np.array_equal(s.float().cpu().numpy(), so.astype(np.float32))
    ref = O.lora_down_f64(to_np_f32(x), to_np_f32(down))
    mag = np.abs(to_np_f32(x)).astype(np.float64) @ np.abs(to_np_f32(down)).astype(np.float64).T
    assert np.all(np.abs(act32.cpu().numpy() - ref) <= 2.0 ** -20 * mag + 1e-30), "fp32 accumulation error beyond a few ULP of the term magnitudes"
    q1, s1, act = ops.w4a4_quant_lora_down(xd, sd, dd, sdtype)
    assert act.dtype == x.dtype and torch.equal(q1, q0)
    assert_close_tol(to_np_f32(act), O.round_to(ref.astype(np.float32), dt), "low-rank result", abs_floor=2.0 ** -20 * mag)
    q2, s2, act2 = ops.w4a4_quant_lora_down(xd, sd, dd, sdtype)
    assert torch.equal(act2, act) and torch.equal(q2, q1) and torch.equal(s2, s1), "no atomics: repeated calls agree bit for bit"


def test_w4a4_quant_and_lora_down_argument_checks(ops, dev):
    x = torch.zeros(8, 128, dtype=torch.bfloat16, device=dev)
    with pytest.raises(ValueError):
        ops.w4a4_quant_lora_down(x, None, torch.zeros(32, 64, dtype=torch.bfloat16, device=dev))
    with pytest.raises(RuntimeError):  # rank 16: neither route takes it
        ops.w4a4_quant_lora_down(x, None, torch.zeros(16, 128, dtype=torch.bfloat16, device=dev))
    q, s, act = ops.w4a4_quant_lora_down(x[:0], None, torch.zeros(32, 128, dtype=torch.bfloat16, device=dev))
    assert q.shape == (0, 16) and act.shape == (0, 32)


@pytest.mark.parametrize("sdt", ["f32", "f16"])
@pytest.mark.parametrize("m,n,k,rank,tactic", [(333, 416, 640, 32, 0), (333, 416, 640, 32, 1), (333, 416, 640, 16, 2), (512, 3072, 3072, 32, -1)])
def test_w4a4_gemm_with_low_rank_branch(ops, dev, sdt, m, n, k, rank, tactic, tactic_guard):
    g = rng_t(m + n + k + rank)
    x = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(n, k, generator=g) * 0.02).bfloat16()
    bias = (torch.randn(n, generator=g) * 0.1).bfloat16()
    act = (torch.randn(m, rank, generator=g) * 0.3).bfloat16()
    up = (torch.randn(n, rank, generator=g) * 0.3).bfloat16()
    qa, sA = O.w4a4_quant(to_np_f32(x), None, 64, sdt)
    qb, sB = O.w4a4_quant(to_np_f32(w), None, 64, sdt)
    sdt_t = TORCH_DT[sdt]
    ops.gemm_set_tactic("int4", tactic)
    args = (torch.from_numpy(qa.view(np.int32)).to(dev), ops.repack_weight(torch.from_numpy(qb.view(np.uint8).reshape(n, k // 2)).to(dev)),
            torch.from_numpy(sA).to(sdt_t).to(dev), torch.from_numpy(sB).to(sdt_t).to(dev))
    y = ops.w4a4_linear(*args, bias.to(dev), torch.bfloat16, 64, act.to(dev), up.to(dev))
    y32 = OC.w4a4_gemm(qa, qb, sA, sB, None)
    ref = O.w4a4_gemm_lora_f64(y32, to_np_f32(act), to_np_f32(up), to_np_f32(bias), "bf16")
    mag = np.abs(y32).astype(np.float64) + np.abs(to_np_f32(act)).astype(np.float64) @ np.abs(to_np_f32(up)).astype(np.float64).T
    assert_close_tol(to_np_f32(y), ref, "w4a4 + low rank", abs_floor=2.0 ** -20 * mag)
    # without the branch the result is still the bit-exact one
    y0 = ops.w4a4_linear(*args, None, torch.float32)
    assert np.array_equal(y0.cpu().numpy(), y32)
    # fp16 operands take the fp16 matrix instruction
    yh = ops.w4a4_linear(*args, None, torch.float32, 64, act.half().to(dev), up.half().to(dev))
    refh = y32.astype(np.float64) + to_np_f32(act.half()).astype(np.float64) @ to_np_f32(up.half()).astype(np.float64).T
    assert np.all(np.abs(yh.cpu().numpy() - refh) <= 2.0 ** -20 * mag + 1e-6 * np.abs(refh))


# ---- random shapes ---------------------------------------------------------------------------------------------------
def test_random_shapes_all_gemms(ops, dev):
    """Forty random (M, N, K) with every alignment the API allows (M free, N % 32, K % 64 or % 128): the default tile
    choice must be exact on all of them."""
    rs = np.random.default_rng(2024)
    for it in range(40):
        m = int(rs.integers(1, 700))
        n = 32 * int(rs.integers(1, 24))
        k = 64 * int(rs.integers(1, 20))
        g = rng_t(it)
        a = torch.randint(-128, 128, (m, k), generator=g, dtype=torch.int8)
        w = torch.randint(-127, 128, (n, k), generator=g, dtype=torch.int8)
        acc = ops.int8_linear(a.to(dev), ops.repack_weight(w.to(dev)), None, None, None, torch.int32)
        assert np.array_equal(acc.cpu().numpy(), O.gemm_i8_acc(a.numpy(), w.numpy())), ("int8", m, n, k)
        k4 = 128 * int(rs.integers(1, 8))
        x = torch.randn(m, k4, generator=g).bfloat16()
        wt = (torch.randn(n, k4, generator=g) * 0.05).bfloat16()
        sdt = "f16" if it % 2 else "f32"
        qa, sA = O.w4a4_quant(to_np_f32(x), None, 64, sdt)
        qb, sB = O.w4a4_quant(to_np_f32(wt), None, 64, sdt)
        y = ops.w4a4_linear(torch.from_numpy(qa.view(np.int32)).to(dev),
                            ops.repack_weight(torch.from_numpy(qb.view(np.uint8).reshape(n, k4 // 2)).to(dev)),
                            torch.from_numpy(sA).to(TORCH_DT[sdt]).to(dev), torch.from_numpy(sB).to(TORCH_DT[sdt]).to(dev), None, torch.float32)
        assert np.array_equal(y.cpu().numpy(), OC.w4a4_gemm(qa, qb, sA, sB, None)), ("w4a4", m, n, k4, sdt)
        qf, sf = O.fp8_amax_cast(to_np_f32(x))
        qw, sw = O.fp8_amax_cast(to_np_f32(wt))
        yf = ops.fp8_linear(torch.from_numpy(qf).to(dev), ops.repack_weight(torch.from_numpy(qw).to(dev)),
                            torch.tensor([sf], dtype=torch.float32, device=dev), torch.tensor([sw], dtype=torch.float32, device=dev),
                            None, False, None, 0.0, torch.float32)
        check_fp8_gemm(yf.cpu().numpy(), O.fp8_gemm(qf, qw, sf, sw, None, False, None, 0.0, "f32"), qf, qw, sf, sw, "f32",
                       f"fp8 {m}x{n}x{k4}", max_share_outside=2e-2)  # tiny K: a larger share of sums cancels


# ---- GEMM that leaves its largest output, then activation + dynamic quantisation in one pass -----------------------------
@pytest.mark.parametrize("dt", ["bf16", "f16"])
def test_gelu_of_a_stored_tensor_is_monotone_from_zero_up_and_bounded_below_it(ops, dev, dt):
    """What fp8_gelu_quant's scale rests on, value by value over every finite number of T: h = T(gelu(y)) never decreases as y
    grows from 0, and no negative y gives |h| above the bound the kernel falls back to.  h itself against the oracle's GELU."""
    t = TORCH_DT[dt]
    bits = torch.arange(0, 1 << 16, dtype=torch.int32).to(torch.int16)
    y = bits.view(t)
    y = y[torch.isfinite(y.float())]
    big = torch.full((1,), 1e30, dtype=torch.float32, device=dev)
    _, _, h = ops.fp8_gelu_quant(y.to(dev), big, want_h=True)
    yf, hf = y.float().numpy(), h.float().cpu().numpy()
    order = np.argsort(yf, kind="stable")
    yf, hf = yf[order], hf[order]
    pos = yf >= 0
    assert np.all(np.diff(hf[pos]) >= 0), "T(gelu(y)) decreases somewhere on y >= 0"
    assert np.abs(hf[~pos]).max() <= 0.171875 < hf[pos][np.searchsorted(yf[pos], 0.5)]
    ref = O.round_to(O.gelu_tanh_f32(yf), dt)
    fin = np.abs(yf) < 1e4  # beyond that the oracle's x^3 overflows to inf - inf
    assert_close_tol(hf[fin], ref[fin], "gelu of a stored tensor")


@pytest.mark.parametrize("dt", ["bf16", "f16"])
# the first three run the persistent kernel (whole 256x256 tiles, k % 128 == 0), with and without a round of half tiles; the
# last two the two-workgroups-per-CU kernels, ragged edges included
@pytest.mark.parametrize("m,n,k", [(512, 1024, 256), (4608, 12288, 128), (6912, 9216, 256), (333, 416, 704), (1024, 3072, 192)])
def test_fp8_linear_max_then_gelu_quant(ops, dev, m, n, k, dt):
    """C and its running maximum, then h = T(gelu(C)) quantised with the scale derived from that maximum: the same codes
    and scale as the amax + cast kernels give on h (checked against the oracle in test_gpu_quant.py)."""
    g = rng_t(m + n + k + 3)
    t = TORCH_DT[dt]
    qa, sa = ops.fp8_quant(torch.randn(m, k, generator=g).to(t).to(dev))
    qw, sw = ops.fp8_quant((torch.randn(n, k, generator=g) * 0.05).to(t).to(dev))
    wp = ops.repack_weight(qw)
    bias = (torch.randn(n, generator=g) * 0.1).to(t).to(dev)
    ymax = torch.zeros(1, dtype=torch.float32, device=dev)
    c = ops.fp8_linear_max(qa, wp, sa, sw, bias, ymax, t)
    ref = O.fp8_gemm(qa.cpu().numpy(), qw.cpu().numpy(), sa.item(), sw.item(), to_np_f32(bias.cpu()), False, None, 0.0, dt)
    check_fp8_gemm(to_np_f32(c.cpu()), ref, qa.cpu().numpy(), qw.cpu().numpy(), sa.item(), sw.item(), dt, "fp8 gemm with running maximum")
    assert ymax.item() == max(c.float().max().item(), 0.0) and ymax.item() >= 0.5
    # accumulation semantics: a larger value already in the slot wins
    big = torch.full((1,), 1e6, dtype=torch.float32, device=dev)
    assert torch.equal(ops.fp8_linear_max(qa, wp, sa, sw, bias, big, t), c) and big.item() == 1e6
    q, s, h = ops.fp8_gelu_quant(c, ymax, want_h=True)
    q_ref, s_ref = ops.fp8_quant(h)
    assert torch.equal(s, s_ref) and torch.equal(q, q_ref)
    nxt = torch.full((1,), 7.0, dtype=torch.float32, device=dev)
    q2, s2 = ops.fp8_gelu_quant(c, ymax, clear_max=nxt)
    assert torch.equal(q2, q) and torch.equal(s2, s) and nxt.item() == 0.0
    with pytest.raises(RuntimeError):
        ops.fp8_gelu_quant(c, ymax, clear_max=ymax)
    assert_close_tol(to_np_f32(h.cpu()), O.round_to(O.gelu_tanh_f32(to_np_f32(c.cpu())), dt), "gelu of the stored output")


@pytest.mark.parametrize("dt", ["bf16", "f16", "f32"])
# the persistent kernel with and without a round of half tiles, the one-wavefront-per-SIMD and two-workgroups-per-CU kernels
# with ragged edges, a tensor below the one-launch quantiser's size, one whose element count is not a multiple of 1024
@pytest.mark.parametrize("m,n,k", [(512, 1024, 256), (4608, 12288, 128), (2304, 1536, 3072), (333, 416, 704), (1024, 3072, 192), (7, 64, 64),
                                   (70, 96, 64)])
def test_fp8_chain_on_activations_in_k_panels(ops, dev, m, n, k, dt):
    """Quantisers that write [K/64, M, 64] k-panels and the GEMM that reads them give the bits of the row-major calls."""
    g = rng_t(m + 2 * n + 3 * k)
    t = TORCH_DT[dt]
    tout = torch.bfloat16 if dt == "f32" else t
    x = torch.randn(m, k, generator=g).to(t).to(dev)
    qa, sa = ops.fp8_quant(x)
    qp, sp = ops.fp8_quant_panels(x)
    assert qp.shape == (k // 64, m, 64) and torch.equal(sp, sa) and torch.equal(ops.fp8_panels_to_rows(qp), qa)
    static = torch.full((1,), 0.03125, dtype=torch.float32, device=dev)  # a given scale, as the reference's static input scale
    assert torch.equal(ops.fp8_panels_to_rows(ops.fp8_scale_cast_panels(x, static)), ops.fp8_scale_cast(x, static))
    qw, sw = ops.fp8_quant((torch.randn(n, k, generator=g) * 0.05).to(tout).to(dev))
    wp = ops.repack_weight(qw)
    bias = (torch.randn(n, generator=g) * 0.1).to(tout).to(dev)
    ymax, ymax_p = torch.zeros(1, dtype=torch.float32, device=dev), torch.zeros(1, dtype=torch.float32, device=dev)
    c = ops.fp8_linear_max(qa, wp, sa, sw, bias, ymax, tout)
    c_p = ops.fp8_linear_panels(qp, wp, sp, sw, bias, ymax_p, tout)
    assert torch.equal(c_p, c) and torch.equal(ymax_p, ymax)
    assert torch.equal(ops.fp8_linear_panels(qp, wp, sp, sw, bias, None, tout), c)
    for tactic in range(ops.gemm_tactic_count("fp8")):
        with ops.gemm_thread_tactic(tactic):
            assert torch.equal(ops.fp8_linear_panels(qp, wp, sp, sw, None, None, tout),
                               ops.fp8_linear(qa, wp, sa, sw, None, False, None, 0.0, tout)), f"tactic {tactic}"
    if n % 64 == 0:
        y = c.to(t)
        q, s = ops.fp8_gelu_quant(y, ymax)
        nxt = torch.full((1,), 7.0, dtype=torch.float32, device=dev)
        q_p, s_p = ops.fp8_gelu_quant_panels(y, ymax, clear_max=nxt)
        assert q_p.shape == (n // 64, m, 64) and torch.equal(s_p, s) and torch.equal(ops.fp8_panels_to_rows(q_p), q) and nxt.item() == 0.0


@pytest.mark.parametrize("dt", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("m,n,k,pre", [(512, 1024, 256, True), (4608, 1536, 3072, True), (333, 416, 704, False), (71, 96, 64, True),
                                       (1024, 768, 12288, False)])
def test_int8_chain_on_activations_in_k_panels(ops, dev, m, n, k, pre, dt):
    """The per-token quantiser writing k-panels and the INT8 GEMM reading them give the bits of the row-major calls."""
    g = rng_t(5 * m + n + k)
    t = TORCH_DT[dt]
    x = (torch.randn(m, k, generator=g) * 3).to(t).to(dev)
    ps = (torch.rand(k, generator=g) + 0.5).to(dev) if pre else None
    q, s = ops.sq_quant_dynamic(x, ps)
    qp, sp = ops.sq_quant_dynamic_panels(x, ps)
    assert qp.shape == (k // 64, m, 64) and torch.equal(sp, s) and torch.equal(ops.fp8_panels_to_rows(qp), q)
    w = ops.repack_weight(torch.randint(-127, 128, (n, k), generator=g, dtype=torch.int8).to(dev))
    ac = (torch.rand(n, generator=g) * 1e-2 + 1e-3).to(dev)
    bias = (torch.randn(n, generator=g) * 0.1).half().to(dev)
    assert torch.equal(ops.int8_linear_panels(qp, w, ac, sp, bias, torch.float16), ops.int8_linear(q, w, ac, s, bias, torch.float16))
    assert torch.equal(ops.int8_linear_panels(qp, w, None, None, None, torch.int32), ops.int8_linear(q, w, None, None, None, torch.int32))
    for tactic in range(ops.gemm_tactic_count("int8")):
        with ops.gemm_thread_tactic(tactic):
            assert torch.equal(ops.int8_linear_panels(qp, w, ac, sp, None, torch.bfloat16),
                               ops.int8_linear(q, w, ac, s, None, torch.bfloat16)), f"tactic {tactic}"
    with pytest.raises(ValueError):
        ops.sq_quant_dynamic_panels(torch.zeros(8, 96, dtype=torch.float16, device=dev))


def test_fp8_panel_ops_under_stream_capture_and_argument_checks(ops, dev):
    g = rng_t(77)
    x = torch.randn(300, 192, generator=g).bfloat16().to(dev)
    qa, sa = ops.fp8_quant(x)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # a capturing stream takes the exchange-free kernel sequence
        warm = ops.fp8_quant_panels(x)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            qp, sp = ops.fp8_quant_panels(x)
        for _ in range(3):
            qp.zero_()
            graph.replay()
            side.synchronize()
            assert torch.equal(ops.fp8_panels_to_rows(qp), qa) and torch.equal(sp, sa)
    torch.cuda.current_stream().wait_stream(side)
    assert torch.equal(ops.fp8_panels_to_rows(warm[0]), qa)
    with pytest.raises(ValueError):
        ops.fp8_quant_panels(torch.zeros(8, 96, dtype=torch.bfloat16, device=dev))
    lib = ops._l.load()
    buf = torch.zeros(4096, dtype=torch.uint8, device=dev)
    sc = torch.zeros(1, dtype=torch.float32, device=dev)
    assert lib.lq_fp8_amax_cast_panels(buf.data_ptr(), sc.data_ptr(), x.data_ptr(), 2, 8, 96, 0) < 0  # k % 64 != 0
    assert lib.lq_fp8_gelu_cast_panels(buf.data_ptr(), sc.data_ptr(), x.data_ptr(), 2, 8, 96, sc.data_ptr(), None, 0) < 0
    assert lib.lq_fp8_amax_cast_panels(buf.data_ptr(), sc.data_ptr(), x.data_ptr(), 2, 0, 64, 0) == 0  # empty
    with ops.gemm_thread_tactic(1):  # the 128-byte k-tile configuration reads row-major activations only: another one runs
        w = ops.repack_weight(ops.fp8_quant((torch.randn(256, 192, generator=g) * 0.05).bfloat16().to(dev))[0])
        qp, sp = ops.fp8_quant_panels(x)
        assert torch.equal(ops.fp8_linear_panels(qp, w, sp, sp, None), ops.fp8_linear(qa, w, sa, sa, None, False, None, 0.0, torch.bfloat16))


def test_fp8_gelu_quant_without_a_large_value_takes_the_bound(ops, dev):
    g = rng_t(9)
    y = (torch.rand(5000, generator=g) - 0.7).clamp(max=0.4).bfloat16().to(dev)
    ymax = y.float().max().clamp(min=0).reshape(1)
    q, s, h = ops.fp8_gelu_quant(y, ymax, want_h=True)
    assert s.item() == np.float32(max(h.float().max().item(), 0.171875)) / np.float32(448.0)
    assert torch.equal(q, ops.fp8_scale_cast(h, s))
    assert h.float().abs().max().item() <= s.item() * 448.0 * (1 + 1e-6)  # nothing saturates


# ---- FP8 GEMM epilogue outputs for the next FP8 linear -----------------------------------------------------------------
@pytest.mark.parametrize("m,n,k,gelu", [(333, 416, 704, True), (1024, 3072, 3072, False), (4608, 12288, 3072, True)])
@pytest.mark.parametrize("dt", ["bf16", "f16"])
def test_fp8_gemm_epilogue_scale_and_codes(ops, dev, m, n, k, gelu, dt):
    """The scale the epilogue accumulates and the codes it writes are exactly those of the separate amax / cast kernels
    applied to the GEMM's own 16-bit output (those kernels are checked against the oracle in test_gpu_quant.py)."""
    g = rng_t(m + n + k)
    t = TORCH_DT[dt]
    qa, sa = ops.fp8_quant(torch.randn(m, k, generator=g).to(t).to(dev))
    qw, sw = ops.fp8_quant((torch.randn(n, k, generator=g) * 0.02).to(t).to(dev))
    wp = ops.repack_weight(qw)
    bias = (torch.randn(n, generator=g) * 0.1).to(t).to(dev)
    plain = ops.fp8_linear(qa, wp, sa, sw, bias, gelu, None, 0.0, t)
    # dynamic: scale of the output
    s_out = torch.zeros(1, dtype=torch.float32, device=dev)
    c = ops.fp8_linear(qa, wp, sa, sw, bias, gelu, None, 0.0, t, out_scale=s_out)
    assert torch.equal(c, plain)
    q_ref, s_ref = ops.fp8_quant(plain)
    assert torch.equal(s_out, s_ref), (s_out.item(), s_ref.item())
    assert torch.equal(ops.fp8_scale_cast(c, s_out), q_ref)
    # accumulation semantics: a larger value already in the slot wins
    big = torch.full((1,), 1e6, dtype=torch.float32, device=dev)
    ops.fp8_linear(qa, wp, sa, sw, bias, gelu, None, 0.0, t, out_scale=big)
    assert big.item() == 1e6
    # static: codes with a given scale, with and without the 16-bit output
    s_static = torch.tensor([0.037], dtype=torch.float32, device=dev)
    c2, codes = ops.fp8_linear(qa, wp, sa, sw, bias, gelu, None, 0.0, t, out_fp8_scale=s_static)
    assert torch.equal(c2, plain)
    assert torch.equal(codes, ops.fp8_scale_cast(plain, s_static))
    only = ops.fp8_linear(qa, wp, sa, sw, bias, gelu, None, 0.0, t, out_fp8_scale=s_static, want_output=False)
    assert torch.equal(only, codes)
