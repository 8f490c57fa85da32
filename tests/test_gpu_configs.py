"""The five benchmark configurations at their full sizes, chained the way the reference's blocks chain
them, through the C ABI on the GPU.

Where the CPU oracle finishes in seconds the whole result is compared (configs 1 and 2, every
quantisation step of configs 3-5).  The large GEMMs of configs 3-5 are compared on one row out of
every 32-row band and all columns -- every output tile of every tile configuration is hit -- and the
remaining rows are covered by a size-independent property: a GEMM row depends on its own input row
only, so permuting the input rows must permute the output rows bit for bit.

Seeds: configuration i uses 1000 + i.  Tolerances: integer outputs and the INT8/W4A4 dequantised
outputs bit-exact against the oracle's fp32 formula; FP8 GEMM outputs within 1e-2 relative or 2 fp16
ULP of an fp64 evaluation (plus the documented accumulation floor of the fp8 matrix instruction)."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from oracle import oracle_c as OC
from tests.helpers import (assert_close_tol, check_fp8_against_instruction_model, check_fp8_gemm, make_outlier_acts, rng_t,
                           to_np_f32)

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops(dev):
    from lyradiff_amd import ops as _ops

    return _ops


def band_rows(m, seed, band=32):
    """One random row out of every `band` consecutive rows."""
    g = np.random.default_rng(seed)
    starts = np.arange(0, m, band)
    return np.minimum(starts + g.integers(0, band, size=starts.size), m - 1)


def dev_scalar(v, dev):
    return torch.tensor([float(v)], dtype=torch.float32, device=dev)


# ---- config 1: SDXL attention projection, INT8 SmoothQuant, dynamic per-token --------------------------------------
def test_config1_sdxl_attn_proj_int8(ops, dev):
    m, k, n = 1024, 1280, 1280
    g = rng_t(1001)
    x = make_outlier_acts(m, k, 8, 20.0, torch.float16, 1001)
    w = torch.randint(-127, 128, (n, k), generator=g, dtype=torch.int8)
    w_scale = (torch.rand(n, generator=g) * 9e-3 + 1e-3).float()
    bias = (torch.randn(n, generator=g) * 0.02).half()
    pre = (1.0 / O.smooth_vector(to_np_f32(x), w.numpy().astype(np.float32))).astype(np.float32)

    q, s = ops.sq_quant_dynamic(x.to(dev), torch.from_numpy(pre).to(dev))
    y = ops.int8_linear(q, ops.repack_weight(w.to(dev)), w_scale.to(dev), s, bias.to(dev), torch.float16)
    acc = ops.int8_linear(q, ops.repack_weight(w.to(dev)), None, None, None, torch.int32)

    q_ref, s_ref = O.sq_dynamic_quant(to_np_f32(x), pre)
    assert np.array_equal(q.cpu().numpy(), q_ref)
    assert np.array_equal(s.cpu().numpy(), s_ref)
    acc_ref = O.gemm_i8_acc(q_ref, w.numpy())
    assert np.array_equal(acc.cpu().numpy(), acc_ref)
    y_ref = O.int8_epilogue(acc_ref, w_scale.numpy(), s_ref, to_np_f32(bias), "f16")
    assert np.array_equal(to_np_f32(y), y_ref)
    # the same result evaluated in fp64 and rounded once: the tolerance the task states
    y64 = acc_ref.astype(np.float64) * (w_scale.numpy().astype(np.float64)[None, :] * s_ref.astype(np.float64)[:, None])
    assert_close_tol(to_np_f32(y), y64 + to_np_f32(bias).astype(np.float64)[None, :], "config 1 vs fp64")


def test_config1_end_to_end_with_the_smoothing_vector_made_on_the_device(ops, dev):
    """BASELINE config 1 with nothing precomputed on the host: column maxima of X and W (lq_col_absmax), the smoothing
    vector s[k] = max|X_k|^a / max|W_k|^(1-a) (lq_smooth_vector), the weight divided by pre = 1/s and quantised per
    output channel (lq_int8_weight_quant, the reference's loader kernel quant_kernels.cu:173-223), the dynamic per-token
    activation quantiser and the INT8 GEMM.  The device's powf may differ from numpy's in the last place, so the vector is
    compared with the oracle to 2e-6 and then handed to the oracle: everything after it is bit-exact."""
    m, k, n = 1024, 1280, 1280
    g = rng_t(1001)
    x = make_outlier_acts(m, k, 8, 20.0, torch.float16, 1001)
    w = (torch.randn(n, k, generator=g) * 0.02).half()
    bias = (torch.randn(n, generator=g) * 0.02).half()
    for alpha in (0.5, 0.8):
        ax = ops.col_absmax(x.to(dev))
        aw = ops.col_absmax(w.to(dev))
        pre, s = ops.smooth_vector(ax, aw, alpha)
        s_ref = O.smooth_vector(to_np_f32(x), to_np_f32(w), alpha)
        assert np.allclose(s.cpu().numpy(), s_ref, rtol=2e-6) and np.allclose(pre.cpu().numpy(), 1.0 / s_ref, rtol=3e-6)
        qw, sw = ops.int8_weight_quant(w.to(dev), pre)
        qx, sx = ops.sq_quant_dynamic(x.to(dev), pre)
        y = ops.int8_linear(qx, ops.repack_weight(qw), sw, sx, bias.to(dev), torch.float16)
        pre_np = pre.cpu().numpy()
        qw_ref, sw_ref = O.int8_weight_quant_device(to_np_f32(w), pre_np)
        qx_ref, sx_ref = O.sq_dynamic_quant(to_np_f32(x), pre_np)
        assert np.array_equal(qw.cpu().numpy(), qw_ref) and np.array_equal(sw.cpu().numpy(), sw_ref)
        assert np.array_equal(qx.cpu().numpy(), qx_ref) and np.array_equal(sx.cpu().numpy(), sx_ref)
        y_ref = O.int8_epilogue(O.gemm_i8_acc(qx_ref, qw_ref), sw_ref, sx_ref, to_np_f32(bias), "f16")
        assert np.array_equal(to_np_f32(y), y_ref)
        # SmoothQuant's purpose: the W8A8 product stays close to the 16-bit one despite the outlier columns
        full = to_np_f32(x).astype(np.float64) @ to_np_f32(w).astype(np.float64).T + to_np_f32(bias).astype(np.float64)
        err = np.abs(y_ref - full)
        assert np.sqrt((err ** 2).mean()) < 0.03 * np.sqrt((full ** 2).mean())


# ---- config 2: SDXL GEGLU feed-forward, INT8 W8A8 -----------------------------------------------------------------
def test_config2_sdxl_geglu_ffn_int8(ops, dev):
    m, d, inner = 4096, 640, 2560
    g = rng_t(1002)
    x = make_outlier_acts(m, d, 6, 15.0, torch.float16, 1002)
    w_up = torch.randint(-127, 128, (2 * inner, d), generator=g, dtype=torch.int8)
    w_dn = torch.randint(-127, 128, (d, inner), generator=g, dtype=torch.int8)
    # weight scales sized so that the hidden activations stay O(1), as a calibrated checkpoint's would
    ws_up = (torch.rand(2 * inner, generator=g) * 9e-4 + 1e-4).float()
    ws_dn = (torch.rand(d, generator=g) * 9e-3 + 1e-3).float()
    b_dn = (torch.randn(d, generator=g) * 0.02).half()

    q1, s1 = ops.sq_quant_dynamic(x.to(dev), None)
    h = ops.int8_linear(q1, ops.repack_weight(w_up.to(dev)), ws_up.to(dev), s1, None, torch.float16)
    q2, s2 = ops.geglu_int8_dynamic(h, None, None)
    y = ops.int8_linear(q2, ops.repack_weight(w_dn.to(dev)), ws_dn.to(dev), s2, b_dn.to(dev), torch.float16)

    q1_ref, s1_ref = O.sq_dynamic_quant(to_np_f32(x), None)
    assert np.array_equal(q1.cpu().numpy(), q1_ref) and np.array_equal(s1.cpu().numpy(), s1_ref)
    h_ref = O.int8_epilogue(O.gemm_i8_acc(q1_ref, w_up.numpy()), ws_up.numpy(), s1_ref, None, "f16")
    assert np.array_equal(to_np_f32(h), h_ref)
    q2_ref, s2_ref = O.geglu_int8_dynamic(h_ref, None, None, "f16")
    assert np.array_equal(q2.cpu().numpy(), q2_ref) and np.array_equal(s2.cpu().numpy(), s2_ref)
    y_ref = O.int8_epilogue(O.gemm_i8_acc(q2_ref, w_dn.numpy()), ws_dn.numpy(), s2_ref, to_np_f32(b_dn), "f16")
    assert np.array_equal(to_np_f32(y), y_ref)


# ---- FP8 helpers ---------------------------------------------------------------------------------------------------
def fp8_weight(ops, dev, n, k, gen):
    """N(0, 0.02) weight -> e4m3 codes + scale, quantised on the GPU and checked against the oracle."""
    w = (torch.randn(n, k, generator=gen) * 0.02).bfloat16()
    q, s = ops.fp8_quant(w.to(dev))
    q_ref, s_ref = O.fp8_amax_cast(to_np_f32(w))
    assert float(s.cpu()) == float(s_ref)
    assert np.array_equal(q.cpu().numpy(), q_ref)
    return q_ref, np.float32(s_ref), ops.repack_weight(q), s


def check_fp8_linear(ops, dev, qa_d, sa_d, wq, ws, wp, ws_d, bias, gelu, seed, what):
    """Runs the GEMM at full size, compares one row per 32-row band with the fp64 contract, and checks
    row-permutation equivariance over all rows.  Returns the device output."""
    m = qa_d.shape[0]
    y = ops.fp8_linear(qa_d, wp, sa_d, ws_d, bias.to(dev), gelu, None, 0.0, torch.bfloat16)
    rows = band_rows(m, seed)
    qa_rows = qa_d[torch.from_numpy(rows).to(dev)].cpu().numpy()
    sa = float(sa_d.cpu())
    ref = O.fp8_gemm(qa_rows, wq, sa, ws, to_np_f32(bias), gelu, None, 0.0, "bf16")
    got = to_np_f32(y[torch.from_numpy(rows).to(dev)])
    share = check_fp8_gemm(got, ref, qa_rows, wq, sa, ws, "bf16", what, extra_abs=2e-6 if gelu else 0.0)
    print(f"{what}: {share:.3e} of the compared outputs outside 1e-2 rel / 2 fp16 ULP (inside the instruction bound)")
    if not gelu:  # the GELU uses the hardware's exp2 / rcp: tolerance only
        check_fp8_against_instruction_model(got[::16], qa_rows[::16], wq, sa, ws, to_np_f32(bias), "bf16", what)
    perm = torch.randperm(m, generator=rng_t(seed)).to(dev)
    y_perm = ops.fp8_linear(qa_d[perm].contiguous(), wp, sa_d, ws_d, bias.to(dev), gelu, None, 0.0, torch.bfloat16)
    assert torch.equal(y_perm, y[perm]), f"{what}: output rows do not follow a permutation of the input rows"
    return y


def check_fp8_quant(ops, dev, x_d, seed, what):
    """Fused amax+cast at full size against the oracle: scale exact, codes exact on every row when the
    tensor is small enough for the CPU encoder, otherwise on one row per band."""
    q, s = ops.fp8_quant(x_d)
    x = to_np_f32(x_d)
    s_ref = O.fp8_scale(x)
    assert float(s.cpu()) == float(s_ref), what
    if x.size <= 24 * 1024 * 1024:
        assert np.array_equal(q.cpu().numpy(), O.fp8_scale_cast(x, s_ref, True)), what
    else:
        rows = band_rows(x.shape[0], seed)
        assert np.array_equal(q.cpu().numpy()[rows], O.fp8_scale_cast(x[rows], s_ref, True)), what
    return q, s


# ---- config 3: FLUX MLP, FP8 e4m3 per-tensor ----------------------------------------------------------------------
def test_config3_flux_mlp_fp8(ops, dev):
    m, d, hdim = 4608, 3072, 12288
    g = rng_t(1003)
    x = torch.randn(m, d, generator=g).bfloat16().to(dev)
    b_up = (torch.randn(hdim, generator=g) * 0.1).bfloat16()
    b_dn = (torch.randn(d, generator=g) * 0.1).bfloat16()
    wq_up, ws_up, wp_up, ws_up_d = fp8_weight(ops, dev, hdim, d, g)
    wq_dn, ws_dn, wp_dn, ws_dn_d = fp8_weight(ops, dev, d, hdim, g)

    qa, sa = check_fp8_quant(ops, dev, x, 31, "config 3 input quant")
    h = check_fp8_linear(ops, dev, qa, sa, wq_up, ws_up, wp_up, ws_up_d, b_up, True, 32, "config 3 up+GELU")
    qh, sh = check_fp8_quant(ops, dev, h, 33, "config 3 hidden quant")
    check_fp8_linear(ops, dev, qh, sh, wq_dn, ws_dn, wp_dn, ws_dn_d, b_dn, False, 34, "config 3 down")


def test_config3_flux_mlp_fp8_as_benchmarked(ops, dev):
    """The chain bench.py times: the up projection leaves its largest output (persistent kernel at this shape), the GELU and the
    dynamic quantisation of the hidden tensor are one pass that derives its scale from that maximum, then the down projection."""
    m, d, hdim = 4608, 3072, 12288
    g = rng_t(1003)
    x = torch.randn(m, d, generator=g).bfloat16().to(dev)
    b_up = (torch.randn(hdim, generator=g) * 0.1).bfloat16()
    b_dn = (torch.randn(d, generator=g) * 0.1).bfloat16()
    wq_up, ws_up, wp_up, ws_up_d = fp8_weight(ops, dev, hdim, d, g)
    wq_dn, ws_dn, wp_dn, ws_dn_d = fp8_weight(ops, dev, d, hdim, g)
    qa, sa = ops.fp8_quant(x)
    umax = torch.zeros(1, dtype=torch.float32, device=dev)
    u = ops.fp8_linear_max(qa, wp_up, sa, ws_up_d, b_up.to(dev), umax, torch.bfloat16)
    rows = band_rows(m, 41)
    qa_rows = qa[torch.from_numpy(rows).to(dev)].cpu().numpy()
    ref = O.fp8_gemm(qa_rows, wq_up, float(sa.cpu()), ws_up, to_np_f32(b_up), False, None, 0.0, "bf16")
    got = to_np_f32(u[torch.from_numpy(rows).to(dev)])
    check_fp8_gemm(got, ref, qa_rows, wq_up, float(sa.cpu()), ws_up, "bf16", "config 3 up, running maximum")
    check_fp8_against_instruction_model(got[::16], qa_rows[::16], wq_up, float(sa.cpu()), ws_up, to_np_f32(b_up), "bf16", "config 3 up")
    assert umax.item() == u.float().max().item() >= 0.5
    nxt = torch.ones(1, dtype=torch.float32, device=dev)
    qh, sh, h = ops.fp8_gelu_quant(u, umax, want_h=True)
    qh2, sh2 = ops.fp8_gelu_quant(u, umax, clear_max=nxt)
    assert torch.equal(qh2, qh) and torch.equal(sh2, sh) and nxt.item() == 0.0
    hn = to_np_f32(h)
    assert_close_tol(hn[rows], O.round_to(O.gelu_tanh_f32(to_np_f32(u)[rows]), "bf16"), "config 3 GELU of the stored output")
    s_ref = O.fp8_scale(hn)  # scale and codes: exactly the amax and cast of the activated tensor
    assert float(sh.cpu()) == float(s_ref)
    assert np.array_equal(qh.cpu().numpy()[rows], O.fp8_scale_cast(hn[rows], s_ref, True))
    y = check_fp8_linear(ops, dev, qh, sh, wq_dn, ws_dn, wp_dn, ws_dn_d, b_dn, False, 44, "config 3 down")
    # bench.py passes the quantised activations between these kernels as k-panels [K/64, M, 64]: the same bits at every step
    qa_p, sa_p = ops.fp8_quant_panels(x)
    assert torch.equal(sa_p, sa) and torch.equal(ops.fp8_panels_to_rows(qa_p), qa)
    umax_p = torch.zeros(1, dtype=torch.float32, device=dev)
    assert torch.equal(ops.fp8_linear_panels(qa_p, wp_up, sa_p, ws_up_d, b_up.to(dev), umax_p, torch.bfloat16), u) and torch.equal(umax_p, umax)
    qh_p, sh_p = ops.fp8_gelu_quant_panels(u, umax, clear_max=nxt)
    assert torch.equal(sh_p, sh) and torch.equal(ops.fp8_panels_to_rows(qh_p), qh)
    assert torch.equal(ops.fp8_linear_panels(qh_p, wp_dn, sh_p, ws_dn_d, b_dn.to(dev), None, torch.bfloat16), y)


# ---- config 4: FLUX attention projection, W4A4 group 64, fp16 scales ----------------------------------------------
@pytest.mark.parametrize("sdt", ["f16", "f32"])
def test_config4_flux_attn_proj_w4a4(ops, dev, sdt):
    m, k, n = 4608, 3072, 3072
    g = rng_t(1004)
    x = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(n, k, generator=g) * 0.02).bfloat16()
    bias = (torch.randn(n, generator=g) * 0.1).bfloat16()
    sdt_t = torch.float16 if sdt == "f16" else torch.float32

    qa, sA = ops.w4a4_quant(x.to(dev), None, sdt_t)
    qb, sB = ops.w4a4_quant(w.to(dev), None, sdt_t)
    qa_ref, sA_ref = O.w4a4_quant(to_np_f32(x), None, 64, sdt)
    qb_ref, sB_ref = O.w4a4_quant(to_np_f32(w), None, 64, sdt)
    assert np.array_equal(qa.cpu().numpy().view(np.uint32), qa_ref) and np.array_equal(to_np_f32(sA), sA_ref)
    assert np.array_equal(qb.cpu().numpy().view(np.uint32), qb_ref) and np.array_equal(to_np_f32(sB), sB_ref)

    wp = ops.repack_weight(qb.view(torch.uint8).reshape(n, k // 2))
    y = ops.w4a4_linear(qa, wp, sA, sB, bias.to(dev), torch.bfloat16)
    rows = band_rows(m, 41)
    ref = O.round_to(OC.w4a4_gemm(qa_ref[rows], qb_ref, sA_ref[rows], sB_ref, to_np_f32(bias)), "bf16")
    assert np.array_equal(to_np_f32(y)[rows], ref)
    perm = torch.randperm(m, generator=rng_t(42)).to(dev)
    y_perm = ops.w4a4_linear(qa[perm].contiguous(), wp, sA[perm].contiguous(), sB, bias.to(dev), torch.bfloat16)
    assert torch.equal(y_perm, y[perm])


# ---- config 5: FLUX double-stream block linear chain at 1280^2, FP8 ------------------------------------------------
def test_config5_flux_double_block_fp8_chain(ops, dev):
    m, d = 6912, 3072
    g = rng_t(1005)
    x = torch.randn(m, d, generator=g).bfloat16().to(dev)
    attn = torch.randn(m, d, generator=g).bfloat16().to(dev)  # stands in for the attention output between QKV and out-proj
    layers = {}
    for name, (n, k) in {"qkv": (3 * d, d), "out": (d, d), "up": (4 * d, d), "down": (d, 4 * d)}.items():
        layers[name] = fp8_weight(ops, dev, n, k, g) + ((torch.randn(n, generator=g) * 0.1).bfloat16(),)

    def linear(name, inp, gelu, seed):
        q, s = check_fp8_quant(ops, dev, inp, seed, f"config 5 {name} quant")
        wq, ws, wp, ws_d, bias = layers[name]
        return check_fp8_linear(ops, dev, q, s, wq, ws, wp, ws_d, bias, gelu, seed + 1, f"config 5 {name}")

    linear("qkv", x, False, 51)
    o = linear("out", attn, False, 53)
    hid = linear("up", o, True, 55)
    linear("down", hid, False, 57)


# ---- sizes beyond 2^31 bytes: every row offset must be computed in 64 bits -----------------------------------------------
def test_more_than_two_gib_of_activations(ops, dev):
    m, k, n = 720_000, 3072, 64  # fp16 activations 4.4 GB, int8 2.2 GB
    g = torch.Generator(device=dev).manual_seed(9)
    x = torch.randn(m, k, generator=g, device=dev, dtype=torch.float16)
    w = torch.randint(-127, 128, (n, k), generator=rng_t(9), dtype=torch.int8)
    q, s = ops.sq_quant_dynamic(x, None)
    acc = ops.int8_linear(q, ops.repack_weight(w.to(dev)), None, None, None, torch.int32)
    rows = np.concatenate([np.arange(0, 4), np.arange(349_520, 349_530), np.arange(699_046, 699_056), np.arange(m - 4, m)])
    idx = torch.from_numpy(rows).to(dev)
    q_ref, s_ref = O.sq_dynamic_quant(to_np_f32(x[idx]), None)
    assert np.array_equal(q[idx].cpu().numpy(), q_ref) and np.array_equal(s[idx].cpu().numpy(), s_ref)
    assert np.array_equal(acc[idx].cpu().numpy(), O.gemm_i8_acc(q_ref, w.numpy()))
    del x
    xb = torch.randn(m, 1024, generator=g, device=dev, dtype=torch.bfloat16)  # 1.5 GB in, 0.7 GB out
    qb, sb = ops.fp8_quant(xb)
    assert np.float32(sb.cpu().numpy()[0]) == np.float32(xb.abs().max().float().cpu().numpy()) / np.float32(448.0)
    ref = O.fp8_scale_cast(to_np_f32(xb[idx]), np.float32(sb.cpu().numpy()[0]), True)
    assert np.array_equal(qb[idx].cpu().numpy(), ref)
