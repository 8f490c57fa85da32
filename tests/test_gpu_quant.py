"""GPU parity of the activation-quantisation kernels against the CPU oracle, through the C ABI.

Bit-exact for every integer / byte output and for the fp32 scales."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from oracle import oracle_c as OC
from tests.helpers import TORCH_DT, make_outlier_acts, rng_t, to_np_f32

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops(dev):
    from lyradiff_amd import ops as _ops

    return _ops


@pytest.mark.parametrize("dt", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("m,k", [(1024, 1280), (37, 640), (5, 8), (3, 2560), (64, 12288), (7, 1283), (301, 3072), (19, 2056), (3, 16384), (301, 6152)])
def test_sq_dynamic_quant(ops, dev, dt, m, k):
    x = make_outlier_acts(m, k, min(8, k), 20.0, TORCH_DT[dt], 1000 + m + k)
    pre = (torch.rand(k, generator=rng_t(7)) * 1.5 + 0.25).float()
    q, s = ops.sq_quant_dynamic(x.to(dev), pre.to(dev))
    q_ref, s_ref = O.sq_dynamic_quant(to_np_f32(x), pre.numpy())
    assert np.array_equal(s.cpu().numpy(), s_ref)
    assert np.array_equal(q.cpu().numpy(), q_ref)
    # no smoothing vector
    q2, s2 = ops.sq_quant_dynamic(x.to(dev), None)
    q2_ref, s2_ref = O.sq_dynamic_quant(to_np_f32(x), None)
    assert np.array_equal(s2.cpu().numpy(), s2_ref) and np.array_equal(q2.cpu().numpy(), q2_ref)


@pytest.mark.parametrize("k", [64, 2080])
def test_sq_dynamic_nan_and_inf_rows(ops, dev, k):
    """NaN never enters the row maximum and quantises to 0; a row holding an infinity gets an infinite scale,
    its finite elements become 0 and inf/inf = NaN becomes 0 as well (the oracle's IEEE arithmetic decides)."""
    x = torch.randn(6, k, generator=rng_t(k)) * 3
    x[1, 5] = float("nan")
    x[2, 7] = float("inf")
    x[3, 9] = float("-inf"); x[3, 11] = float("nan")
    x[4, :] = float("nan")
    x[5, k - 1] = float("nan"); x[5, k - 2] = 1e30
    for pre in (None, (torch.rand(k, generator=rng_t(3)) + 0.5).float()):
        q, s = ops.sq_quant_dynamic(x.to(dev), None if pre is None else pre.to(dev))
        q_ref, s_ref = O.sq_dynamic_quant(x.numpy(), None if pre is None else pre.numpy())
        assert np.array_equal(s.cpu().numpy(), s_ref, equal_nan=True)
        assert np.array_equal(q.cpu().numpy(), q_ref)


def test_sq_dynamic_zero_rows(ops, dev):
    x = torch.randn(16, 1280).half()
    x[3] = 0
    x[9] = 0
    q, s = ops.sq_quant_dynamic(x.to(dev), None)
    assert s[3].item() == 1.0 and s[9].item() == 1.0
    assert int(q[3].abs().max()) == 0 and int(q[9].abs().max()) == 0
    q_ref, s_ref = O.sq_dynamic_quant(to_np_f32(x), None)
    assert np.array_equal(q.cpu().numpy(), q_ref) and np.array_equal(s.cpu().numpy(), s_ref)


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("per_token", [False, True])
@pytest.mark.parametrize("k", [1280, 3080, 6152])
def test_sq_static_quant(ops, dev, dt, per_token, k):
    m = 300 if k < 6144 else 301  # rows of 6144 columns and more go two to a workgroup: an odd count leaves the last one half empty
    x = make_outlier_acts(m, k, 8, 20.0, TORCH_DT[dt], 5)
    pre = (torch.rand(k, generator=rng_t(8)) + 0.5).float()
    # a static scale small enough that saturation to -128 / 127 happens
    scale = (torch.rand(m if per_token else 1, generator=rng_t(9)) * 0.02 + 0.01).float()
    q = ops.sq_quant(x.to(dev), pre.to(dev), scale.to(dev), per_token)
    q_ref = O.sq_input_quant(to_np_f32(x), pre.numpy(), scale.numpy(), per_token)
    assert q_ref.min() == -128 and q_ref.max() == 127
    assert np.array_equal(q.cpu().numpy(), q_ref)


@pytest.mark.parametrize("reps", [4, 130])  # 64 columns (one wavefront per row) and 2080 (row split over wavefronts)
def test_sq_quant_ties_and_specials(ops, dev, reps):
    # exact half-integers, saturation edges, NaN and inf, with s = 1 and a power-of-two s
    vals = [0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5, 127.5, -127.5, -128.5, 300.0, -300.0,
            float("nan"), float("inf"), float("-inf"), 0.0]
    x = torch.tensor(vals * reps, dtype=torch.float32).reshape(1, -1)
    for s in (1.0, 0.5, 3.0):
        sc = torch.tensor([s], dtype=torch.float32)
        q = ops.sq_quant(x.to(dev), None, sc.to(dev), False)
        assert np.array_equal(q.cpu().numpy(), O.sq_input_quant(x.numpy(), None, sc.numpy(), False))


@pytest.mark.parametrize("dt", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("with_bias", [True, False])
def test_geglu_int8(ops, dev, dt, with_bias):
    m, d = 200, 2560
    g = rng_t(11)
    x = (torch.randn(m, 2 * d, generator=g) * 1.5).to(TORCH_DT[dt])
    bias = (torch.randn(2 * d, generator=g) * 0.1).to(TORCH_DT[dt]) if with_bias else None
    pre = (torch.rand(d, generator=g) + 0.5).float()
    xn, bn = to_np_f32(x), (to_np_f32(bias) if with_bias else None)
    q, s = ops.geglu_int8_dynamic(x.to(dev), bias.to(dev) if with_bias else None, pre.to(dev))
    q_ref, s_ref = O.geglu_int8_dynamic(xn, bn, pre.numpy(), dt)
    assert np.array_equal(s.cpu().numpy(), s_ref)
    assert np.array_equal(q.cpu().numpy(), q_ref)
    sc = torch.tensor([0.03], dtype=torch.float32)
    q2 = ops.geglu_int8(x.to(dev), bias.to(dev) if with_bias else None, pre.to(dev), sc.to(dev))
    assert np.array_equal(q2.cpu().numpy(), O.geglu_int8(xn, bn, pre.numpy(), sc.numpy(), dt))


@pytest.mark.parametrize("dt", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("m,d", [(37, 5120), (2051, 2568), (5, 4096), (9, 8192), (3, 5128)])
def test_geglu_int8_wide_rows(ops, dev, dt, m, d):
    """Rows of 2561..5120 columns are shared by two wavefronts (row maximum exchanged through LDS); wider ones take the
    one-wavefront form again.  Row counts that leave wavefront pairs idle in the last trip, widths that leave the second
    wavefront a ragged or almost empty half, a maximum that sits in either half."""
    g = rng_t(m + d)
    x = (torch.randn(m, 2 * d, generator=g) * 1.5)
    x[0::2, 7] *= 9.0            # row maximum in the first half of the value columns
    x[1::2, d - 3] *= 9.0        # ... and in the last columns
    x = x.to(TORCH_DT[dt])
    bias = (torch.randn(2 * d, generator=g) * 0.1).to(TORCH_DT[dt])
    pre = (torch.rand(d, generator=g) + 0.5).float()
    xn, bn = to_np_f32(x), to_np_f32(bias)
    q, s = ops.geglu_int8_dynamic(x.to(dev), bias.to(dev), pre.to(dev))
    q_ref, s_ref = O.geglu_int8_dynamic(xn, bn, pre.numpy(), dt)
    assert np.array_equal(s.cpu().numpy(), s_ref) and np.array_equal(q.cpu().numpy(), q_ref)
    sc = torch.tensor([0.04], dtype=torch.float32)
    q2 = ops.geglu_int8(x.to(dev), None, None, sc.to(dev))
    assert np.array_equal(q2.cpu().numpy(), O.geglu_int8(xn, None, None, sc.numpy(), dt))


@pytest.mark.parametrize("dt", ["f16", "bf16", "f32"])
def test_geglu_int8_gate_values_outside_the_table(ops, dev, dt):
    """Gate inputs below 2^-12, at the table's two ends, beyond 8, subnormal, infinite and NaN (the HIP kernel looks the gate
    factor up for 2^-12 <= |g| < 8 and uses its constant forms elsewhere), with and without a bias."""
    m, d = 64, 1024
    g = rng_t(23)
    x = (torch.randn(m, 2 * d, generator=g) * 1.5)
    gate = x[:, d:]
    gate[:, 0::7] *= 1e-4
    gate[:, 1::11] *= 20.0
    gate[0, :12] = torch.tensor([2.0 ** -12, -2.0 ** -12, 8.0, -8.0, 7.99, -7.99, 2.4e-4, -2.4e-4, 6e-8, -6e-8, 0.0, -0.0])
    gate[1, :4] = torch.tensor([float("inf"), float("-inf"), float("nan"), 65504.0])
    x = x.to(TORCH_DT[dt])
    xn = to_np_f32(x)
    pre = (torch.rand(d, generator=g) + 0.5).float()
    for bias in (None, (torch.randn(2 * d, generator=g) * 1e-3).to(TORCH_DT[dt])):
        bn = None if bias is None else to_np_f32(bias)
        bd = None if bias is None else bias.to(dev)
        sc = torch.tensor([0.05], dtype=torch.float32)
        with np.errstate(all="ignore"):
            q_ref = O.geglu_int8(xn, bn, pre.numpy(), sc.numpy(), dt)
            qd_ref, sd_ref = O.geglu_int8_dynamic(xn, bn, pre.numpy(), dt)
        assert np.array_equal(ops.geglu_int8(x.to(dev), bd, pre.to(dev), sc.to(dev)).cpu().numpy(), q_ref)
        qd, sd = ops.geglu_int8_dynamic(x.to(dev), bd, pre.to(dev))
        assert np.array_equal(sd.cpu().numpy(), sd_ref, equal_nan=True) and np.array_equal(qd.cpu().numpy(), qd_ref)


@pytest.mark.parametrize("dt", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("n", [4608 * 3072, 1000003, 17, 4096, 35000003])  # the last: more than two workgroups per CU hold with 8 chunks
def test_fp8_amax_cast(ops, dev, dt, n):
    x = (torch.randn(n, generator=rng_t(n % 1000)) * 3).to(TORCH_DT[dt])
    q, s = ops.fp8_quant(x.to(dev))
    q_ref, s_ref = O.fp8_amax_cast(to_np_f32(x))
    assert s.item() == float(s_ref)
    assert np.array_equal(q.cpu().numpy(), q_ref)


def test_fp8_static_cast_saturates_and_nan(ops, dev):
    x = torch.tensor([1.0, -1.0, 447.0, 449.0, 1e6, -1e6, float("nan"), float("inf"), 0.0, 1e-4, -3e-3, 0.0175] * 4,
                     dtype=torch.float32)
    for sc, inv in ((1.0, True), (0.5, True), (2.0, False)):
        s = torch.tensor([sc], dtype=torch.float32)
        q = ops.fp8_scale_cast(x.to(dev), s.to(dev), inv)
        assert np.array_equal(q.cpu().numpy(), O.fp8_scale_cast(x.numpy(), s.numpy(), inv))


def test_fp8_amax_scale_accumulates(ops, dev):
    x = torch.randn(100000).bfloat16()
    s = torch.tensor([10.0], dtype=torch.float32, device=dev)  # larger than any |x|/448
    ops.fp8_amax_scale(x.to(dev), s)
    assert s.item() == 10.0
    s2 = ops.fp8_amax_scale(x.to(dev))
    assert s2.item() == float(O.fp8_scale(to_np_f32(x)))


@pytest.mark.parametrize("dt", ["bf16", "f16", "f32"])
@pytest.mark.parametrize("sdt", ["f32", "f16"])
@pytest.mark.parametrize("m,k", [(4608, 3072), (33, 64), (256, 12288), (5, 640)])
def test_w4a4_quant(ops, dev, dt, sdt, m, k):
    g = rng_t(m + k)
    x = torch.randn(m, k, generator=g).to(TORCH_DT[dt])
    x[0, :64] = 0  # an all-zero group
    smooth = (torch.rand(k, generator=g) * 1.5 + 0.5).float()
    for sm in (smooth, None):
        q, s = ops.w4a4_quant(x.to(dev), None if sm is None else sm.to(dev), TORCH_DT[sdt])
        q_ref, s_ref = O.w4a4_quant(to_np_f32(x), None if sm is None else sm.numpy(), 64, sdt)
        assert np.array_equal(s.cpu().float().numpy(), s_ref)
        assert np.array_equal(q.cpu().numpy().view(np.uint32), q_ref)


@pytest.mark.parametrize("sdt", ["f32", "f16"])
@pytest.mark.parametrize("k", [256, 3072])
def test_w4a4_quant_special_groups(ops, dev, sdt, k):
    """Groups holding NaN or infinity, and groups so small that an fp16 scale is subnormal (rounded down by a large
    factor, so the quotients exceed 7 and must saturate) or zero."""
    g = rng_t(k)
    x = torch.randn(8, k, generator=g)
    x[0, 3] = float("nan")
    x[1, 70] = float("inf")
    x[2, 130] = float("-inf"); x[2, 131] = float("nan")
    x[3, :64] = torch.randn(64, generator=g) * 1.1e-7   # absmax/7 between fp16 subnormal steps
    x[4, :64] = torch.randn(64, generator=g) * 3e-9     # fp16 scale underflows to zero
    x[5, 64:128] = torch.randn(64, generator=g) * 2.5e-7
    x[6, :64] = 1e-30
    smooth = (torch.rand(k, generator=g) * 1.5 + 0.5).float()
    for sm in (None, smooth):
        q, s = ops.w4a4_quant(x.to(dev), None if sm is None else sm.to(dev), TORCH_DT[sdt])
        q_ref, s_ref = O.w4a4_quant(x.numpy(), None if sm is None else sm.numpy(), 64, sdt)
        assert np.array_equal(s.cpu().float().numpy(), s_ref, equal_nan=True)
        assert np.array_equal(q.cpu().numpy().view(np.uint32), q_ref)


def test_repack_roundtrip(ops, dev):
    w = torch.randint(-128, 128, (1280, 640), dtype=torch.int8)
    p = ops.repack_weight(w.to(dev))
    assert np.array_equal(p.cpu().numpy().view(np.uint8).reshape(-1), O.repack_rows32(w.numpy()))
    assert torch.equal(ops.unpack_weight(p).cpu(), w)


def test_golden_vectors_on_gpu(ops, dev):
    """The hand-derived known-answer vectors of tests/golden/ straight through the HIP kernels."""
    import os

    G = np.load(os.path.join(os.path.dirname(__file__), "golden", "quant_golden.npz"))
    one = torch.ones(1, dtype=torch.float32, device=dev)
    # float_to_int8_rn table (static scale 1)
    xin = torch.from_numpy(G["s8_in"]).reshape(1, -1)
    assert np.array_equal(ops.sq_quant(xin.to(dev), None, one, False).cpu().numpy().reshape(-1), G["s8_out"])
    # e4m3 encode table (scale 1, both directions of the scale flag)
    xe = torch.from_numpy(G["e4m3_in"])
    assert np.array_equal(ops.fp8_scale_cast(xe.to(dev), one, True).cpu().numpy(), G["e4m3_out"])
    assert np.array_equal(ops.fp8_scale_cast(xe.to(dev), one, False).cpu().numpy(), G["e4m3_out"])
    # per-token INT8 quant
    q, s = ops.sq_quant_dynamic(torch.from_numpy(G["sq_x"]).to(dev), torch.from_numpy(G["sq_pre"]).to(dev))
    assert np.array_equal(q.cpu().numpy(), G["sq_q"]) and np.array_equal(s.cpu().numpy(), G["sq_scale"])
    # W4A4 group quant + packing
    w, sc = ops.w4a4_quant(torch.from_numpy(G["w4_x"]).to(dev), None)
    assert np.array_equal(sc.cpu().numpy(), G["w4_scale"])
    assert np.array_equal(O.unpack_int4(w.cpu().numpy().view(np.uint32)), G["w4_xq"])
    # INT8 GEMM 4x8x16 embedded in the smallest shape the tiled kernel takes (n % 32, k % 64), zero padded
    a = np.zeros((4, 64), np.int8)
    a[:, :16] = G["gemm_a"]
    wt = np.zeros((32, 64), np.int8)
    wt[:8, :16] = G["gemm_w"]
    acc = ops.int8_linear(torch.from_numpy(a).to(dev), ops.repack_weight(torch.from_numpy(wt).to(dev)), None, None, None,
                          torch.int32).cpu().numpy()
    assert np.array_equal(acc[:, :8], G["gemm_acc"]) and not acc[:, 8:].any()
    # W4A4 GEMM on the packed golden words (unit scales): exact integer dot products of the nibbles
    qv = G["w4_q"].astype(np.int32)
    aw = np.zeros((8, 16), np.uint32)
    aw[:, :8] = G["w4_words"]  # K = 128: second group zero
    bw = np.zeros((32, 16), np.uint32)
    bw[:8, :8] = G["w4_words"]
    ones_a = torch.ones(8, 2, device=dev)
    ones_b = torch.ones(32, 2, device=dev)
    y = ops.w4a4_linear(torch.from_numpy(aw.view(np.int32)).to(dev),
                        ops.repack_weight(torch.from_numpy(bw.view(np.uint8).reshape(32, 64)).to(dev)),
                        ones_a, ones_b, None, torch.float32).cpu().numpy()
    assert np.array_equal(y[:, :8], (qv @ qv.T).astype(np.float32)) and not y[:, 8:].any()
    # rows32 repack
    p = ops.repack_weight(torch.from_numpy(G["rows32_src"]).to(dev))
    assert np.array_equal(p.cpu().numpy().reshape(-1), G["rows32_dst"])


def test_fp8_amax_cast_stream_slots_fallback_and_status(ops, dev):
    """The one-launch dynamic quantiser meets at a grid barrier in a slot that belongs to the calling stream; at most 16
    streams per device get one, the others run the scratch-free kernel sequence.  Both routes give the oracle's codes and
    scale, and after normal runs the time-out status reads clean."""
    import ctypes as C

    from lyradiff_amd import lib as L

    lib = L.load()
    streams = [torch.cuda.Stream() for _ in range(20)]
    slots = [lib.lq_fp8_amax_cast_slot(C.c_void_p(st.cuda_stream)) for st in streams]
    assert all(-1 <= v < 16 for v in slots)
    owned = [v for v in slots if v >= 0]
    assert len(set(owned)) == len(owned) and slots.count(-1) >= 4  # distinct slots; 20 streams cannot all have one
    if -1 in slots:
        assert all(v == -1 for v in slots[slots.index(-1):])  # once they run out they stay out
    assert [lib.lq_fp8_amax_cast_slot(C.c_void_p(st.cuda_stream)) for st in streams] == slots  # stable per stream
    x = (torch.randn(300, 1024, generator=rng_t(3)) * 3).bfloat16()
    q_ref, s_ref = O.fp8_amax_cast(to_np_f32(x))
    xd = x.to(dev)
    torch.cuda.synchronize()
    outs = []
    for st in (streams[0], streams[-1]):  # one with a slot (unless earlier tests used them up), one without
        with torch.cuda.stream(st):
            outs.append(ops.fp8_quant(xd))
    torch.cuda.synchronize()
    for q, s in outs:
        assert s.item() == float(s_ref) and np.array_equal(q.cpu().numpy(), q_ref)
    assert ops.fp8_amax_cast_status() is False
    # slots are given back: afterwards a new stream finds one again, and a stream that owns none reports -1
    freed = [ops.fp8_quant_release_stream(st) for st in streams]
    assert sorted(v for v in freed if v >= 0) == sorted(owned) and freed.count(-1) == slots.count(-1)
    assert ops.fp8_quant_release_stream(streams[0]) == -1
    fresh = torch.cuda.Stream()
    assert lib.lq_fp8_amax_cast_slot(C.c_void_p(fresh.cuda_stream)) >= 0
    with torch.cuda.stream(fresh):
        q, s = ops.fp8_quant(xd)
    torch.cuda.synchronize()
    assert s.item() == float(s_ref) and np.array_equal(q.cpu().numpy(), q_ref)
    assert ops.fp8_quant_release_stream(fresh) >= 0


@pytest.mark.parametrize("dt", ["bf16", "f16", "f32"])
@pytest.mark.parametrize("n", [4096, 5000, 1024 * 16 * 256 * 4 + 1024 + 7, 23 * 1024 * 1024 + 1000, 52 * 1024 * 1024 + 13])
def test_fp8_amax_cast_one_launch_sizes(ops, dev, dt, n):
    """The one-launch quantiser over its register budgets: tensors that fit with 4, 8 and 12 chunks per thread, one that does
    not (its rest is read twice), ragged tails shorter than a 2 KiB block; codes and scale equal the oracle's, and the
    two-launch allocation-free form gives the same bits."""
    if dt == "f32" and n > 30 * 1024 * 1024:
        pytest.skip("the fp32 form is covered at the smaller sizes")
    x = (torch.randn(n, generator=rng_t(n % 1000 + 5)) * 2.5).to(TORCH_DT[dt])
    x[n // 3] = 37.0
    xd = x.to(dev)
    q, s = ops.fp8_quant(xd)
    xf = to_np_f32(x)
    s_ref = OC.fp8_scale(xf)
    q_ref = OC.fp8_scale_cast(xf, s_ref)
    assert s.item() == float(s_ref)
    assert np.array_equal(q.cpu().numpy(), q_ref)
    q2, s2 = torch.empty_like(q), torch.empty_like(s)
    ops.fp8_quant_static(xd, q2, s2)
    assert torch.equal(q, q2) and torch.equal(s, s2)
    assert ops.fp8_amax_cast_status() is False


@pytest.mark.parametrize("dt,m,k", [("bf16", 4608, 12288), ("f32", 4608, 12288), ("f16", 6912, 3072), ("bf16", 5000, 8256)])
def test_fp8_quant_panels_of_tensors_beyond_the_kept_chunks(ops, dev, dt, m, k):
    """The one-launch quantiser writing k-panels keeps eight chunks per lane and reads the rest of a larger tensor twice (the
    second loop of its walk); 5000 x 8256 also ends in a partial row block."""
    g = torch.Generator(device=dev).manual_seed(m + k)
    x = (torch.randn(m, k, generator=g, device=dev) * 2).to(TORCH_DT[dt])
    q, s = ops.fp8_quant(x)
    qp, sp = ops.fp8_quant_panels(x)
    assert torch.equal(sp, s) and torch.equal(ops.fp8_panels_to_rows(qp), q)
    assert ops.fp8_amax_cast_status() is False
    assert torch.equal(ops.fp8_panels_to_rows(ops.fp8_scale_cast_panels(x, s)), q)  # the cast with a given scale, same walk


def test_fp8_amax_cast_timeline_gives_the_same_bits_and_ordered_stamps(ops, dev):
    x = (torch.randn(4608 * 3072, generator=rng_t(3)) * 2).bfloat16().to(dev)
    q0, s0 = ops.fp8_quant(x)
    q, s, st = ops.fp8_quant_timeline(x)
    assert torch.equal(q, q0) and torch.equal(s, s0)
    st = st.cpu().numpy()
    assert 1 <= st.shape[0] <= 512 and np.all(np.diff(st, axis=1) >= 0), "started <= loads back <= released <= stores acknowledged"
    assert st[:, 2].min() >= st[:, 1].max(), "nobody is released from the exchange before the last partial maximum is formed"
    assert (st[:, 3].max() - st[:, 0].min()) * 0.01 < 1000.0  # microseconds
    with pytest.raises(RuntimeError):
        ops.fp8_quant_timeline(x[:100])


def test_fp8_quant_static_reset(ops, dev):
    """The repair call of the allocation-free quantiser: after it the status is clean and the quantiser works."""
    x = (torch.randn(70000, generator=rng_t(9)) * 3).bfloat16().to(dev)
    ops.fp8_quant_static_reset()
    q, s = torch.empty(70000, dtype=torch.uint8, device=dev), torch.empty(1, device=dev)
    ops.fp8_quant_static(x, q, s)
    q_ref, s_ref = O.fp8_amax_cast(to_np_f32(x.cpu()))
    assert s.item() == float(s_ref) and np.array_equal(q.cpu().numpy(), q_ref)
    assert ops.fp8_amax_cast_status() is False


# ---- per-output-channel weight quantisation on the device (invokeGetINT8WeightScale, quant_kernels.cu:173-223,270-312) ---
@pytest.mark.parametrize("dt", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("with_pre", [True, False])
@pytest.mark.parametrize("n,k", [(1280, 1280), (640, 2560), (33, 8), (5, 4099)])
def test_int8_weight_quant_device(ops, dev, dt, with_pre, n, k):
    g = rng_t(300 + n + k)
    w = (torch.randn(n, k, generator=g) * 0.05).to(TORCH_DT[dt])
    w[n // 2] = 0  # zero row: amax 0, scale 0, 0/0 = NaN -> code 0
    w[1, k - 1] = -w[1].abs().max() * 2  # the row maximum on a negative element: -127, never -128
    pre = (torch.rand(k, generator=g) * 2.7 + 0.3).float() if with_pre else None
    q, s = ops.int8_weight_quant(w.to(dev), None if pre is None else pre.to(dev))
    q_ref, s_ref = O.int8_weight_quant_device(to_np_f32(w), None if pre is None else pre.numpy())
    assert np.array_equal(s.cpu().numpy(), s_ref)
    assert np.array_equal(q.cpu().numpy(), q_ref)
    assert s_ref[n // 2] == 0.0 and not q_ref[n // 2].any()
    assert np.array_equal(np.abs(q_ref[np.arange(n) != n // 2].astype(np.int32)).max(axis=1), np.full(n - 1, 127))
    if not with_pre:
        assert q_ref[1, k - 1] == -127


def test_int8_weight_quant_device_specials_and_many_rows(ops, dev):
    """NaN never enters the row maximum and quantises to 0, an infinity makes the scale infinite (finite/inf = 0,
    inf/inf = NaN -> 0), an all-NaN row has scale 0; more rows than one grid dimension holds (d_out > 65535)."""
    k = 72
    w = torch.randn(70001, k, generator=rng_t(12))
    w[0, 3] = float("nan")
    w[1, 5] = float("inf")
    w[2, :] = float("nan")
    w[3, 6] = float("-inf"); w[3, 9] = float("nan")
    w[70000, k - 1] = 1e30
    pre = (torch.rand(k, generator=rng_t(13)) + 0.5).float()
    for p in (None, pre):
        q, s = ops.int8_weight_quant(w.to(dev), None if p is None else p.to(dev))
        with np.errstate(invalid="ignore"):
            q_ref, s_ref = O.int8_weight_quant_device(w.numpy(), None if p is None else p.numpy())
        assert np.array_equal(s.cpu().numpy(), s_ref, equal_nan=True)
        assert np.array_equal(q.cpu().numpy(), q_ref)
    assert np.isinf(s_ref[1]) and not q_ref[1].any() and s_ref[2] == 0.0 and not q_ref[2].any()
    with pytest.raises(ValueError):
        ops.int8_weight_quant(w[:4].to(dev), pre[:8].to(dev))


def test_int8_weight_quant_feeds_the_gemm(ops, dev):
    """The reference's loader path: fp16 weight -> device quantiser (dividing by pre_quant_scale) -> INT8 GEMM with the
    per-channel scales it produced (layers/basic_transformer/BasicTransformerInt8BlockWeight.cc, quant_kernels.cu:270-312)."""
    m, n, k = 96, 320, 640
    g = rng_t(77)
    x = make_outlier_acts(m, k, 6, 15.0, torch.float16, 78)
    w = (torch.randn(n, k, generator=g) * 0.03).half()
    pre = (torch.rand(k, generator=g) * 1.5 + 0.5).float()
    qw, sw = ops.int8_weight_quant(w.to(dev), pre.to(dev))
    qx, sx = ops.sq_quant_dynamic(x.to(dev), pre.to(dev))
    y = ops.int8_linear(qx, ops.repack_weight(qw), sw, sx, None, torch.float16)
    qw_ref, sw_ref = O.int8_weight_quant_device(to_np_f32(w), pre.numpy())
    qx_ref, sx_ref = O.sq_dynamic_quant(to_np_f32(x), pre.numpy())
    y_ref = O.int8_epilogue(O.gemm_i8_acc(qx_ref, qw_ref), sw_ref, sx_ref, None, "f16")
    assert np.array_equal(to_np_f32(y), y_ref)
    # and the quantised product approximates the unquantised one: (x*pre) . (w/pre) = x . w
    full = to_np_f32(x).astype(np.float64) @ to_np_f32(w).astype(np.float64).T
    assert np.sqrt(((y_ref - full) ** 2).mean()) < 0.08 * np.sqrt((full ** 2).mean())


# ---- unfused dequant (invokeSqOutputDequant, quant_kernels.cu:117-171,250-268) -------------------------------------------
@pytest.mark.parametrize("dt", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("per_token", [False, True])
@pytest.mark.parametrize("m,n", [(1024, 1280), (37, 642), (3, 2)])
def test_sq_output_dequant(ops, dev, dt, per_token, m, n):
    g = rng_t(500 + m + n)
    acc = torch.randint(-(2 ** 22), 2 ** 22, (m, n), generator=g, dtype=torch.int32)
    acc[0, 0] = 2 ** 24 + 1  # not an fp32 number: the int -> float conversion rounds
    acc[m - 1, n - 1] = -(2 ** 24) - 3
    s_in = (torch.rand(m if per_token else 1, generator=g) * 4e-2 + 1e-2).float()
    s_w = (torch.rand(n, generator=g) * 9e-3 + 1e-3).float()
    y = ops.sq_dequant(acc.to(dev), s_in.to(dev), s_w.to(dev), per_token, TORCH_DT[dt])
    y_ref = O.sq_output_dequant(acc.numpy(), s_in.numpy(), s_w.numpy(), per_token, dt)
    assert np.array_equal(to_np_f32(y), y_ref)
    if dt == "f32":  # the order (acc*s_in)*s_w is visible in fp32: the fused epilogue's (s_w*s_in)*acc differs somewhere
        other = acc.numpy().astype(np.float32) * (s_w.numpy()[None, :] * (s_in.numpy()[:, None] if per_token else s_in.numpy()[0]))
        assert m * n < 1000 or (other != y_ref).any()
    with pytest.raises(ValueError):
        ops.sq_dequant(acc.to(dev), s_in.to(dev), s_w[:-1].to(dev), per_token, TORCH_DT[dt])


def test_int32_gemm_then_unfused_dequant_matches_the_two_step_reference(ops, dev):
    """cublasMMWrapper's int32-output GEMM followed by invokeSqOutputDequant, the reference's unfused route."""
    m, n, k = 64, 128, 256
    g = rng_t(31)
    a = torch.randint(-128, 128, (m, k), generator=g, dtype=torch.int8)
    w = torch.randint(-127, 128, (n, k), generator=g, dtype=torch.int8)
    s_in = (torch.rand(m, generator=g) * 4e-2 + 1e-2).float()
    s_w = (torch.rand(n, generator=g) * 9e-3 + 1e-3).float()
    acc = ops.int8_linear(a.to(dev), ops.repack_weight(w.to(dev)), None, None, None, torch.int32)
    y = ops.sq_dequant(acc, s_in.to(dev), s_w.to(dev), True, torch.float16)
    acc_ref = O.gemm_i8_acc(a.numpy(), w.numpy())
    assert np.array_equal(acc.cpu().numpy(), acc_ref)
    assert np.array_equal(to_np_f32(y), O.sq_output_dequant(acc_ref, s_in.numpy(), s_w.numpy(), True, "f16"))
