"""GPU parity of the fusions around the FP8 linears of the FLUX blocks, through the C ABI.

What is compared with what:
  * gate/residual epilogue, codes-only epilogue (gelu 0/1), strided cast, LoRA merge, re-quantisation: BIT-EXACT
    against the CPU oracle applied to the plain GEMM output / the inputs.
  * gate+residual+adaLN+cast: the hidden state bit-exact against the oracle; the codes bit-exact against the
    library's own unfused layernorm_mod_fp8 on that hidden state (which test_gpu_layernorm.py holds against the
    oracle to one quantisation step).
  * gelu mode 2 and the whole blocks: tolerance (the kernel's GELU uses hardware exp/reciprocal): codes within one
    e4m3 step of the oracle, block outputs within 1e-2 relative / 2 fp16 ULP of an fp64 evaluation of the
    reference's call sequence on the same quantised operands.
"""
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


def _fp8_operands(ops, dev, m, n, k, seed, dt):
    g = rng_t(seed)
    t = TORCH_DT[dt]
    x = torch.randn(m, k, generator=g).to(t).to(dev)
    w = (0.05 * torch.randn(n, k, generator=g)).to(t).to(dev)
    qa, sa = ops.fp8_quant(x)
    qw, sw = ops.fp8_quant(w)
    bias = (0.1 * torch.randn(n, generator=g)).to(t).to(dev)
    return qa, sa, ops.repack_weight(qw), qw, sw, bias


def _step_ok(got, ref, what, frac=2e-2):
    """e4m3 codes equal, or one code apart (sign-magnitude codes: neighbours differ by 1) in a small fraction."""
    d = np.abs(got.astype(np.int32) - ref.astype(np.int32))
    # +0 and -0 (0x00 / 0x80) are the same value
    d = np.where(((got & 0x7F) == 0) & ((ref & 0x7F) == 0), 0, d)
    assert d.max() <= 1, f"{what}: codes differ by {d.max()} steps"
    assert (d != 0).mean() <= frac, f"{what}: {(d != 0).mean():.3%} of the codes differ"


@pytest.mark.parametrize("dt", ["bf16", "f16"])
@pytest.mark.parametrize("m,n,k,rpg", [(4608, 3072, 1024, 4608), (600, 256, 128, 77), (512, 128, 64, 128), (37, 64, 64, 5),
                                       (1024, 3072, 512, 512)])
def test_gemm_fp8_gated_matches_unfused_bit_for_bit(ops, dev, dt, m, n, k, rpg):
    qa, sa, wr, _, sw, bias = _fp8_operands(ops, dev, m, n, k, 100 + m + n, dt)
    g = rng_t(m * 3 + n)
    t = TORCH_DT[dt]
    nb = (m + rpg - 1) // rpg
    gate = torch.randn(nb, n, generator=g).to(t).to(dev)
    res = (2 * torch.randn(m, n, generator=g)).to(t).to(dev)
    plain = ops.fp8_linear(qa, wr, sa, sw, bias, out_dtype=t)
    want = O.gate_residual(to_np_f32(plain), to_np_f32(gate), to_np_f32(res), rpg, dt)
    got = ops.fp8_linear_gated(qa, wr, sa, sw, bias, gate, res, rpg)
    assert np.array_equal(to_np_f32(got), want)
    # in place on the residual, as the single block does with its input/output pair
    res2 = res.clone()
    out = ops.fp8_linear_gated(qa, wr, sa, sw, bias, gate, res2, rpg, out=res2)
    assert out.data_ptr() == res2.data_ptr() and np.array_equal(to_np_f32(res2), want)


@pytest.mark.parametrize("dt", ["bf16", "f16"])
@pytest.mark.parametrize("m,n,k,rpg", [(4608, 3072, 1024, 4608), (600, 256, 128, 77), (37, 64, 64, 5)])
def test_static_scale_ops_on_k_panels_give_the_row_major_bits(ops, dev, dt, m, n, k, rpg):
    """The FLUX blocks' static-scale sequence with its FP8 activations as k-panels [K/64, M, 64]: LayerNorm + cast kernels
    that write them, the GEMM that reads them and writes the next activation's codes as panels (also into a block of
    columns of a wider tensor), the gated GEMM that reads those."""
    t = TORCH_DT[dt]
    g = rng_t(m + 7 * n + k)
    qa, sa, wr, _, sw, bias = _fp8_operands(ops, dev, m, n, k, 300 + m + n, dt)
    qa_p = qa.view(m, k // 64, 64).permute(1, 0, 2).contiguous()
    nb = (m + rpg - 1) // rpg
    gate = torch.randn(nb, n, generator=g).to(t).to(dev)
    res = (2 * torch.randn(m, n, generator=g)).to(t).to(dev)
    assert torch.equal(ops.fp8_linear_gated_panels(qa_p, wr, sa, sw, bias, gate, res, rpg), ops.fp8_linear_gated(qa, wr, sa, sw, bias, gate, res, rpg))
    s_out = torch.tensor([0.013], dtype=torch.float32, device=dev)
    for gelu in (0, 2):
        dense = ops.fp8_linear_codes(qa, wr, sa, sw, bias, s_out, gelu=gelu, round_dtype=t)
        assert torch.equal(ops.fp8_panels_to_rows(ops.fp8_linear_codes_panels(qa_p, wr, sa, sw, bias, s_out, gelu=gelu, round_dtype=t)), dense)
        wide = torch.full(((128 + n + 64) // 64, m, 64), 0xAB, dtype=torch.uint8, device=dev)
        ops.fp8_linear_codes_panels(qa_p, wr, sa, sw, bias, s_out, gelu=gelu, round_dtype=t, out=wide, col_offset=128)
        rows = ops.fp8_panels_to_rows(wide)
        assert torch.equal(rows[:, 128:128 + n], dense) and (rows[:, :128] == 0xAB).all() and (rows[:, 128 + n:] == 0xAB).all()
    for tac in range(ops.gemm_tactic_count("fp8")):
        with ops.gemm_thread_tactic(tac):
            assert torch.equal(ops.fp8_panels_to_rows(ops.fp8_linear_codes_panels(qa_p, wr, sa, sw, bias, s_out, gelu=1, round_dtype=t)),
                               ops.fp8_linear_codes(qa, wr, sa, sw, bias, s_out, gelu=1, round_dtype=t)), tac
    # the static cast into a block of columns of wider panels
    xs = torch.randn(m, 128, generator=g).to(t).to(dev)
    wide = torch.full((5, m, 64), 0xAB, dtype=torch.uint8, device=dev)
    ops.fp8_scale_cast_panels(xs, s_out, out=wide, col_offset=64)
    rows = ops.fp8_panels_to_rows(wide)
    assert torch.equal(rows[:, 64:192], ops.fp8_scale_cast(xs, s_out)) and (rows[:, :64] == 0xAB).all() and (rows[:, 192:] == 0xAB).all()
    with pytest.raises(ValueError):
        ops.fp8_linear_codes_panels(qa_p, wr, sa, sw, bias, s_out, round_dtype=t, out=wide, col_offset=32)


@pytest.mark.parametrize("dt", ["bf16", "f16"])
@pytest.mark.parametrize("batch,seq,dim", [(2, 2304, 3072), (3, 50, 768), (1, 37, 2560)])
def test_layernorm_fp8_kernels_writing_k_panels(ops, dev, dt, batch, seq, dim):
    t = TORCH_DT[dt]
    g = rng_t(batch + seq + dim)
    x = (torch.randn(batch, seq, dim, generator=g) * 1.5).to(t).to(dev)
    attn = torch.randn(batch, seq, dim, generator=g).to(t).to(dev)
    gate, scale, shift = [(0.3 * torch.randn(batch, dim, generator=g)).to(t).to(dev) for _ in range(3)]
    s_a = torch.tensor([0.011], dtype=torch.float32, device=dev)
    s_b = torch.tensor([0.017], dtype=torch.float32, device=dev)
    rows = lambda q: ops.fp8_panels_to_rows(q).view(batch, seq, dim)
    q_p = ops.layernorm_mod_fp8(x, scale, shift, s_a, panels=True)
    assert q_p.shape == (dim // 64, batch * seq, 64) and torch.equal(rows(q_p), ops.layernorm_mod_fp8(x, scale, shift, s_a))
    qa_p, qb_p = ops.layernorm_mod_fp8_dual(x, scale, shift, s_a, s_b, panels=True)
    qa, qb = ops.layernorm_mod_fp8_dual(x, scale, shift, s_a, s_b)
    assert torch.equal(rows(qa_p), qa) and torch.equal(rows(qb_p), qb)
    q2_p, h_p = ops.gate_residual_layernorm_mod_fp8(attn, gate, x, scale, shift, s_a, panels=True)
    q2, h = ops.gate_residual_layernorm_mod_fp8(attn, gate, x, scale, shift, s_a)
    assert torch.equal(rows(q2_p), q2) and torch.equal(h_p, h)


def test_gemm_fp8_gated_every_tactic(ops, dev):
    m, n, k, rpg = 700, 512, 256, 300
    qa, sa, wr, _, sw, bias = _fp8_operands(ops, dev, m, n, k, 7, "bf16")
    g = rng_t(8)
    gate = torch.randn(3, n, generator=g).bfloat16().to(dev)
    res = torch.randn(m, n, generator=g).bfloat16().to(dev)
    try:
        for tac in range(ops.gemm_tactic_count("fp8")):
            ops.gemm_set_tactic("fp8", tac)
            plain = ops.fp8_linear(qa, wr, sa, sw, bias, out_dtype=torch.bfloat16)
            want = O.gate_residual(to_np_f32(plain), to_np_f32(gate), to_np_f32(res), rpg, "bf16")
            assert np.array_equal(to_np_f32(ops.fp8_linear_gated(qa, wr, sa, sw, bias, gate, res, rpg)), want), tac
    finally:
        ops.gemm_set_tactic("fp8", -1)


@pytest.mark.parametrize("dt", ["bf16", "f16"])
@pytest.mark.parametrize("gelu", [0, 1, 2])
def test_gemm_fp8_codes_into_a_column_block(ops, dev, dt, gelu):
    m, n, k, left, right = 520, 384, 256, 128, 64
    qa, sa, wr, _, sw, bias = _fp8_operands(ops, dev, m, n, k, 40 + gelu, dt)
    t = TORCH_DT[dt]
    s_out = torch.tensor([0.013], dtype=torch.float32, device=dev)
    dst = torch.full((m, left + n + right), 0xAB, dtype=torch.uint8, device=dev)
    ops.fp8_linear_codes(qa, wr, sa, sw, bias, s_out, gelu=gelu, round_dtype=t, out=dst, col_offset=left)
    got = dst.cpu().numpy()
    assert (got[:, :left] == 0xAB).all() and (got[:, left + n:] == 0xAB).all()
    if gelu < 2:
        plain = ops.fp8_linear(qa, wr, sa, sw, bias, gelu=bool(gelu), out_dtype=t)
        assert np.array_equal(got[:, left:left + n], O.fp8_scale_cast(to_np_f32(plain), s_out.cpu().numpy()[0], True))
        dense = ops.fp8_linear_codes(qa, wr, sa, sw, bias, s_out, gelu=gelu, round_dtype=t)
        assert np.array_equal(dense.cpu().numpy(), got[:, left:left + n])
    else:
        plain = ops.fp8_linear(qa, wr, sa, sw, bias, out_dtype=t)
        ref = O.cat_gelu(np.zeros((m, 0), np.float32), to_np_f32(plain), dt)
        _step_ok(got[:, left:left + n], O.fp8_scale_cast(ref, s_out.cpu().numpy()[0], True), "gelu of the rounded output")


@pytest.mark.parametrize("dt", ["bf16", "f16", "f32"])
def test_fp8_scale_cast_into_a_column_block(ops, dev, dt):
    m, c, w, off = 333, 96, 256, 64
    x = (3 * torch.randn(m, c, generator=rng_t(5))).to(TORCH_DT[dt])
    x[0, :4] = torch.tensor([float("nan"), float("inf"), -float("inf"), 1e4])
    s = torch.tensor([0.02], dtype=torch.float32, device=dev)
    dst = torch.full((m, w), 0x5A, dtype=torch.uint8, device=dev)
    ops.fp8_scale_cast_into(x.to(dev), s, dst, off)
    got = dst.cpu().numpy()
    assert np.array_equal(got[:, off:off + c], O.fp8_scale_cast(to_np_f32(x), s.cpu().numpy()[0], True))
    assert (got[:, :off] == 0x5A).all() and (got[:, off + c:] == 0x5A).all()
    from lyradiff_amd.lib import LyraQuantError

    with pytest.raises(LyraQuantError):
        ops.fp8_scale_cast_into(x[:, :40].contiguous().to(dev), s, dst, 0)  # 40 columns: rows not 16-byte multiples
    with pytest.raises(ValueError):
        ops.fp8_scale_cast_into(x.to(dev), s, dst, w - c + 16)


@pytest.mark.parametrize("dt", ["bf16", "f16"])
@pytest.mark.parametrize("batch,seq,dim", [(1, 4608, 3072), (2, 300, 768), (3, 7, 3072)])
def test_gate_residual_layernorm_mod_fp8(ops, dev, dt, batch, seq, dim):
    g = rng_t(batch * 1000 + seq + dim)
    t = TORCH_DT[dt]
    x = (1.5 * torch.randn(batch, seq, dim, generator=g)).to(t)
    attn = torch.randn(batch, seq, dim, generator=g).to(t)
    gate, scale, shift = ((0.4 * torch.randn(batch, dim, generator=g)).to(t) for _ in range(3))
    s_in = torch.tensor([0.012], dtype=torch.float32)
    q, hidden = ops.gate_residual_layernorm_mod_fp8(attn.to(dev), gate.to(dev), x.to(dev), scale.to(dev), shift.to(dev), s_in.to(dev))
    want_h = O.gate_residual(to_np_f32(attn).reshape(-1, dim), to_np_f32(gate), to_np_f32(x).reshape(-1, dim), seq, dt)
    assert np.array_equal(to_np_f32(hidden).reshape(-1, dim), want_h)
    q_unfused = ops.layernorm_mod_fp8(hidden, scale.to(dev), shift.to(dev), s_in.to(dev))
    assert torch.equal(q, q_unfused)
    ref, _ = O.gate_residual_layernorm_mod_fp8(to_np_f32(attn).reshape(-1, dim), to_np_f32(gate), to_np_f32(x).reshape(-1, dim),
                                               to_np_f32(scale), to_np_f32(shift), s_in.numpy(), seq, dt)
    assert (q.cpu().numpy().reshape(-1, dim) != ref).mean() <= 5e-3
    # in place: the hidden state may overwrite the block input
    xin = x.to(dev).clone()
    q2, h2 = ops.gate_residual_layernorm_mod_fp8(attn.to(dev), gate.to(dev), xin, scale.to(dev), shift.to(dev), s_in.to(dev), hidden_out=xin)
    assert h2.data_ptr() == xin.data_ptr() and torch.equal(h2, hidden) and torch.equal(q2, q)


def test_layernorm_mod_fp8_dual_equals_two_single_calls(ops, dev):
    g = rng_t(77)
    x = (1.5 * torch.randn(2, 513, 3072, generator=g)).bfloat16().to(dev)
    scale, shift = ((0.3 * torch.randn(2, 3072, generator=g)).bfloat16().to(dev) for _ in range(2))
    sa = torch.tensor([0.011], dtype=torch.float32, device=dev)
    sb = torch.tensor([0.017], dtype=torch.float32, device=dev)
    qa, qb = ops.layernorm_mod_fp8_dual(x, scale, shift, sa, sb)
    assert torch.equal(qa, ops.layernorm_mod_fp8(x, scale, shift, sa))
    assert torch.equal(qb, ops.layernorm_mod_fp8(x, scale, shift, sb))
    assert not torch.equal(qa, qb)


@pytest.mark.parametrize("dt", ["bf16", "f16", "f32"])
def test_load_lora_merge(ops, dev, dt):
    g = rng_t(3)
    t = TORCH_DT[dt]
    w = (0.05 * torch.randn(1000, 96, generator=g)).to(t)
    l = (0.01 * torch.randn(1000, 96, generator=g)).to(t)
    for alpha in (1.0, 0.7, -0.33):
        got = ops.load_lora(w.to(dev).clone(), l.to(dev), alpha)
        assert np.array_equal(to_np_f32(got), O.load_lora(to_np_f32(w), to_np_f32(l), alpha, dt)), alpha


def test_fp8_linear_lora_requantise_and_clear(ops, dev):
    from lyradiff_amd.weights import load_fp8_linear

    g = rng_t(9)
    d_out, d_in = 256, 192
    sd = {"blk.net.2.weight": (0.04 * torch.randn(d_out, d_in, generator=g)).bfloat16(),
          "blk.net.2.bias": torch.randn(d_out, generator=g).bfloat16(),
          "blk.net.2_input_scale": torch.tensor([0.02])}
    lin = load_fp8_linear(sd, "blk.", "net.2", d_out, d_in, torch.bfloat16, dev, keep_master=True)
    codes0, scale0 = ops.unpack_weight(lin.weight_rows32).cpu().numpy(), float(lin.weight_scale.cpu()[0])
    ref_codes0, ref_s0 = O.fp8_requantise(to_np_f32(sd["blk.net.2.weight"]))
    assert np.array_equal(codes0, ref_codes0) and scale0 == float(ref_s0)
    ptr = lin.weight_rows32.data_ptr()
    delta = (0.02 * torch.randn(d_out, d_in, generator=g)).bfloat16()
    delta[3, 5] = 1.0  # raises the per-tensor maximum, so the scale must change
    lin.load_lora(delta, 0.8)
    merged = O.load_lora(to_np_f32(sd["blk.net.2.weight"]), to_np_f32(delta), 0.8, "bf16")
    ref_codes, ref_s = O.fp8_requantise(merged)
    assert lin.weight_rows32.data_ptr() == ptr
    assert float(lin.weight_scale.cpu()[0]) == float(ref_s) and float(ref_s) > scale0
    assert np.array_equal(ops.unpack_weight(lin.weight_rows32).cpu().numpy(), ref_codes)
    lin.clear_lora()
    assert float(lin.weight_scale.cpu()[0]) == scale0
    assert np.array_equal(ops.unpack_weight(lin.weight_rows32).cpu().numpy(), codes0)
    with pytest.raises(RuntimeError):
        load_fp8_linear(sd, "blk.", "net.2", d_out, d_in, torch.bfloat16, dev).load_lora(delta, 1.0)


def _state_dict(names_shapes, seed, scale_w=0.03, prefix="p."):
    g = rng_t(seed)
    sd = {}
    for name, (n, k) in names_shapes.items():
        sd[f"{prefix}{name}.weight"] = (scale_w * torch.randn(n, k, generator=g)).bfloat16()
        sd[f"{prefix}{name}.bias"] = (0.1 * torch.randn(n, generator=g)).bfloat16()
    return sd


def test_flux_attn_post_fp8_block(ops, dev):
    """Three fused launches == the reference's seven-step sequence run with this library's unfused kernels, bit for
    bit; and both within tolerance of an fp64 evaluation on the same quantised operands."""
    from lyradiff_amd import flux_fp8 as F

    b, s, d = 2, 320, 512
    g = rng_t(21)
    sd = _state_dict({"net.0.proj": (4 * d, d), "net.2": (d, 4 * d)}, 22)
    sd["p.net.0.proj_input_scale"] = torch.tensor([4.5 / 448])
    sd["p.net.2_input_scale"] = torch.tensor([3.0 / 448])
    w = F.load_flux_attn_post_fp8(sd, "p.", d, torch.bfloat16, dev)
    x = torch.randn(b, s, d, generator=g).bfloat16().to(dev)
    attn = torch.randn(b, s, d, generator=g).bfloat16().to(dev)
    msa = (0.5 * torch.randn(6, b, d, generator=g)).bfloat16().to(dev)
    out = F.flux_attn_post_fp8(x, attn, msa, w)
    # the same sequence, one kernel (or one T-rounded torch op) per reference launch
    hidden = x + msa[2][:, None, :] * attn
    q1 = ops.layernorm_mod_fp8(hidden, msa[4].contiguous(), msa[3].contiguous(), w.gelu_proj.input_scale)
    inner = ops.fp8_linear(q1.view(b * s, d), w.gelu_proj.weight_rows32, w.gelu_proj.input_scale, w.gelu_proj.weight_scale,
                           w.gelu_proj.bias, gelu=True, out_dtype=torch.bfloat16)
    q2 = ops.fp8_scale_cast(inner, w.ff_linear.input_scale)
    ff = ops.fp8_linear(q2, w.ff_linear.weight_rows32, w.ff_linear.input_scale, w.ff_linear.weight_scale, w.ff_linear.bias,
                        out_dtype=torch.bfloat16)
    unfused = hidden + msa[5][:, None, :] * ff.view(b, s, d)
    assert torch.equal(out, unfused)
    # fp64 evaluation from the second GEMM's quantised operands
    w2 = O.e4m3_decode(ops.unpack_weight(w.ff_linear.weight_rows32).cpu().numpy()).astype(np.float64)
    y = (O.e4m3_decode(q2.cpu().numpy()).astype(np.float64) @ w2.T) * float(w.ff_linear.input_scale.cpu()[0]) \
        * float(w.ff_linear.weight_scale.cpu()[0]) + to_np_f32(w.ff_linear.bias).astype(np.float64)[None, :]
    ref = to_np_f32(hidden).reshape(-1, d).astype(np.float64) + np.repeat(to_np_f32(msa[5]).astype(np.float64), s, axis=0) * y
    # the sequence rounds ff, gate*ff and the sum to bf16 (unit roundoff 2^-8 each): where hidden and gate*ff cancel,
    # the error is relative to their size, not to the small result
    assert_close_tol(to_np_f32(out).reshape(-1, d), ref.astype(np.float32), "flux attn-post block",
                     abs_floor=2.0 ** -6 * (np.abs(to_np_f32(hidden).reshape(-1, d)) + np.abs(ref)))


def test_flux_single_mlp_fp8_block(ops, dev):
    from lyradiff_amd import flux_fp8 as F

    b, s, d, ms = 2, 200, 256, 4
    g = rng_t(31)
    sd = _state_dict({"proj_mlp": (ms * d, d), "proj_out": (d, (ms + 1) * d)}, 32)
    sd["p.proj_mlp_input_scale"] = torch.tensor([4.0 / 448])
    sd["p.proj_out_input_scale"] = torch.tensor([4.0 / 448])
    w = F.load_flux_single_mlp_fp8(sd, "p.", d, ms, torch.bfloat16, dev)
    x = torch.randn(b, s, d, generator=g).bfloat16().to(dev)
    norm_hidden = torch.randn(b, s, d, generator=g).bfloat16().to(dev)
    attn = torch.randn(b, s, d, generator=g).bfloat16().to(dev)
    gate = (0.5 * torch.randn(b, d, generator=g)).bfloat16().to(dev)
    out = F.flux_single_mlp_fp8(x, norm_hidden, attn, gate, w)
    # codes in, same result
    q1 = ops.fp8_scale_cast(norm_hidden, w.proj_mlp.input_scale)
    assert torch.equal(out, F.flux_single_mlp_fp8(x, q1, attn, gate, w))
    # the reference's sequence on the CPU oracle, from this library's plain GEMM output
    mlp = ops.fp8_linear(q1.view(b * s, d), w.proj_mlp.weight_rows32, w.proj_mlp.input_scale, w.proj_mlp.weight_scale,
                         w.proj_mlp.bias, out_dtype=torch.bfloat16)
    cat = O.cat_gelu(to_np_f32(attn).reshape(-1, d), to_np_f32(mlp), "bf16")
    q2_ref = O.fp8_scale_cast(cat, float(w.proj_out.input_scale.cpu()[0]), True)
    wo = O.e4m3_decode(ops.unpack_weight(w.proj_out.weight_rows32).cpu().numpy()).astype(np.float64)
    y = (O.e4m3_decode(q2_ref).astype(np.float64) @ wo.T) * float(w.proj_out.input_scale.cpu()[0]) \
        * float(w.proj_out.weight_scale.cpu()[0]) + to_np_f32(w.proj_out.bias).astype(np.float64)[None, :]
    ref = to_np_f32(x).reshape(-1, d).astype(np.float64) + np.repeat(to_np_f32(gate).astype(np.float64), s, axis=0) * y
    # the GELU'd codes may sit one e4m3 step from the oracle's in a small fraction of places: allow what such steps
    # move the projection by (a few 2^-4 relative steps of single terms), on top of the stated tolerance
    assert_close_tol(to_np_f32(out).reshape(-1, d), ref.astype(np.float32), "flux single-block mlp",
                     abs_floor=2.0 ** -6 * (np.abs(to_np_f32(x).reshape(-1, d)) + np.abs(ref)) + 0.02)


# ---- W4A4 linears with the same epilogues (FLUX INT4 blocks) ---------------------------------------------------------
def _w4a4_operands(ops, dev, m, n, k, seed, dt, rank=32):
    g = rng_t(seed)
    t = TORCH_DT[dt]
    x = torch.randn(m, k, generator=g).to(t).to(dev)
    w = (0.05 * torch.randn(n, k, generator=g)).to(t).to(dev)
    qa, sa = ops.w4a4_quant(x, None, torch.float32)
    qw, sw = ops.w4a4_quant(w, None, torch.float32)
    wr = ops.repack_weight(qw.view(torch.uint8).view(n, k // 2))
    bias = (0.1 * torch.randn(n, generator=g)).to(t).to(dev)
    la = (0.3 * torch.randn(m, rank, generator=g)).to(t).to(dev)
    lu = (0.1 * torch.randn(n, rank, generator=g)).to(t).to(dev)
    return qa, sa, wr, sw, bias, la, lu


@pytest.mark.parametrize("dt", ["bf16", "f16"])
@pytest.mark.parametrize("m,n,k,rpg", [(4608, 256, 512, 4608), (300, 128, 256, 77), (64, 3072, 128, 64)])
def test_gemm_w4a4_epilogue_options_match_the_unfused_sequence(ops, dev, dt, m, n, k, rpg):
    qa, sa, wr, sw, bias, la, lu = _w4a4_operands(ops, dev, m, n, k, 500 + m + n, dt)
    g = rng_t(m + 7 * n)
    t = TORCH_DT[dt]
    gate = torch.randn((m + rpg - 1) // rpg, n, generator=g).to(t).to(dev)
    res = (2 * torch.randn(m, n, generator=g)).to(t).to(dev)
    add = torch.randn(m, n, generator=g).to(t).to(dev)
    s_out = torch.tensor([0.02], dtype=torch.float32, device=dev)
    plain = ops.w4a4_linear(qa, wr, sa, sw, bias, t, 64, la, lu)
    p32 = to_np_f32(plain)
    # addend, then gate and residual: every step rounded to T
    joined = O.round_to(p32 + to_np_f32(add), dt)
    want = O.gate_residual(joined, to_np_f32(gate), to_np_f32(res), rpg, dt)
    got = ops.w4a4_linear(qa, wr, sa, sw, bias, t, 64, la, lu, addend=add, gate=gate, residual=res, rows_per_gate=rpg)
    assert np.array_equal(to_np_f32(got), want)
    assert np.array_equal(to_np_f32(ops.w4a4_linear(qa, wr, sa, sw, bias, t, 64, la, lu, addend=add)), joined)
    # e4m3 codes of the plain output, next to the output and alone, dense and into a column block
    c, codes = ops.w4a4_linear(qa, wr, sa, sw, bias, t, 64, la, lu, out_fp8_scale=s_out)
    ref_codes = O.fp8_scale_cast(p32, s_out.cpu().numpy()[0], True)
    assert torch.equal(c, plain) and np.array_equal(codes.cpu().numpy(), ref_codes)
    wide = torch.full((m, n + 96), 0x11, dtype=torch.uint8, device=dev)
    only = ops.w4a4_linear(qa, wr, sa, sw, bias, t, 64, la, lu, out_fp8_scale=s_out, out_fp8=wide, col_offset=32, want_output=False)
    got_wide = only.cpu().numpy()
    assert np.array_equal(got_wide[:, 32:32 + n], ref_codes) and (got_wide[:, :32] == 0x11).all() and (got_wide[:, 32 + n:] == 0x11).all()
    # GELU of the rounded output: tolerance (hardware exp / reciprocal in the kernel)
    gl = to_np_f32(ops.w4a4_linear(qa, wr, sa, sw, bias, t, 64, la, lu, gelu=2))
    ref = O.cat_gelu(np.zeros((m, 0), np.float32), p32, dt)
    ulp = 2.0 ** (-7 if dt == "bf16" else -10)
    assert np.all(np.abs(gl - ref) <= ulp * np.abs(ref) + 1e-6)


def _int4_state(prefix, n, k, g, rank=32, bias=True, lora_scale=0.05):
    """Host-side W4A4 weight container entries with the reference's key names."""
    w = 0.05 * torch.randn(n, k, generator=g)
    wv = w.view(n, k // 64, 64)
    sc = wv.abs().amax(dim=2) / 7.0
    q = torch.clamp(torch.round(wv / sc[..., None]), -8, 7).to(torch.int16).view(n, k)
    packed = ((q[:, 0::2] & 0xF) | ((q[:, 1::2] & 0xF) << 4)).to(torch.uint8).view(torch.int8)
    sd = {prefix + "packed_weight": packed.contiguous(), prefix + "weight_scale": sc.float().contiguous(),
          prefix + "smooth": (0.5 + torch.rand(k, generator=g)).float(),
          prefix + "lora_up": (lora_scale * torch.randn(n, rank, generator=g)).bfloat16(),
          prefix + "lora_down": (lora_scale * torch.randn(rank, k, generator=g)).bfloat16()}
    if bias:
        sd[prefix + "bias"] = (0.1 * torch.randn(n, generator=g)).bfloat16()
    return sd


def test_flux_attn_post_int4_block(ops, dev):
    from lyradiff_amd import flux_int4 as F

    b, s, d = 2, 192, 256
    g = rng_t(61)
    sd = _int4_state("p.net.0.proj.", 4 * d, d, g)
    sd.update(_state_dict({"net.2": (d, 4 * d)}, 62))
    sd["p.net.2_input_scale"] = torch.tensor([3.0 / 448])
    w = F.load_flux_attn_post_int4(sd, "p.", d, torch.bfloat16, dev)
    x = torch.randn(b, s, d, generator=g).bfloat16().to(dev)
    attn = torch.randn(b, s, d, generator=g).bfloat16().to(dev)
    msa = (0.5 * torch.randn(6, b, d, generator=g)).bfloat16().to(dev)
    out = F.flux_attn_post_int4(x, attn, msa, w)
    # the reference's sequence with this library's unfused kernels and T-rounded torch ops
    hidden = x + msa[2][:, None, :] * attn
    norm = ops.gate_residual_layernorm_mod(hidden, msa[4], msa[3])
    assert torch.equal(norm, ops.gate_residual_layernorm_mod(x, msa[4], msa[3], attn, msa[2])[0])
    inner = w.gelu_proj.forward(norm.view(b * s, d))                              # GEMM + low-rank + bias
    inner = torch.nn.functional.gelu(inner.float(), approximate="tanh").bfloat16()
    q2 = ops.fp8_scale_cast(inner, w.ff_linear.input_scale)
    ff = ops.fp8_linear(q2, w.ff_linear.weight_rows32, w.ff_linear.input_scale, w.ff_linear.weight_scale, w.ff_linear.bias,
                        out_dtype=torch.bfloat16)
    seq = hidden + msa[5][:, None, :] * ff.view(b, s, d)
    # differences come only from the GELU flavour (codes one e4m3 step apart in a few places)
    assert_close_tol(to_np_f32(out).reshape(-1, d), to_np_f32(seq).reshape(-1, d), "flux int4 attn-post block",
                     abs_floor=2.0 ** -6 * (np.abs(to_np_f32(hidden).reshape(-1, d)) + np.abs(to_np_f32(seq).reshape(-1, d))) + 0.02)


def test_flux_single_mlp_int4_block(ops, dev):
    from lyradiff_amd import flux_int4 as F

    b, s, d, ms = 2, 160, 256, 4
    g = rng_t(71)
    sd = _int4_state("p.proj_mlp.", ms * d, d, g)
    sd.update(_int4_state("p.proj_out.linears.0.", d, d, g))
    sd.update(_int4_state("p.proj_out.linears.1.linear.", d, ms * d, g, bias=False))
    w = F.load_flux_single_mlp_int4(sd, "p.", d, ms, torch.bfloat16, dev)
    x, norm, attn = (torch.randn(b, s, d, generator=g).bfloat16().to(dev) for _ in range(3))
    gate = (0.5 * torch.randn(b, d, generator=g)).bfloat16().to(dev)
    out = F.flux_single_mlp_int4(x, norm, attn, gate, w)
    m = b * s
    mlp = torch.nn.functional.gelu(w.proj_mlp.forward(norm.view(m, d)).float(), approximate="tanh").bfloat16()
    h1 = w.proj_out_1.forward(attn.view(m, d))
    h2 = w.proj_out_2.forward(mlp)
    seq = x + gate[:, None, :] * (h1 + h2).view(b, s, d)
    assert_close_tol(to_np_f32(out).reshape(-1, d), to_np_f32(seq).reshape(-1, d), "flux int4 single-block tail",
                     abs_floor=2.0 ** -6 * (np.abs(to_np_f32(x).reshape(-1, d)) + np.abs(to_np_f32(seq).reshape(-1, d))) + 0.03)


def test_new_entry_points_reject_bad_arguments_and_accept_empty_inputs(ops, dev):
    """Error paths return a status and a message (nothing is launched); zero rows is a no-op."""
    from lyradiff_amd.lib import LyraQuantError

    qa, sa, wr, _, sw, bias = _fp8_operands(ops, dev, 64, 128, 64, 3, "bf16")
    gate = torch.ones(1, 128, dtype=torch.bfloat16, device=dev)
    res = torch.zeros(64, 128, dtype=torch.bfloat16, device=dev)
    s_out = torch.tensor([0.02], dtype=torch.float32, device=dev)
    with pytest.raises(ValueError):  # gate has the wrong number of rows for rows_per_gate
        ops.fp8_linear_gated(qa, wr, sa, sw, bias, gate, res, 16)
    with pytest.raises(LyraQuantError, match="gelu"):
        ops.fp8_linear_codes(qa, wr, sa, sw, bias, s_out, gelu=3)
    with pytest.raises(ValueError):  # destination too narrow for the column offset
        ops.fp8_linear_codes(qa, wr, sa, sw, bias, s_out, out=torch.empty(64, 160, dtype=torch.uint8, device=dev), col_offset=64)
    with pytest.raises(LyraQuantError, match="ldc"):  # row pitch not a multiple of 4
        ops.fp8_linear_codes(qa, wr, sa, sw, bias, s_out, out=torch.empty(64, 130, dtype=torch.uint8, device=dev))
    with pytest.raises(TypeError):
        ops.fp8_linear_gated(qa, wr, sa, sw, bias, gate.half(), res, 64)
    # zero rows: no launch, empty results
    e = torch.empty(0, 64, dtype=torch.uint8, device=dev)
    assert ops.fp8_linear_codes(e, wr, sa, sw, bias, s_out).shape == (0, 128)
    assert ops.fp8_linear_gated(e, wr, sa, sw, bias, gate[:0], res[:0], 1).shape == (0, 128)
    x0 = torch.empty(2, 0, 128, dtype=torch.bfloat16, device=dev)
    mod = torch.zeros(2, 128, dtype=torch.bfloat16, device=dev)
    q, h = ops.gate_residual_layernorm_mod_fp8(x0, mod, x0, mod, mod, s_out)
    assert q.shape == (2, 0, 128) and h.shape == (2, 0, 128)
    # NaN and infinity travel through the gate/residual epilogue and the codes as in the unfused kernels
    qa2 = qa.clone()
    sa_nan = torch.tensor([float("nan")], dtype=torch.float32, device=dev)
    y = ops.fp8_linear_gated(qa2, wr, sa_nan, sw, bias, gate, res, 64)
    assert torch.isnan(y).all()
    codes = ops.fp8_linear_codes(qa2, wr, sa_nan, sw, bias, s_out)
    assert ((codes & 0x7F) == 0x7F).all()


@pytest.mark.parametrize("batch", [1, 3])
def test_ada_fp8_layernorm(ops, dev, batch):
    from lyradiff_amd import flux_fp8 as F

    s, d, nch = 96, 256, 6
    g = rng_t(80 + batch)
    sd = _state_dict({"linear": (nch * d, d)}, 81)
    sd["p.linear_input_scale"] = torch.tensor([4.0 / 448])
    lin = F.load_ada_fp8_layernorm(sd, "p.", d, nch, torch.bfloat16, dev)
    x = torch.randn(batch, s, d, generator=g).bfloat16().to(dev)
    temb = torch.randn(batch, d, generator=g).bfloat16().to(dev)
    norm, msa = F.ada_fp8_layernorm(x, temb, lin, nch)
    assert msa.shape == (nch, batch, d) and norm.shape == x.shape
    # msa against the oracle's FP8 GEMM contract on the same codes, chunk-major
    q = O.fp8_scale_cast(to_np_f32(temb), float(lin.input_scale.cpu()[0]), True)
    wq = ops.unpack_weight(lin.weight_rows32).cpu().numpy()
    ref = O.fp8_gemm(q, wq, lin.input_scale.cpu().numpy(), lin.weight_scale.cpu().numpy(), to_np_f32(lin.bias), out_dtype="bf16")
    ref = ref.reshape(batch, nch, d).transpose(1, 0, 2)
    assert_close_tol(to_np_f32(msa), ref, "ada layernorm msa", abs_floor=2.0 ** -8 * np.abs(ref) + 1e-3)
    # the normalised tensor and its fused-cast forms all come from the same kernel arithmetic
    s1 = torch.tensor([0.02], dtype=torch.float32, device=dev)
    s2 = torch.tensor([0.03], dtype=torch.float32, device=dev)
    assert torch.equal(norm, ops.gate_residual_layernorm_mod(x, msa[1].contiguous(), msa[0].contiguous()))
    c1, _ = F.ada_fp8_layernorm(x, temb, lin, nch, (s1,))
    assert torch.equal(c1, ops.fp8_scale_cast(norm, s1))
    (ca, cb), _ = F.ada_fp8_layernorm(x, temb, lin, nch, (s1, s2))
    assert torch.equal(ca, c1) and torch.equal(cb, ops.fp8_scale_cast(norm, s2))
    sw, _ = F.ada_fp8_layernorm(x, temb, lin, nch, switch_scale=True)
    assert torch.equal(sw, ops.gate_residual_layernorm_mod(x, msa[0].contiguous(), msa[1].contiguous()))
    # 16-bit output against the oracle's adaLN (statistics order differs: one ULP of T)
    y = to_np_f32(norm).reshape(-1, d)
    n = O._ln_normalised(to_np_f32(x).reshape(-1, d), 1e-6)
    bidx = np.arange(batch * s) // s
    want = O.round_to(O.round_to(O.round_to(to_np_f32(msa[1])[bidx] + 1.0, "bf16") * O.round_to(n, "bf16"), "bf16") + to_np_f32(msa[0])[bidx], "bf16")
    assert (y != want).mean() < 0.02 and np.all(np.abs(y - want) <= 2.0 ** -7 * (np.abs(want) + np.abs(to_np_f32(msa[0])[bidx]) + 1.0))


def _toy_attention(heads):
    """q/k/v split + scaled-dot-product attention in fp32 torch: stands in for the caller's (unquantized) attention."""
    def run(qkv):
        b, s, d3 = qkv.shape
        d = d3 // 3
        q, k, v = (t.reshape(b, s, heads, d // heads).transpose(1, 2).float() for t in qkv.split(d, dim=-1))
        o = torch.nn.functional.scaled_dot_product_attention(q, k, v)
        return o.transpose(1, 2).reshape(b, s, d).to(qkv.dtype)
    return run


def test_whole_fp8_blocks_around_a_caller_supplied_attention(ops, dev):
    from lyradiff_amd import flux_fp8 as F

    b, s, sc, d = 2, 96, 32, 256
    g = rng_t(91)
    names = {"norm.linear": (3 * d, d), "attn.to_qkv": (3 * d, d), "proj_mlp": (4 * d, d), "proj_out": (d, 5 * d),
             "norm1.linear": (6 * d, d), "norm1_context.linear": (6 * d, d), "attn.to_added_qkv": (3 * d, d),
             "attn.to_out.0": (d, d), "attn.to_add_out": (d, d), "ff.net.0.proj": (4 * d, d), "ff.net.2": (d, 4 * d),
             "ff_context.net.0.proj": (4 * d, d), "ff_context.net.2": (d, 4 * d)}
    sd = _state_dict(names, 92)
    for n in names:
        sd[f"p.{n}_input_scale"] = torch.tensor([5.0 / 448])
    x = torch.randn(b, s, d, generator=g).bfloat16().to(dev)
    ctx = torch.randn(b, sc, d, generator=g).bfloat16().to(dev)
    temb = torch.randn(b, d, generator=g).bfloat16().to(dev)
    att = _toy_attention(4)
    # single block == the same steps called one by one
    ws = F.load_flux_single_block_fp8(sd, "p.", d, 4, torch.bfloat16, dev)
    out = F.flux_single_block_fp8(x, temb, ws, att)
    norm, msa = F.ada_fp8_layernorm(x, temb, ws.norm, 3)
    qkv = ws.to_qkv.forward(norm)
    want = F.flux_single_mlp_fp8(x, norm, att(qkv), msa[2].contiguous(), ws.mlp)
    assert out.shape == x.shape and torch.equal(out, want) and torch.isfinite(out.float()).all()
    # double block likewise, both streams
    wd = F.load_flux_double_block_fp8(sd, "p.", d, torch.bfloat16, dev)

    def joint(qkv, cqkv):
        o = att(torch.cat([cqkv, qkv], dim=1))
        return o[:, cqkv.shape[1]:], o[:, :cqkv.shape[1]]

    o1, o2 = F.flux_double_block_fp8(x, ctx, temb, wd, joint)
    n1, m1 = F.ada_fp8_layernorm(x, temb, wd.norm1, 6)
    n2, m2 = F.ada_fp8_layernorm(ctx, temb, wd.norm1_context, 6)
    a1, a2 = joint(wd.to_qkv.forward(n1), wd.to_added_qkv.forward(n2))
    w1 = F.flux_attn_post_fp8(x, wd.to_out.forward(a1.contiguous()), m1, wd.ff)
    w2 = F.flux_attn_post_fp8(ctx, wd.to_add_out.forward(a2.contiguous()), m2, wd.ff_context)
    assert torch.equal(o1, w1) and torch.equal(o2, w2) and o2.shape == ctx.shape


def _rope_table(b, s, dh, seed):
    """[B, S, Dh/2, 2, 2] rotation matrices [[cos, -sin], [sin, cos]] as FLUX's EmbedND produces them."""
    ang = torch.rand(b, s, dh // 2, generator=rng_t(seed)) * 6.28
    return torch.stack([torch.cos(ang), -torch.sin(ang), torch.sin(ang), torch.cos(ang)], dim=-1).reshape(b, s, dh // 2, 2, 2)


def _attention_reference(qkv, cqkv, norms, rope, heads):
    """Independent fp64 restatement: RMSNorm per head, rotation written with complex numbers, softmax attention."""
    def prep(t, wq, wk, rp):
        b, s, d3 = t.shape
        dh = d3 // 3 // heads
        q, k, v = t.double().view(b, s, 3, heads, dh).unbind(2)
        rot = torch.complex(rp[..., 0, 0].double(), rp[..., 1, 0].double()).unsqueeze(2)  # cos + i sin, [B, S, 1, Dh/2]

        def one(x, w):
            n = x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6) * w.double()
            z = torch.view_as_complex(n.reshape(b, s, heads, dh // 2, 2).contiguous()) * rot
            return torch.view_as_real(z).reshape(b, s, heads, dh)

        return one(q, wq), one(k, wk), v

    s, sc = qkv.shape[1], (cqkv.shape[1] if cqkv is not None else 0)
    if cqkv is None:
        q, k, v = prep(qkv, norms[0], norms[1], rope)
    else:
        a = prep(cqkv, norms[2], norms[3], rope[:, :sc])
        c = prep(qkv, norms[0], norms[1], rope[:, sc:])
        q, k, v = (torch.cat([a[i], c[i]], dim=1) for i in range(3))
    w = torch.softmax(torch.einsum("bshd,bthd->bhst", q, k) / q.shape[-1] ** 0.5, dim=-1)
    o = torch.einsum("bhst,bthd->bshd", w, v).reshape(q.shape[0], sc + s, -1)
    return (o[:, sc:], o[:, :sc]) if cqkv is not None else o


def test_flux_attention_core_matches_an_independent_restatement(dev):
    from lyradiff_amd.flux_ops import flux_attention_core

    b, s, sc, heads, dh = 2, 80, 24, 4, 64
    d = heads * dh
    g = rng_t(301)
    qkv = torch.randn(b, s, 3 * d, generator=g).bfloat16()
    cqkv = torch.randn(b, sc, 3 * d, generator=g).bfloat16()
    norms = [(1 + 0.2 * torch.randn(dh, generator=g)).bfloat16() for _ in range(4)]
    rope = _rope_table(b, sc + s, dh, 302).bfloat16()
    got, cgot = flux_attention_core(qkv.to(dev), norms[0].to(dev), norms[1].to(dev), rope.to(dev), heads, cqkv.to(dev),
                                    norms[2].to(dev), norms[3].to(dev))
    want, cwant = _attention_reference(qkv, cqkv, norms, rope, heads)
    # bf16 q/k/v and a bf16 output: a few units of 2^-8 relative to the magnitude of v
    assert (got.cpu().double() - want).abs().max() < 0.05 and (cgot.cpu().double() - cwant).abs().max() < 0.05
    single = flux_attention_core(qkv.to(dev), norms[0].to(dev), norms[1].to(dev), rope[:, sc:].contiguous().to(dev), heads)
    assert (single.cpu().double() - _attention_reference(qkv, None, norms, rope[:, sc:], heads)).abs().max() < 0.05


def test_flux_block_ops_have_the_reference_interface(ops, dev):
    """torch.classes.lyradiff.FluxTransformerBlockOp / FluxSingleTransformerBlockOp call sites
    (lyradiff_flux_transformer_model_v2.py:77-168): constructor, initialize, reload_model_from_state_dict, forward,
    load_lora_by_name, clear_lora; outputs equal the block functions driven with the same attention core."""
    from lyradiff_amd import flux_fp8 as F
    from lyradiff_amd import flux_ops as FO

    b, s, sc, heads, dh = 2, 96, 32, 4, 64
    d = heads * dh
    g = rng_t(311)
    names = {"norm.linear": (3 * d, d), "attn.to_qkv": (3 * d, d), "proj_mlp": (4 * d, d), "proj_out": (d, 5 * d),
             "norm1.linear": (6 * d, d), "norm1_context.linear": (6 * d, d), "attn.to_added_qkv": (3 * d, d),
             "attn.to_out.0": (d, d), "attn.to_add_out": (d, d), "ff.net.0.proj": (4 * d, d), "ff.net.2": (d, 4 * d),
             "ff_context.net.0.proj": (4 * d, d), "ff_context.net.2": (d, 4 * d)}
    sd = _state_dict(names, 312, prefix="transformer_blocks.3.")
    sd.update(_state_dict(names, 313, prefix="single_transformer_blocks.5."))
    for pre in ("transformer_blocks.3.", "single_transformer_blocks.5."):
        for n in names:
            sd[f"{pre}{n}_input_scale"] = torch.tensor([5.0 / 448])
        for n in ("norm_q", "norm_k", "norm_added_q", "norm_added_k"):
            sd[f"{pre}attn.{n}.weight"] = (1 + 0.1 * torch.randn(dh, generator=g)).bfloat16()
    x = torch.randn(b, s, d, generator=g).bfloat16().to(dev)
    ctx = torch.randn(b, sc, d, generator=g).bfloat16().to(dev)
    temb = torch.randn(b, d, generator=g).bfloat16().to(dev)
    rope = _rope_table(b, sc + s, dh, 314).bfloat16().to(dev)

    op = FO.FluxTransformerBlockOp("bf16", d, heads, dh, 6, FO.LyraQuantLevel.FP8_W8A8.value)
    op.initialize(None)
    with pytest.raises(RuntimeError):
        op.forward(x, ctx, rope, temb)  # nothing loaded yet
    op.reload_model_from_state_dict("transformer_blocks.3.", sd, "cpu")
    res = op.forward(x, ctx, rope, temb)
    assert isinstance(res, list) and res[0].shape == x.shape and res[1].shape == ctx.shape
    wd = F.load_flux_double_block_fp8(sd, "transformer_blocks.3.", d, torch.bfloat16, dev, full=False)  # level FP8_W8A8: 16-bit adaLN linear
    nq, nk, naq, nak = (sd[f"transformer_blocks.3.attn.{n}.weight"].to(dev) for n in ("norm_q", "norm_k", "norm_added_q", "norm_added_k"))
    w1, w2 = F.flux_double_block_fp8(x, ctx, temb, wd, lambda a, c: FO.flux_attention_core(a, nq, nk, rope, heads, c, naq, nak))
    assert torch.equal(res[0], w1) and torch.equal(res[1], w2) and torch.isfinite(w1.float()).all()
    # LoRA: merging a delta changes the output, clearing it restores the original bit for bit
    delta = (0.05 * torch.randn(3 * d, d, generator=g)).bfloat16()
    op.load_lora_by_name(["attn", "to_qkv"], delta, 0.8)
    assert not torch.equal(op.forward(x, ctx, rope, temb)[0], res[0])
    op.clear_lora()
    again = op.forward(x, ctx, rope, temb)
    assert torch.equal(again[0], res[0]) and torch.equal(again[1], res[1])
    with pytest.raises(KeyError):
        op.load_lora_by_name(["attn", "nope"], delta, 1.0)
    # argument checks of the reference's forward
    with pytest.raises(RuntimeError):
        op.forward(x.float(), ctx, rope, temb)
    with pytest.raises(RuntimeError):
        op.forward(x.cpu(), ctx, rope, temb)
    with pytest.raises(RuntimeError):
        op.forward(x.transpose(0, 1), ctx, rope, temb)
    # unsupported levels and dtypes fail at construction
    with pytest.raises(NotImplementedError):
        FO.FluxTransformerBlockOp("bf16", d, heads, dh, 6, FO.LyraQuantLevel.NONE.value)
    with pytest.raises(ValueError):
        FO.FluxSingleTransformerBlockOp("int8", d, heads, dh, 4, 1)
    with pytest.raises(KeyError):
        FO.FluxSingleTransformerBlockOp("bf16", d, heads, dh, 4, 2).reload_model_from_state_dict("missing.", sd, "cpu")

    sop = FO.FluxSingleTransformerBlockOp("bf16", d, heads, dh, 4, FO.LyraQuantLevel.FP8_W8A8_FULL.value)
    sop.initialize(None)
    sop.reload_model_from_state_dict("single_transformer_blocks.5.", sd, "cpu")
    xs = torch.cat([ctx, x], dim=1).contiguous()
    y = sop.forward(xs, rope, temb)
    ws = F.load_flux_single_block_fp8(sd, "single_transformer_blocks.5.", d, 4, torch.bfloat16, dev)
    snq, snk = (sd[f"single_transformer_blocks.5.attn.{n}.weight"].to(dev) for n in ("norm_q", "norm_k"))
    want = F.flux_single_block_fp8(xs, temb, ws, lambda a: FO.flux_attention_core(a, snq, snk, rope, heads))
    assert y.shape == xs.shape and torch.equal(y, want) and torch.isfinite(y.float()).all()


_BLOCK_LINEARS = lambda d: {"norm.linear": (3 * d, d), "attn.to_qkv": (3 * d, d), "proj_mlp": (4 * d, d), "proj_out": (d, 5 * d),
                            "norm1.linear": (6 * d, d), "norm1_context.linear": (6 * d, d), "attn.to_added_qkv": (3 * d, d),
                            "attn.to_out.0": (d, d), "attn.to_add_out": (d, d), "ff.net.0.proj": (4 * d, d), "ff.net.2": (d, 4 * d),
                            "ff_context.net.0.proj": (4 * d, d), "ff_context.net.2": (d, 4 * d)}


def _block_state(d, dh, seed, prefixes):
    """Weights large enough that every branch of the block matters as much as the residual stream (gates, scales and
    shifts of order one): a mis-wired block then differs by tens of per cent, not by a rounding error."""
    g = rng_t(seed)
    sd = {}
    for i, pre in enumerate(prefixes):
        sd.update(_state_dict(_BLOCK_LINEARS(d), seed + 1 + i, scale_w=0.06, prefix=pre))
        for n in _BLOCK_LINEARS(d):
            sd[f"{pre}{n}_input_scale"] = torch.tensor([6.0 / 448])
        for n in ("norm_q", "norm_k", "norm_added_q", "norm_added_k"):
            sd[f"{pre}attn.{n}.weight"] = (1 + 0.1 * torch.randn(dh, generator=g)).bfloat16()
    return sd


def _rel(a, b):
    return float((a.double() - b.double()).norm() / b.double().norm())


@pytest.mark.parametrize("level", ["FP8_W8A8_FULL", "FP8_W8A8"])
def test_flux_block_ops_against_an_independent_fp64_restatement(ops, dev, level):
    """FluxTransformerBlockOp.forward and FluxSingleTransformerBlockOp.forward against oracle/flux_blocks_f64.py, an fp64
    restatement of the reference's block code that shares nothing with lyradiff_amd/flux_fp8.py.  The outputs agree to
    within the noise of e4m3 codes that flip on 16-bit rounding differences; every deliberately mis-wired variant of the
    restatement (scale/shift swapped, wrong msa chunk, image tokens first, projections swapped, a dropped residual, the
    concatenation of the single block reversed) is many times further away."""
    from lyradiff_amd import flux_ops as FO
    from oracle import flux_blocks_f64 as FB

    b, s, sc, heads, dh = 2, 96, 32, 4, 64
    d = heads * dh
    full = level == "FP8_W8A8_FULL"
    g = rng_t(401)
    sd = _block_state(d, dh, 402, ("transformer_blocks.0.", "single_transformer_blocks.0."))
    x = torch.randn(b, s, d, generator=g).bfloat16()
    ctx = torch.randn(b, sc, d, generator=g).bfloat16()
    temb = torch.randn(b, d, generator=g).bfloat16()
    rope = _rope_table(b, sc + s, dh, 403).bfloat16()

    op = FO.FluxTransformerBlockOp("bf16", d, heads, dh, 4, FO.LyraQuantLevel[level].value)
    op.reload_model_from_state_dict("transformer_blocks.0.", sd, "cpu")
    out, cout = op.forward(x.to(dev), ctx.to(dev), rope.to(dev), temb.to(dev))
    want, cwant = FB.flux_double_block(sd, "transformer_blocks.0.", x, ctx, temb, rope, heads, "bf16", full)
    e1, e2 = _rel(out.cpu(), want), _rel(cout.cpu(), cwant)
    print(f"double block {level}: relative L2 distance to the fp64 restatement {e1:.4f} (image), {e2:.4f} (text)")
    assert e1 < 0.04 and e2 < 0.04
    for w in ("swap_scale_shift", "image_first", "swap_mlp_scale_shift", "swap_gates", "no_second_residual", "swap_out_projections"):
        bad, cbad = FB.flux_double_block(sd, "transformer_blocks.0.", x, ctx, temb, rope, heads, "bf16", full, wiring=(w,))
        assert _rel(out.cpu(), bad) > 4 * max(e1, 0.02) and _rel(cout.cpu(), cbad) > 4 * max(e2, 0.02), w

    sop = FO.FluxSingleTransformerBlockOp("bf16", d, heads, dh, 4, FO.LyraQuantLevel[level].value)
    sop.reload_model_from_state_dict("single_transformer_blocks.0.", sd, "cpu")
    xs = torch.cat([ctx, x], dim=1).contiguous()
    y = sop.forward(xs.to(dev), rope.to(dev), temb.to(dev))
    ywant = FB.flux_single_block(sd, "single_transformer_blocks.0.", xs, temb, rope, heads, "bf16", full)
    e3 = _rel(y.cpu(), ywant)
    print(f"single block {level}: relative L2 distance to the fp64 restatement {e3:.4f}")
    assert e3 < 0.04
    for w in ("swap_scale_shift", "mlp_first", "gate_is_chunk0"):
        assert _rel(y.cpu(), FB.flux_single_block(sd, "single_transformer_blocks.0.", xs, temb, rope, heads, "bf16", full, wiring=(w,))) > 4 * max(e3, 0.02), w


@pytest.mark.parametrize("file_dtype", ["fp32", "fp16"])
def test_flux_block_ops_reload_model_from_bin(ops, dev, tmp_path, file_dtype):
    """reload_model_from_bin(model_path, model_dtype) (th_op/flux_transformer_block/FluxTransformerBlockOp.h:239-258): the
    block's tensors as raw files model_path + name + ".bin", 16-bit members written in `model_dtype` and converted on
    the way in, scales as fp32.  With fp32 files (exact for bf16 values) the outputs equal those of the state-dict route bit for bit;
    with fp16 files the weights are rounded to fp16 and back, and the op equals a state-dict load of those rounded weights."""
    from lyradiff_amd import flux_ops as FO

    b, s, sc, heads, dh = 1, 64, 32, 4, 64
    d = heads * dh
    sd = _block_state(d, dh, 412, ("transformer_blocks.7.", "single_transformer_blocks.9."))
    ft = {"fp32": torch.float32, "fp16": torch.float16}[file_dtype]
    sd_files = {}
    for k, v in sd.items():
        if v.dtype == torch.bfloat16:
            v.to(ft).numpy().tofile(str(tmp_path / (k + ".bin")))
            sd_files[k] = v.to(ft).bfloat16()
        else:
            v.numpy().tofile(str(tmp_path / (k + ".bin")))
            sd_files[k] = v
    g = rng_t(413)
    x = torch.randn(b, s, d, generator=g).bfloat16().to(dev)
    ctx = torch.randn(b, sc, d, generator=g).bfloat16().to(dev)
    temb = torch.randn(b, d, generator=g).bfloat16().to(dev)
    rope = _rope_table(b, sc + s, dh, 414).bfloat16().to(dev)
    for level in (FO.LyraQuantLevel.FP8_W8A8_FULL, FO.LyraQuantLevel.FP8_W8A8):
        a = FO.FluxTransformerBlockOp("bf16", d, heads, dh, 4, level.value)
        a.reload_model_from_state_dict("transformer_blocks.7.", sd_files, "cpu")
        f = FO.FluxTransformerBlockOp("bf16", d, heads, dh, 4, level.value)
        f.reload_model_from_bin(str(tmp_path) + "/transformer_blocks.7.", file_dtype)
        ra, rf = a.forward(x, ctx, rope, temb), f.forward(x, ctx, rope, temb)
        assert torch.equal(ra[0], rf[0]) and torch.equal(ra[1], rf[1])
    sa = FO.FluxSingleTransformerBlockOp("bf16", d, heads, dh, 4, FO.LyraQuantLevel.FP8_W8A8_FULL.value)
    sa.reload_model_from_state_dict("single_transformer_blocks.9.", sd_files, "cpu")
    sf = FO.FluxSingleTransformerBlockOp("bf16", d, heads, dh, 4, FO.LyraQuantLevel.FP8_W8A8_FULL.value)
    sf.reload_model_from_bin(str(tmp_path) + "/single_transformer_blocks.9.", file_dtype)
    xs = torch.cat([ctx, x], dim=1).contiguous()
    assert torch.equal(sa.forward(xs, rope, temb), sf.forward(xs, rope, temb))
    with pytest.raises(ValueError):
        sf.reload_model_from_bin(str(tmp_path) + "/single_transformer_blocks.9.", "int8")  # the reference: "wrong model_dtype"
    with pytest.raises((FileNotFoundError, ValueError, OSError)):
        sf.reload_model_from_bin(str(tmp_path) + "/absent.", "fp32")


def _int4_block_state(d, dh, g, scale_w=0.03, lora_scale=0.05):
    """State dict of one double ("transformer_blocks.0.") and one single ("single_transformer_blocks.0.") INT4 block in the
    reference's container layout; the adaLN linears carry FP8 input scales, which the non-FULL level ignores."""
    _state_dict_ = lambda names, seed, prefix: _state_dict(names, seed, scale_w=scale_w, prefix=prefix)
    _int4_state_ = lambda prefix, n, k, g, bias=True: _int4_state(prefix, n, k, g, bias=bias, lora_scale=lora_scale)
    sd = {}
    for pre, ada in (("transformer_blocks.0.", ("norm1.linear", "norm1_context.linear")), ("single_transformer_blocks.0.", ("norm.linear",))):
        chunks = 6 if len(ada) == 2 else 3
        sd.update(_state_dict_({a: (chunks * d, d) for a in ada}, 402, prefix=pre))
        for a in ada:
            sd[f"{pre}{a}_input_scale"] = torch.tensor([4.0 / 448])
        for n in ("norm_q", "norm_k", "norm_added_q", "norm_added_k"):
            sd[f"{pre}attn.{n}.weight"] = (1 + 0.1 * torch.randn(dh, generator=g)).bfloat16()
    for name, n in (("attn.to_qkv.", 3 * d), ("attn.to_added_qkv.", 3 * d), ("attn.to_out.0.", d), ("attn.to_add_out.", d)):
        sd.update(_int4_state_("transformer_blocks.0." + name, n, d, g))
    for ff in ("ff.", "ff_context."):
        sd.update(_int4_state_(f"transformer_blocks.0.{ff}net.0.proj.", 4 * d, d, g))
        sd.update(_state_dict_({f"{ff}net.2": (d, 4 * d)}, 403, prefix="transformer_blocks.0."))
        sd[f"transformer_blocks.0.{ff}net.2_input_scale"] = torch.tensor([3.0 / 448])
    sd.update(_int4_state_("single_transformer_blocks.0.attn.to_qkv.", 3 * d, d, g))
    sd.update(_int4_state_("single_transformer_blocks.0.proj_mlp.", 4 * d, d, g))
    sd.update(_int4_state_("single_transformer_blocks.0.proj_out.linears.0.", d, d, g))
    sd.update(_int4_state_("single_transformer_blocks.0.proj_out.linears.1.linear.", d, 4 * d, g, bias=False))
    return sd


@pytest.mark.parametrize("full", [True, False])
def test_flux_int4_block_ops(ops, dev, full):
    """Quant levels INT4_W4A4 (16-bit adaLN linear) and INT4_W4A4_FULL (FP8 adaLN linear) of the block classes: the op output
    equals the block function driven with the same attention core, and the block function equals its steps one by one."""
    from lyradiff_amd import flux_fp8 as F8
    from lyradiff_amd import flux_int4 as F
    from lyradiff_amd import flux_ops as FO

    b, s, sc, heads, dh = 1, 128, 64, 4, 64
    d = heads * dh
    g = rng_t(401)
    level = FO.LyraQuantLevel.INT4_W4A4_FULL if full else FO.LyraQuantLevel.INT4_W4A4
    sd = _int4_block_state(d, dh, g)
    x = torch.randn(b, s, d, generator=g).bfloat16().to(dev)
    ctx = torch.randn(b, sc, d, generator=g).bfloat16().to(dev)
    temb = torch.randn(b, d, generator=g).bfloat16().to(dev)
    rope = _rope_table(b, sc + s, dh, 404).bfloat16().to(dev)

    op = FO.FluxTransformerBlockOp("bf16", d, heads, dh, 6, level.value)
    op.initialize(None)
    op.reload_model_from_state_dict("transformer_blocks.0.", sd, "cpu")
    res = op.forward(x, ctx, rope, temb)
    w = F.load_flux_double_block_int4(sd, "transformer_blocks.0.", d, full, torch.bfloat16, dev)
    assert isinstance(w.norm1, F8.FP8Linear) == full
    nq, nk, naq, nak = (sd[f"transformer_blocks.0.attn.{n}.weight"].to(dev) for n in ("norm_q", "norm_k", "norm_added_q", "norm_added_k"))
    core = lambda a, c: FO.flux_attention_core(a, nq, nk, rope, heads, c, naq, nak)
    o1, o2 = F.flux_double_block_int4(x, ctx, temb, w, core)
    assert torch.equal(res[0], o1) and torch.equal(res[1], o2) and torch.isfinite(o1.float()).all() and torch.isfinite(o2.float()).all()
    # the same steps one by one
    n1, m1 = F.ada_layernorm_int4(x, temb, w.norm1, 6)
    n2, m2 = F.ada_layernorm_int4(ctx, temb, w.norm1_context, 6)
    if not full:  # the 16-bit adaLN linear is a plain matmul: msa = temb . W^T + b, chunk c of batch j at [c, j]
        want = torch.nn.functional.linear(temb, w.norm1.weight, w.norm1.bias).view(b, 6, d).transpose(0, 1)
        assert torch.equal(m1, want)
    a1, a2 = core(w.to_qkv.forward(n1), w.to_added_qkv.forward(n2))
    w1 = F.flux_attn_post_int4(x, w.to_out.forward(a1.contiguous()), m1, w.ff)
    w2 = F.flux_attn_post_int4(ctx, w.to_add_out.forward(a2.contiguous()), m2, w.ff_context)
    assert torch.equal(o1, w1) and torch.equal(o2, w2)
    with pytest.raises(KeyError):
        op.load_lora_by_name(["attn", "to_qkv"], torch.zeros(3 * d, d).bfloat16(), 1.0)
    op.clear_lora()

    sop = FO.FluxSingleTransformerBlockOp("bf16", d, heads, dh, 4, level.value)
    sop.reload_model_from_state_dict("single_transformer_blocks.0.", sd, "cpu")
    xs = torch.cat([ctx, x], dim=1).contiguous()
    y = sop.forward(xs, rope, temb)
    ws = F.load_flux_single_block_int4(sd, "single_transformer_blocks.0.", d, 4, full, torch.bfloat16, dev)
    snq, snk = (sd[f"single_transformer_blocks.0.attn.{n}.weight"].to(dev) for n in ("norm_q", "norm_k"))
    score = lambda a: FO.flux_attention_core(a, snq, snk, rope, heads)
    assert torch.equal(y, F.flux_single_block_int4(xs, temb, ws, score)) and torch.isfinite(y.float()).all()
    ns, ms = F.ada_layernorm_int4(xs, temb, ws.norm, 3)
    want = F.flux_single_mlp_int4(xs, ns, score(ws.to_qkv.forward(ns)).contiguous(), ms[2].contiguous(), ws.mlp)
    assert torch.equal(y, want)


_INT4_DOUBLE_MUTATIONS = ("swap_scale_shift", "swap_mlp_scale_shift", "swap_gates", "no_second_residual", "swap_qkv_projections",
                          "swap_out_projections", "swap_feed_forwards", "no_low_rank", "low_rank_from_smoothed", "no_gelu")
_INT4_SINGLE_MUTATIONS = ("swap_scale_shift", "gate_is_chunk0", "mlp_from_block_input", "linears0_from_norm", "drop_linears1",
                          "no_low_rank", "low_rank_from_smoothed")


def check_int4_blocks_against_the_restatement(make_double, make_single, dev, full):
    """Shared by the Python op classes (here) and the C++ torch classes (tests/test_gpu_torch_classes.py).

    A 4-bit group quantiser turns a one-ULP difference in its 16-bit input (the attention output of a bf16 softmax against
    an fp64 one) into code flips worth a seventh of the group maximum, so a correct block sits further from the fp64
    restatement than the FP8 blocks do: measured 0.05-0.08 relative L2 when the W4A4 main product and its low-rank branch
    contribute alike (low-rank weights of std 0.1), 0.016-0.019 when the low-rank branch -- 16-bit arithmetic, no flips --
    dominates (std 0.2).  Both settings run; the nearest mis-wired variant measured 0.34 and 0.28 away."""
    from oracle import flux_blocks_f64 as FB

    b, s, sc, heads, dh = 2, 96, 32, 4, 64
    d = heads * dh
    for lora_scale, e_max, far in ((0.1, 0.10, 0.30), (0.2, 0.03, 0.25)):
        g = rng_t(441)
        sd = _int4_block_state(d, dh, g, scale_w=0.06, lora_scale=lora_scale)
        x = torch.randn(b, s, d, generator=g).bfloat16()
        ctx = torch.randn(b, sc, d, generator=g).bfloat16()
        temb = torch.randn(b, d, generator=g).bfloat16()
        rope = _rope_table(b, sc + s, dh, 443).bfloat16()
        op = make_double(d, heads, dh)
        op.reload_model_from_state_dict("transformer_blocks.0.", sd, "cpu")
        out, cout = op.forward(x.to(dev), ctx.to(dev), rope.to(dev), temb.to(dev))
        want, cwant = FB.flux_double_block_int4(sd, "transformer_blocks.0.", x, ctx, temb, rope, heads, "bf16", full)
        e1, e2 = _rel(out.cpu(), want), _rel(cout.cpu(), cwant)
        print(f"INT4 double block (full={full}, low-rank std {lora_scale}): relative L2 distance to the fp64 restatement "
              f"{e1:.4f} (image), {e2:.4f} (text)")
        assert e1 < e_max and e2 < e_max
        for w in _INT4_DOUBLE_MUTATIONS:
            bad, cbad = FB.flux_double_block_int4(sd, "transformer_blocks.0.", x, ctx, temb, rope, heads, "bf16", full, wiring=(w,))
            r1, r2 = _rel(out.cpu(), bad), _rel(cout.cpu(), cbad)
            assert r1 > far and r2 > far and min(r1, r2) > 3 * max(e1, e2), (w, r1, r2)
        sop = make_single(d, heads, dh)
        sop.reload_model_from_state_dict("single_transformer_blocks.0.", sd, "cpu")
        xs = torch.cat([ctx, x], dim=1).contiguous()
        y = sop.forward(xs.to(dev), rope.to(dev), temb.to(dev))
        ywant = FB.flux_single_block_int4(sd, "single_transformer_blocks.0.", xs, temb, rope, heads, "bf16", full)
        e3 = _rel(y.cpu(), ywant)
        print(f"INT4 single block (full={full}, low-rank std {lora_scale}): relative L2 distance to the fp64 restatement {e3:.4f}")
        assert e3 < e_max
        for w in _INT4_SINGLE_MUTATIONS:
            r3 = _rel(y.cpu(), FB.flux_single_block_int4(sd, "single_transformer_blocks.0.", xs, temb, rope, heads, "bf16", full, wiring=(w,)))
            assert r3 > far and r3 > 3 * e3, (w, r3)


@pytest.mark.parametrize("level", ["INT4_W4A4_FULL", "INT4_W4A4"])
def test_flux_int4_block_ops_against_an_independent_fp64_restatement(ops, dev, level):
    """Both INT4 levels of FluxTransformerBlockOp and FluxSingleTransformerBlockOp against the fp64 restatement of
    FluxTransformerInt4Block / FluxAttentionInt4Processor / FluxAttnPostInt4Processor / FluxSingleTransformerInt4Block
    (oracle/flux_blocks_f64.py), which shares nothing with lyradiff_amd/flux_int4.py.  The outputs agree to within the noise of
    4-bit codes that flip on 16-bit rounding differences; every mis-wired variant of the restatement (a wrong msa chunk, gates
    or projections or feed-forwards swapped, a dropped residual or projection, the low-rank branch missing or fed from the
    smoothed input, proj_mlp or proj_out.linears.0 fed from the wrong tensor) is many times further away."""
    from lyradiff_amd import flux_ops as FO

    lv = FO.LyraQuantLevel[level].value
    check_int4_blocks_against_the_restatement(lambda d, h, dh: FO.FluxTransformerBlockOp("bf16", d, h, dh, 4, lv),
                                              lambda d, h, dh: FO.FluxSingleTransformerBlockOp("bf16", d, h, dh, 4, lv),
                                              dev, level == "INT4_W4A4_FULL")


@pytest.mark.parametrize("dt", ["bf16", "f16"])
@pytest.mark.parametrize("b,s,sc,heads,dh", [(2, 70, 21, 3, 128), (1, 33, 0, 2, 64), (2, 5, 9, 24, 128)])
def test_rmsnorm_rope_against_the_oracle(ops, dev, dt, b, s, sc, heads, dh):
    """lq_rmsnorm_rope (invokeFusedRmsNormCatAndRope / invokeFusedRmsNormAndRope): v and the layout bit for bit; q and k within one
    ULP of T per rounding step of the oracle (the mean of squares is summed in the kernel's own fp32 order), at most 2 % of the
    elements differing at all; rope given per batch and shared by the batch."""
    t = TORCH_DT[dt]
    g = rng_t(b * 1000 + s + dh)
    d3 = 3 * heads * dh
    qkv = (torch.randn(b, s, d3, generator=g) * 1.7).to(t)
    cqkv = (torch.randn(b, sc, d3, generator=g) * 0.8).to(t) if sc else None
    nqk = (1 + 0.2 * torch.randn(2 * dh, generator=g)).to(t)
    naqk = (1 + 0.2 * torch.randn(2 * dh, generator=g)).to(t) if sc else None
    for rope_b in (b, 1):
        rope = _rope_table(rope_b, sc + s, dh, 77 + rope_b).to(t)
        out = ops.rmsnorm_rope(qkv.to(dev), nqk.to(dev), rope.to(dev), heads, None if cqkv is None else cqkv.to(dev),
                               None if naqk is None else naqk.to(dev))
        want = O.rmsnorm_rope(to_np_f32(qkv), None if cqkv is None else to_np_f32(cqkv), to_np_f32(nqk),
                              None if naqk is None else to_np_f32(naqk), to_np_f32(rope), heads, dt)
        got = to_np_f32(out)
        assert got.shape == want.shape == (b, sc + s, 3, heads, dh)
        assert np.array_equal(got[:, :, 2], want[:, :, 2])
        ulp = 2.0 ** (-8 if dt == "bf16" else -11)
        diff = np.abs(got[:, :, :2] - want[:, :, :2])
        mag = np.abs(want[:, :, :2]).reshape(b, sc + s, 2, heads, dh // 2, 2).sum(-1, keepdims=True).repeat(2, -1).reshape(diff.shape)
        assert np.all(diff <= 3 * ulp * mag + 1e-6), f"max excess {(diff - 3 * ulp * mag).max()}"
        assert (diff != 0).mean() < 0.02
    with pytest.raises(Exception):
        ops.rmsnorm_rope(qkv.to(dev)[..., :-8].contiguous(), nqk.to(dev), rope.to(dev), heads)
