"""Loaders for the reference's weight formats (raw .bin files / state-dict caches) and the linear modules built from
them: file handling on the CPU, end-to-end parity with the oracle on the GPU."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from oracle import oracle_c as OC
from tests.helpers import assert_close_tol, check_fp8_gemm, rng_t, to_np_f32


def write_bin(path, t):
    a = t.view(torch.int16).numpy() if t.dtype == torch.bfloat16 else t.numpy()
    a.tofile(path)


def test_read_bin_and_missing_tensors(tmp_path):
    from lyradiff_amd import weights as W

    x = torch.randn(6, 8).bfloat16()
    write_bin(tmp_path / "a.weight.bin", x)
    assert torch.equal(W.read_bin(str(tmp_path / "a.weight.bin"), (6, 8), torch.bfloat16), x)
    f = torch.rand(5)
    write_bin(tmp_path / "s.bin", f)
    assert torch.equal(W.read_bin(str(tmp_path / "s.bin"), (5,), torch.float32), f)
    with pytest.raises(ValueError, match="expected 7"):
        W.read_bin(str(tmp_path / "s.bin"), (7,), torch.float32)
    with pytest.raises(KeyError, match="blk.net.2.weight"):
        W._source({})("blk.net.2.weight", (2, 2), torch.bfloat16)
    with pytest.raises(ValueError):
        W._source({"w": torch.zeros(2, 2)})("w", (2, 2), torch.int8)


@pytest.mark.gpu
def test_int8_linear_from_bin_files(dev, tmp_path):
    from lyradiff_amd import weights as W

    m, n, k = 300, 640, 320
    g = rng_t(31)
    w = torch.randint(-127, 128, (n, k), generator=g, dtype=torch.int8)
    ws = (torch.rand(n, generator=g) * 9e-3 + 1e-3).float()
    s_in = torch.tensor([0.04], dtype=torch.float32)
    pre = (0.5 + torch.rand(k, generator=g)).float()
    bias = (torch.randn(n, generator=g) * 0.02).half()
    for name, t in ((".weight_int8", w), (".weight_quant_scale", ws), (".input_quant_scale", s_in), (".pre_quant_scale", pre), (".bias", bias)):
        write_bin(tmp_path / ("unet.attn1.to_out.0" + name + ".bin"), t)
    lin = W.load_int8_linear(str(tmp_path), "unet.", "attn1.to_out.0", n, k, dev, torch.float16)
    x = torch.randn(2, m // 2, k, generator=g).half()
    y = lin.forward(x.to(dev))
    q = O.sq_input_quant(to_np_f32(x).reshape(m, k), pre.numpy(), s_in.numpy(), False)
    ref = O.int8_epilogue(O.gemm_i8_acc(q, w.numpy()), ws.numpy(), s_in.numpy(), to_np_f32(bias), "f16")
    assert y.shape == (2, m // 2, n) and np.array_equal(to_np_f32(y).reshape(m, n), ref)
    yd = lin.forward(x.to(dev), dynamic=True)
    qd, sd = O.sq_dynamic_quant(to_np_f32(x).reshape(m, k), pre.numpy())
    assert np.array_equal(to_np_f32(yd).reshape(m, n), O.int8_epilogue(O.gemm_i8_acc(qd, w.numpy()), ws.numpy(), sd, to_np_f32(bias), "f16"))


@pytest.mark.gpu
def test_fp8_linear_from_state_dict(dev):
    from lyradiff_amd import weights as W

    m, n, k = 200, 512, 384
    g = rng_t(32)
    sd = {"blk.net.0.proj.weight": (torch.randn(n, k, generator=g) * 0.02).bfloat16(),
          "blk.net.0.proj.bias": (torch.randn(n, generator=g) * 0.1).bfloat16(),
          "blk.net.0.proj_input_scale": torch.tensor([0.012], dtype=torch.float32)}
    lin = W.load_fp8_linear(sd, "blk.", "net.0.proj", n, k, torch.bfloat16, dev)
    qw, sw = O.fp8_amax_cast(to_np_f32(sd["blk.net.0.proj.weight"]))
    assert lin.weight_scale.item() == float(sw)
    from lyradiff_amd import ops
    assert np.array_equal(ops.unpack_weight(lin.weight_rows32).cpu().numpy(), qw)
    x = torch.randn(m, k, generator=g).bfloat16()
    y = lin.forward(x.to(dev), gelu=True)
    qa = O.fp8_scale_cast(to_np_f32(x), np.float32(0.012), True)
    ref = O.fp8_gemm(qa, qw, 0.012, sw, to_np_f32(sd["blk.net.0.proj.bias"]), True, None, 0.0, "bf16")
    check_fp8_gemm(to_np_f32(y), ref, qa, qw, 0.012, sw, "bf16", "fp8 linear from state dict", extra_abs=2e-6)


@pytest.mark.gpu
def test_w4a4_linear_from_bin_files(dev, tmp_path):
    from lyradiff_amd import weights as W

    m, n, k, r = 130, 256, 512, 32
    g = rng_t(33)
    wt = (torch.randn(n, k, generator=g) * 0.05).bfloat16()
    qb, sB = O.w4a4_quant(to_np_f32(wt), None, 64, "f32")
    smooth = (0.5 + torch.rand(k, generator=g)).float()
    up = (torch.randn(n, r, generator=g) * 0.3).bfloat16()
    down = (torch.randn(r, k, generator=g) * 0.05).bfloat16()
    bias = (torch.randn(n, generator=g) * 0.1).bfloat16()
    write_bin(tmp_path / "l.packed_weight.bin", torch.from_numpy(qb.view(np.int8).reshape(n, k // 2)))
    write_bin(tmp_path / "l.weight_scale.bin", torch.from_numpy(sB))
    for name, t in (("smooth", smooth), ("lora_up", up), ("lora_down", down), ("bias", bias)):
        write_bin(tmp_path / f"l.{name}.bin", t)
    lin = W.load_w4a4_linear(str(tmp_path), "l.", n, k, r, True, torch.bfloat16, dev)
    x = torch.randn(m, k, generator=g).bfloat16()
    y = lin.forward(x.to(dev))
    qa, sA = O.w4a4_quant(to_np_f32(x), smooth.numpy(), 64, "f32")
    y32 = OC.w4a4_gemm(qa, qb, sA, sB, None)
    act = O.round_to(O.lora_down_f64(to_np_f32(x), to_np_f32(down)).astype(np.float32), "bf16")
    ref = O.w4a4_gemm_lora_f64(y32, act, to_np_f32(up), to_np_f32(bias), "bf16")
    mag = np.abs(y32).astype(np.float64) + np.abs(act).astype(np.float64) @ np.abs(to_np_f32(up)).astype(np.float64).T
    # the low-rank activation is rounded to bf16 from an fp32 sum whose order is free: one bf16 ULP of it is allowed
    assert_close_tol(to_np_f32(y), ref, "w4a4 linear from .bin files", abs_floor=2.0 ** -8 * mag)


def test_int4_pack_helpers_match_the_oracle_packing():
    from lyradiff_amd import weights as W

    q = torch.randint(-8, 8, (6, 32), generator=rng_t(1), dtype=torch.int8)
    packed = W.pack_int8_tensor_to_packed_int4(q)
    assert packed.shape == (6, 16) and packed.dtype == torch.int8
    assert np.array_equal(packed.numpy().view(np.uint32), O.pack_int4(q.numpy()))  # same low-nibble-first convention
    assert torch.equal(W.unpack_int4_packed_tensor_to_int8(packed), q)
    assert W.pack_int8_tensor_to_packed_int4(torch.tensor([[-8, 7]], dtype=torch.int8)).view(torch.uint8).item() == 0x78
    with pytest.raises(ValueError, match="int4 range"):
        W.pack_int8_tensor_to_packed_int4(torch.tensor([[8, 0]], dtype=torch.int8))


def test_flux_block_op_constructor_checks():
    """The constructors of the block classes validate their arguments without touching a GPU."""
    from lyradiff_amd import flux_ops as FO

    assert [l.value for l in FO.LyraQuantLevel] == list(range(9))
    op = FO.FluxSingleTransformerBlockOp("fp16", 256, 4, 64, 4, 2)
    assert op.dtype == torch.float16 and op.quant_level is FO.LyraQuantLevel.FP8_W8A8_FULL and not op.int4
    assert FO.FluxTransformerBlockOp("bf16", 256, 4, 64, 6, 8).int4
    with pytest.raises(RuntimeError, match="reload_model_from_state_dict"):
        op.clear_lora()
    with pytest.raises(ValueError):
        FO.FluxTransformerBlockOp("bf16", 256, 4, 60, 6, 1)  # dim != heads * head_dim
    with pytest.raises(NotImplementedError):
        FO.FluxTransformerBlockOp("bf16", 256, 4, 64, 6, FO.LyraQuantLevel.INT8_SMOOTH_QUANT_LEVEL1.value)


@pytest.mark.gpu
def test_smooth_vector_on_device(dev):
    from lyradiff_amd import ops

    g = rng_t(44)
    x = torch.randn(1000, 1280, generator=g).half()
    x[:, torch.randperm(1280, generator=g)[:8]] *= 20.0
    w = torch.randint(-127, 128, (640, 1280), generator=g, dtype=torch.int8).float()
    ax = ops.col_absmax(x[:600].contiguous().to(dev))
    ax = ops.col_absmax(x[600:].contiguous().to(dev), ax)  # accumulated over two calibration batches
    aw = ops.col_absmax(w.to(dev))
    assert np.array_equal(ax.cpu().numpy(), np.abs(to_np_f32(x)).max(axis=0))
    assert np.array_equal(aw.cpu().numpy(), np.abs(w.numpy()).max(axis=0))
    for alpha in (0.8, 0.25, 1.0, 0.0, 0.5):  # 0.8 is the reference's default (convert_sd_quant_model.py:340)
        pre, s = ops.smooth_vector(ax, aw, alpha)
        s_ref = O.smooth_vector(to_np_f32(x), w.numpy(), alpha)
        assert np.allclose(s.cpu().numpy(), s_ref, rtol=2e-6) and np.allclose(pre.cpu().numpy(), 1.0 / s_ref, rtol=3e-6)
    # hand-computed values at an asymmetric exponent: 16^0.75 / 256^0.25 = 8 / 4 (a swapped exponent gives 2 / 64)
    p2, s2 = ops.smooth_vector(torch.full((8,), 16.0, device=dev), torch.full((8,), 256.0, device=dev), 0.75)
    assert np.allclose(s2.cpu().numpy(), 2.0, rtol=2e-6) and np.allclose(p2.cpu().numpy(), 0.5, rtol=2e-6)
    # the vector does its job: the smoothed activation has a flatter column profile
    t = to_np_f32(x) * pre.cpu().numpy()[None, :]
    assert np.abs(t).max(axis=0).max() / np.median(np.abs(t).max(axis=0)) < 0.3 * np.abs(to_np_f32(x)).max(axis=0).max() / np.median(np.abs(to_np_f32(x)).max(axis=0))
