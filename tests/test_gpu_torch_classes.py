"""torch.classes.lyradiff.* (lyradiff_amd/th_op/th_lyradiff.cpp): the FLUX block classes registered the way the reference's
Python reaches them (src/lyradiff/th_op/pybind.cc:66-96, lyradiff/__init__.py:4-5).  On the CPU: the library loads, the
classes have the reference's constructor arguments and methods, construction errors.  On the GPU: the C++ classes run
the same kernels in the same order as the Python classes of lyradiff_amd/flux_ops.py, so their outputs are equal bit for
bit, and they are checked directly against the independent fp64 restatement of the blocks as well."""
import os

import pytest
import torch

from tests.helpers import rng_t
from tests.test_gpu_flux_blocks import _block_state, _int4_block_state, _rel, _rope_table, check_int4_blocks_against_the_restatement


@pytest.fixture(scope="module")
def ops(dev):
    from lyradiff_amd import ops as _ops

    return _ops


@pytest.fixture(scope="module")
def classes():
    from lyradiff_amd import lib

    lib.load_torch_classes()
    return torch.classes.lyradiff


def test_library_path_follows_the_reference_variable(monkeypatch, tmp_path):
    from lyradiff_amd import lib

    monkeypatch.delenv("LYRA_LIB_PATH", raising=False)
    monkeypatch.delenv("LYRA_LIB_PATH_AMD", raising=False)
    abi, th = lib._paths()
    assert abi.endswith("lyradiff_amd/liblyraquant.so") and th.endswith("lyradiff_amd/libth_lyradiff.so")
    monkeypatch.setenv("LYRA_LIB_PATH", str(tmp_path / "libth_lyradiff.so"))  # what the reference's wrapper is given
    assert lib._paths() == (str(tmp_path / "liblyraquant.so"), str(tmp_path / "libth_lyradiff.so"))
    monkeypatch.setenv("LYRA_LIB_PATH", str(tmp_path / "liblyraquant.so"))
    assert lib._paths() == (str(tmp_path / "liblyraquant.so"), str(tmp_path / "libth_lyradiff.so"))
    monkeypatch.setenv("LYRA_LIB_PATH_AMD", "/x/liblyraquant.so")
    assert lib._paths()[0] == "/x/liblyraquant.so"


def test_classes_are_registered_with_the_reference_interface(classes):
    assert os.path.exists(os.path.join(os.path.dirname(__file__), "..", "lyradiff_amd", "libth_lyradiff.so"))
    ctx = classes.LyraDiffCommonContext()
    for name, nargs in (("FluxTransformerBlockOp", 4), ("FluxSingleTransformerBlockOp", 3)):
        cls = getattr(classes, name)
        op = cls("bf16", 256, 4, 64, 6, 2)
        op.initialize(ctx)
        for method in ("forward", "load_lora_by_name", "clear_lora", "reload_model_from_bin", "reload_model_from_state_dict", "initialize"):
            assert hasattr(op, method), (name, method)
        # keyword arguments and defaults of pybind.cc:66-96 (quant_level defaults to 0, which holds no quantized linear)
        with pytest.raises(RuntimeError, match="quant level 0"):
            cls()
        cls(inference_dtype="fp16", embedding_dim=128, embedding_head_num=2, embedding_head_dim=64, mlp_scale=4, quant_level=7)
        with pytest.raises(RuntimeError, match="wrong inference_dtype"):
            cls("int8", 256, 4, 64, 6, 2)
        with pytest.raises(RuntimeError, match="quant level 4"):
            cls("bf16", 256, 4, 64, 6, 4)
        with pytest.raises(RuntimeError, match="embedding_dim must equal"):
            cls("bf16", 256, 4, 60, 6, 2)
        with pytest.raises(RuntimeError, match="has not been called"):
            op.clear_lora()
        with pytest.raises(RuntimeError, match="Cannot find a tensor of name blk.norm"):
            op.reload_model_from_state_dict("blk.", {}, "cpu")
        with pytest.raises(RuntimeError, match="wrong model_dtype"):
            op.reload_model_from_bin("/nonexistent/", "int8")


def _fp8_inputs(dev, b, s, sc, heads, dh, seed):
    d = heads * dh
    g = rng_t(seed)
    return (torch.randn(b, s, d, generator=g).bfloat16().to(dev), torch.randn(b, sc, d, generator=g).bfloat16().to(dev),
            torch.randn(b, d, generator=g).bfloat16().to(dev), _rope_table(b, sc + s, dh, seed + 1).bfloat16().to(dev))


@pytest.mark.gpu
@pytest.mark.parametrize("level", [2, 1])
def test_fp8_block_classes_equal_the_python_ops_and_match_the_fp64_restatement(classes, ops, dev, level):
    from lyradiff_amd import flux_ops as FO
    from oracle import flux_blocks_f64 as FB

    b, s, sc, heads, dh = 2, 96, 32, 4, 64
    d = heads * dh
    sd = _block_state(d, dh, 402, ("transformer_blocks.0.", "single_transformer_blocks.0."))
    x, ctx, temb, rope = _fp8_inputs(dev, b, s, sc, heads, dh, 501)

    op = classes.FluxTransformerBlockOp("bf16", d, heads, dh, 4, level)
    op.initialize(classes.LyraDiffCommonContext())
    op.reload_model_from_state_dict("transformer_blocks.0.", sd, "cpu")
    out, cout = op.forward(x, ctx, rope, temb)
    py = FO.FluxTransformerBlockOp("bf16", d, heads, dh, 4, level)
    py.reload_model_from_state_dict("transformer_blocks.0.", sd, "cpu")
    pout, pcout = py.forward(x, ctx, rope, temb)
    assert torch.equal(out, pout) and torch.equal(cout, pcout)
    want, cwant = FB.flux_double_block(sd, "transformer_blocks.0.", x.cpu(), ctx.cpu(), temb.cpu(), rope.cpu(), heads, "bf16", level == 2)
    e1, e2 = _rel(out.cpu(), want), _rel(cout.cpu(), cwant)
    print(f"torch.classes double block level {level}: relative L2 distance to the fp64 restatement {e1:.4f} / {e2:.4f}")
    assert e1 < 0.04 and e2 < 0.04

    sop = classes.FluxSingleTransformerBlockOp("bf16", d, heads, dh, 4, level)
    sop.reload_model_from_state_dict("single_transformer_blocks.0.", sd, "cpu")
    xs = torch.cat([ctx, x], dim=1).contiguous()
    y = sop.forward(xs, rope, temb)
    spy = FO.FluxSingleTransformerBlockOp("bf16", d, heads, dh, 4, level)
    spy.reload_model_from_state_dict("single_transformer_blocks.0.", sd, "cpu")
    assert torch.equal(y, spy.forward(xs, rope, temb))
    e3 = _rel(y.cpu(), FB.flux_single_block(sd, "single_transformer_blocks.0.", xs.cpu(), temb.cpu(), rope.cpu(), heads, "bf16", level == 2))
    print(f"torch.classes single block level {level}: {e3:.4f}")
    assert e3 < 0.04

    # LoRA: merge into one linear, the outputs move and equal the Python class's; clear_lora restores the first outputs
    delta = (torch.randn(3 * d, d, generator=rng_t(7)) * 0.05).bfloat16()
    op.load_lora_by_name(["attn", "to_qkv"], delta.to(dev), 0.8)
    py.load_lora_by_name(["attn", "to_qkv"], delta.to(dev), 0.8)
    lo, lco = op.forward(x, ctx, rope, temb)
    plo, plco = py.forward(x, ctx, rope, temb)
    assert torch.equal(lo, plo) and torch.equal(lco, plco) and not torch.equal(lo, out)
    op.clear_lora()
    ro, rco = op.forward(x, ctx, rope, temb)
    assert torch.equal(ro, out) and torch.equal(rco, cout)
    with pytest.raises(RuntimeError, match="no FP8 linear named attn.to_k"):
        op.load_lora_by_name(["attn", "to_k"], delta.to(dev), 1.0)
    if level == 1:  # the 16-bit adaLN linear is no LoRA target of the FP8 weight map
        with pytest.raises(RuntimeError, match="no FP8 linear named norm1.linear"):
            op.load_lora_by_name(["norm1", "linear"], torch.zeros(6 * d, d).bfloat16().to(dev), 1.0)

    # input checks of th_utils.h:14-33
    with pytest.raises(RuntimeError, match="hidden_states must be contiguous"):
        op.forward(x.transpose(0, 1).contiguous().transpose(0, 1), ctx, rope, temb)
    with pytest.raises(RuntimeError, match="temb_emb dtype should be"):
        op.forward(x, ctx, rope, temb.half())
    with pytest.raises(RuntimeError, match="rope_emb must be a CUDA tensor"):
        sop.forward(xs, rope.cpu(), temb)


@pytest.mark.gpu
@pytest.mark.parametrize("file_dtype", ["fp32", "bf16"])
def test_fp8_block_classes_reload_model_from_bin(classes, ops, dev, tmp_path, file_dtype):
    """reload_model_from_bin(model_path, model_dtype) (FluxTransformerBlockOp.h:239-258): raw files model_path + name + ".bin";
    the bf16 test weights survive an fp32 or a bf16 file exactly, so both routes must give the same bits."""
    b, s, sc, heads, dh = 1, 64, 32, 4, 64
    d = heads * dh
    sd = _block_state(d, dh, 412, ("transformer_blocks.7.", "single_transformer_blocks.9."))
    for k, v in sd.items():
        if v.dtype == torch.bfloat16:
            (v.float().numpy() if file_dtype == "fp32" else v.view(torch.int16).numpy()).tofile(str(tmp_path / (k + ".bin")))
        else:
            v.numpy().tofile(str(tmp_path / (k + ".bin")))
    x, ctx, temb, rope = _fp8_inputs(dev, b, s, sc, heads, dh, 511)
    for level in (2, 1):
        a = classes.FluxTransformerBlockOp("bf16", d, heads, dh, 4, level)
        a.reload_model_from_state_dict("transformer_blocks.7.", sd, "cpu")
        f = classes.FluxTransformerBlockOp("bf16", d, heads, dh, 4, level)
        f.reload_model_from_bin(str(tmp_path) + "/transformer_blocks.7.", file_dtype)
        ra, rf = a.forward(x, ctx, rope, temb), f.forward(x, ctx, rope, temb)
        assert torch.equal(ra[0], rf[0]) and torch.equal(ra[1], rf[1])
    sa = classes.FluxSingleTransformerBlockOp("bf16", d, heads, dh, 4, 2)
    sa.reload_model_from_state_dict("single_transformer_blocks.9.", sd, "cpu")
    sf = classes.FluxSingleTransformerBlockOp("bf16", d, heads, dh, 4, 2)
    sf.reload_model_from_bin(str(tmp_path) + "/single_transformer_blocks.9.", file_dtype)
    xs = torch.cat([ctx, x], dim=1).contiguous()
    assert torch.equal(sa.forward(xs, rope, temb), sf.forward(xs, rope, temb))
    with pytest.raises(RuntimeError, match="cannot be opened"):
        sf.reload_model_from_bin(str(tmp_path) + "/absent.", "fp32")
    (tmp_path / "short.norm.linear.weight.bin").write_bytes(b"\0" * 10)
    with pytest.raises(RuntimeError, match="does not hold"):
        sf.reload_model_from_bin(str(tmp_path) + "/short.", "fp32")


@pytest.mark.gpu
@pytest.mark.parametrize("level", [8, 7])
def test_int4_block_classes_equal_the_python_ops(classes, ops, dev, level):
    from lyradiff_amd import flux_ops as FO

    b, s, sc, heads, dh = 1, 128, 64, 4, 64
    d = heads * dh
    g = rng_t(401)
    sd = _int4_block_state(d, dh, g)
    x, ctx, temb, rope = _fp8_inputs(dev, b, s, sc, heads, dh, 521)
    op = classes.FluxTransformerBlockOp("bf16", d, heads, dh, 6, level)
    op.reload_model_from_state_dict("transformer_blocks.0.", sd, "cpu")
    py = FO.FluxTransformerBlockOp("bf16", d, heads, dh, 6, level)
    py.reload_model_from_state_dict("transformer_blocks.0.", sd, "cpu")
    out, cout = op.forward(x, ctx, rope, temb)
    pout, pcout = py.forward(x, ctx, rope, temb)
    assert torch.equal(out, pout) and torch.equal(cout, pcout) and torch.isfinite(out.float()).all()
    with pytest.raises(RuntimeError, match="INT4 blocks carry their low-rank branch"):
        op.load_lora_by_name(["attn", "to_qkv"], torch.zeros(3 * d, d).bfloat16().to(dev), 1.0)
    op.clear_lora()

    sop = classes.FluxSingleTransformerBlockOp("bf16", d, heads, dh, 4, level)
    sop.reload_model_from_state_dict("single_transformer_blocks.0.", sd, "cpu")
    spy = FO.FluxSingleTransformerBlockOp("bf16", d, heads, dh, 4, level)
    spy.reload_model_from_state_dict("single_transformer_blocks.0.", sd, "cpu")
    xs = torch.cat([ctx, x], dim=1).contiguous()
    y = sop.forward(xs, rope, temb)
    assert torch.equal(y, spy.forward(xs, rope, temb)) and torch.isfinite(y.float()).all()


@pytest.mark.gpu
@pytest.mark.parametrize("level", [8, 7])
def test_int4_block_classes_match_the_fp64_restatement(classes, ops, dev, level):
    """The C++ classes at both INT4 levels directly against oracle/flux_blocks_f64.py, with its mis-wired variants."""
    check_int4_blocks_against_the_restatement(lambda d, h, dh: classes.FluxTransformerBlockOp("bf16", d, h, dh, 4, level),
                                              lambda d, h, dh: classes.FluxSingleTransformerBlockOp("bf16", d, h, dh, 4, level),
                                              dev, level == 8)


@pytest.mark.gpu
def test_int4_block_classes_reload_model_from_bin_and_fp16(classes, ops, dev, tmp_path):
    """The INT4 checkpoints as raw files (packed codes int8, scales and smoothing vectors fp32, 16-bit members in the model
    file type) give the same bits as the state-dict route; an fp16 block runs and equals the Python class."""
    from lyradiff_amd import flux_ops as FO

    b, s, sc, heads, dh = 2, 64, 32, 4, 64
    d = heads * dh
    sd = _int4_block_state(d, dh, rng_t(431))
    for k, v in sd.items():
        (v.float().numpy() if v.dtype == torch.bfloat16 else v.numpy()).tofile(str(tmp_path / (k + ".bin")))
    x, ctx, temb, rope = _fp8_inputs(dev, b, s, sc, heads, dh, 531)
    for level in (8, 7):
        a = classes.FluxTransformerBlockOp("bf16", d, heads, dh, 6, level)
        a.reload_model_from_state_dict("transformer_blocks.0.", sd, "cpu")
        f = classes.FluxTransformerBlockOp("bf16", d, heads, dh, 6, level)
        f.reload_model_from_bin(str(tmp_path) + "/transformer_blocks.0.", "fp32")
        ra, rf = a.forward(x, ctx, rope, temb), f.forward(x, ctx, rope, temb)
        assert torch.equal(ra[0], rf[0]) and torch.equal(ra[1], rf[1])
    xs = torch.cat([ctx, x], dim=1).contiguous()
    sa = classes.FluxSingleTransformerBlockOp("bf16", d, heads, dh, 4, 8)
    sa.reload_model_from_state_dict("single_transformer_blocks.0.", sd, "cpu")
    sf = classes.FluxSingleTransformerBlockOp("bf16", d, heads, dh, 4, 8)
    sf.reload_model_from_bin(str(tmp_path) + "/single_transformer_blocks.0.", "fp32")
    assert torch.equal(sa.forward(xs, rope, temb), sf.forward(xs, rope, temb))
    # fp16 inference dtype, FP8 level, batch of two
    sd16 = {k: (v.half() if v.dtype == torch.bfloat16 else v) for k, v in _block_state(d, dh, 432, ("t.", "s.")).items()}
    op = classes.FluxSingleTransformerBlockOp("fp16", d, heads, dh, 4, 2)
    op.reload_model_from_state_dict("s.", sd16, "cpu")
    py = FO.FluxSingleTransformerBlockOp("fp16", d, heads, dh, 4, 2)
    py.reload_model_from_state_dict("s.", sd16, "cpu")
    y = op.forward(xs.half(), rope.half(), temb.half())
    assert torch.equal(y, py.forward(xs.half(), rope.half(), temb.half())) and torch.isfinite(y.float()).all()
    with pytest.raises(RuntimeError, match="hidden_states dtype should be"):
        op.forward(xs, rope.half(), temb.half())
