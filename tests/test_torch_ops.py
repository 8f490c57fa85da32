"""torch.ops.lyradiff.* registration: schema and shape inference on the CPU, parity with the direct
wrappers on the GPU (the operator bodies call the same C ABI entry points)."""
import numpy as np
import pytest
import torch
from torch._subclasses.fake_tensor import FakeTensorMode


@pytest.fixture(scope="module")
def tops():
    import lyradiff_amd.torch_ops as t

    return t


def test_every_operator_is_registered(tops):
    for name in tops.NAMES:
        assert hasattr(torch.ops.lyradiff, name), name
        getattr(torch.ops.lyradiff, name).default  # resolves the overload


def test_shape_inference_without_a_gpu(tops):
    with FakeTensorMode():
        dev = "cuda"
        x = torch.empty(4, 77, 640, dtype=torch.float16, device=dev)
        q, s = torch.ops.lyradiff.sq_quant_dynamic(x, None)
        assert q.shape == x.shape and q.dtype == torch.int8 and s.shape == (4 * 77,) and s.dtype == torch.float32
        w = torch.empty(1280, 640, dtype=torch.int8, device=dev)
        y = torch.ops.lyradiff.int8_linear(q.reshape(-1, 640), w, s, s, None, torch.float16)
        assert y.shape == (308, 1280) and y.dtype == torch.float16
        h = torch.empty(308, 5120, dtype=torch.float16, device=dev)
        q2, s2 = torch.ops.lyradiff.geglu_int8_dynamic(h)
        assert q2.shape == (308, 2560) and s2.shape == (308,)
        xb = torch.empty(4608, 3072, dtype=torch.bfloat16, device=dev)
        qf, sf = torch.ops.lyradiff.fp8_quant(xb)
        assert qf.dtype == torch.uint8 and qf.shape == xb.shape and sf.shape == (1,)
        wf = torch.empty(12288, 3072, dtype=torch.uint8, device=dev)
        yf = torch.ops.lyradiff.fp8_linear(qf, wf, sf, sf, None, True)
        assert yf.shape == (4608, 12288) and yf.dtype == torch.bfloat16
        qa, sa = torch.ops.lyradiff.w4a4_quant(xb, None, torch.float16)
        assert qa.shape == (4608, 384) and qa.dtype == torch.int32 and sa.shape == (4608, 48) and sa.dtype == torch.float16
        w4 = torch.empty(3072, 1536, dtype=torch.uint8, device=dev)
        y4 = torch.ops.lyradiff.w4a4_linear(qa, w4, sa, sa[:3072], None)
        assert y4.shape == (4608, 3072) and y4.dtype == torch.bfloat16
        assert torch.ops.lyradiff.repack_weight(w4).shape == w4.shape


def test_host_tensors_are_rejected(tops):
    # the reference's CHECK_TH_CUDA (src/lyradiff/th_op/th_utils.h:14-33): no silent CPU path
    with pytest.raises(ValueError, match="CUDA"):
        torch.ops.lyradiff.repack_weight(torch.zeros(32, 64, dtype=torch.int8))
    with pytest.raises(ValueError, match="CUDA"):
        torch.ops.lyradiff.fp8_quant(torch.zeros(8, 64, dtype=torch.bfloat16))


@pytest.mark.gpu
def test_operators_match_direct_wrappers(tops, dev):
    from lyradiff_amd import ops

    g = torch.Generator().manual_seed(7)
    x = torch.randn(300, 640, generator=g).half().to(dev)
    w = torch.randint(-127, 128, (320, 640), generator=g, dtype=torch.int8).to(dev)
    ws = (torch.rand(320, generator=g) * 1e-2).to(dev)
    q, s = torch.ops.lyradiff.sq_quant_dynamic(x, None)
    q0, s0 = ops.sq_quant_dynamic(x, None)
    assert torch.equal(q, q0) and torch.equal(s, s0)
    wp = torch.ops.lyradiff.repack_weight(w)
    assert torch.equal(torch.ops.lyradiff.int8_linear(q, wp, ws, s, None, torch.float16), ops.int8_linear(q0, wp, ws, s0))
    xb = torch.randn(256, 512, generator=g).bfloat16().to(dev)
    qf, sf = torch.ops.lyradiff.fp8_quant(xb)
    qf0, sf0 = ops.fp8_quant(xb)
    assert torch.equal(qf, qf0) and torch.equal(sf, sf0)
    wf = torch.ops.lyradiff.repack_weight(qf[:128].contiguous())
    assert torch.equal(torch.ops.lyradiff.fp8_linear(qf, wf, sf, sf, None, True), ops.fp8_linear(qf, wf, sf, sf, None, True))
    qa, sa = torch.ops.lyradiff.w4a4_quant(xb, None, torch.float16)
    w4 = torch.ops.lyradiff.repack_weight(qa[:128].contiguous().view(torch.uint8).reshape(128, 256))
    assert torch.equal(torch.ops.lyradiff.w4a4_linear(qa, w4, sa, sa[:128].contiguous(), None),
                       ops.w4a4_linear(qa, w4, sa, sa[:128].contiguous(), None))
    assert np.isfinite(torch.ops.lyradiff.fp8_scale_cast(xb, sf).float().cpu().numpy()).all()
