"""GPU parity of the LayerNorm + quantisation fusions against the CPU oracle, through the C ABI.

The residual sum h is compared bit for bit.  The quantised codes depend on row statistics whose fp32
summation order is this library's own (the reference's is tied to its thread layout), so they are required
to agree with the oracle (fp64 statistics) to within ONE quantisation step, with at most 0.5 % of the
elements differing at all; the dynamic per-token scale to within one ULP of T at the row maximum."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from tests.helpers import TORCH_DT, rng_t, to_np_f32

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops(dev):
    from lyradiff_amd import ops as _ops

    return _ops


def close_codes(got, ref, what):
    d = np.abs(got.astype(np.int32) - ref.astype(np.int32))
    assert d.max() <= 1, f"{what}: codes differ by {d.max()} steps"
    assert (d != 0).mean() <= 5e-3, f"{what}: {(d != 0).mean():.4%} of the codes differ"


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("rows,dim", [(1024, 1280), (4096, 640), (77, 320), (4608, 3072), (5, 6144), (33, 2056), (7, 4104)])
@pytest.mark.parametrize("dynamic", [False, True])
def test_layernorm_int8(ops, dev, dt, rows, dim, dynamic):
    g = rng_t(rows + dim)
    t = TORCH_DT[dt]
    x = (torch.randn(rows, dim, generator=g) * 2 + 0.3).to(t)
    gamma = (1 + 0.1 * torch.randn(dim, generator=g)).to(t)
    beta = (0.1 * torch.randn(dim, generator=g)).to(t)
    pre = (0.5 + torch.rand(dim, generator=g)).float()
    s_in = torch.tensor([0.031], dtype=torch.float32)
    q, s, h = ops.layernorm_int8(x.to(dev), gamma.to(dev), beta.to(dev), pre.to(dev), None if dynamic else s_in.to(dev))
    q_ref, s_ref, _ = O.layernorm_int8(to_np_f32(x), None, None, to_np_f32(gamma), to_np_f32(beta), pre.numpy(),
                                       None if dynamic else s_in.numpy(), dt)
    assert h is None
    close_codes(q.cpu().numpy(), q_ref, "layernorm int8")
    if dynamic:
        ulp = 2.0 ** (-10 if dt == "f16" else -7)
        assert np.all(np.abs(s.cpu().numpy() - s_ref) <= ulp * s_ref)
    else:
        assert s is None


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("with_bias", [True, False])
def test_fused_residual_bias_layernorm_int8(ops, dev, dt, with_bias):
    rows, dim = 2048, 1280
    g = rng_t(11)
    t = TORCH_DT[dt]
    x = torch.randn(rows, dim, generator=g).to(t)
    res = torch.randn(rows, dim, generator=g).to(t)
    bias = (0.2 * torch.randn(dim, generator=g)).to(t) if with_bias else None
    gamma = (1 + 0.1 * torch.randn(dim, generator=g)).to(t)
    beta = (0.1 * torch.randn(dim, generator=g)).to(t)
    s_in = torch.tensor([0.02], dtype=torch.float32)
    q, _, h = ops.layernorm_int8(x.to(dev), gamma.to(dev), beta.to(dev), None, s_in.to(dev), res.to(dev),
                                 bias.to(dev) if with_bias else None, eps=1e-5)
    q_ref, _, h_ref = O.layernorm_int8(to_np_f32(x), to_np_f32(res), to_np_f32(bias) if with_bias else None, to_np_f32(gamma),
                                       to_np_f32(beta), None, s_in.numpy(), dt, eps=1e-5)
    assert np.array_equal(to_np_f32(h), h_ref), "the residual sum is plain T arithmetic: bit-exact"
    close_codes(q.cpu().numpy(), q_ref, "fused residual layernorm int8")


@pytest.mark.parametrize("dt", ["bf16", "f16"])
@pytest.mark.parametrize("batch,seq,dim", [(2, 2304, 3072), (1, 512, 3072), (3, 50, 768), (2, 37, 2568)])
def test_layernorm_mod_fp8(ops, dev, dt, batch, seq, dim):
    g = rng_t(batch + seq + dim)
    t = TORCH_DT[dt]
    x = (torch.randn(batch, seq, dim, generator=g) * 1.5).to(t)
    scale = (0.3 * torch.randn(batch, dim, generator=g)).to(t)
    shift = (0.3 * torch.randn(batch, dim, generator=g)).to(t)
    s_in = torch.tensor([0.011], dtype=torch.float32)
    q = ops.layernorm_mod_fp8(x.to(dev), scale.to(dev), shift.to(dev), s_in.to(dev))
    ref = O.layernorm_mod_fp8(to_np_f32(x).reshape(batch * seq, dim), to_np_f32(scale), to_np_f32(shift), s_in.numpy(), seq, dt)
    got = q.cpu().numpy().reshape(batch * seq, dim)
    assert (got != ref).mean() <= 5e-3, f"{(got != ref).mean():.4%} of the codes differ"
    # Where they differ: by one e4m3 step, or -- where (1+scale)*n and shift cancel -- by what one ULP of T in the
    # normalised value moves the sum (the statistics' summation order decides such last bits).
    gv, rv = O.e4m3_decode(got).astype(np.float64), O.e4m3_decode(ref).astype(np.float64)
    step = np.maximum(np.exp2(np.floor(np.log2(np.maximum(np.abs(rv), 2.0 ** -6))) - 3), 2.0 ** -9)
    b = np.arange(batch * seq) // seq
    n = np.abs(O._ln_normalised(to_np_f32(x).reshape(batch * seq, dim), 1e-6)).astype(np.float64)
    mag = (np.abs(to_np_f32(scale).astype(np.float64))[b] + 1.0) * n + np.abs(to_np_f32(shift).astype(np.float64))[b]
    ulp_t = 2.0 ** (-10 if dt == "f16" else -7)
    assert np.all(np.abs(gv - rv) <= step + ulp_t * mag / float(s_in[0]))


def test_layernorm_constant_rows_and_argument_checks(ops, dev):
    """A constant row has zero variance: n = 0 and y = beta exactly; bad arguments fail without touching the GPU."""
    from lyradiff_amd.lib import LyraQuantError

    dim = 640
    x = torch.full((8, dim), 3.25, dtype=torch.float16, device=dev)
    gamma = torch.ones(dim, dtype=torch.float16, device=dev)
    beta = torch.full((dim,), 0.5, dtype=torch.float16, device=dev)
    s_in = torch.tensor([0.25], dtype=torch.float32, device=dev)
    q, _, _ = ops.layernorm_int8(x, gamma, beta, None, s_in)
    assert torch.all(q == 2)
    with pytest.raises(LyraQuantError):
        ops.layernorm_int8(x[:, :636].contiguous(), gamma[:636].contiguous(), beta[:636].contiguous(), None, s_in)
    with pytest.raises(LyraQuantError):
        ops.layernorm_int8(x, gamma, beta, None, s_in, None, beta)  # bias without residual
