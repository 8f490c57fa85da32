"""Shared helpers for the parity tests (oracle on CPU vs HIP through the C ABI)."""
import numpy as np
import torch

TORCH_DT = {"f16": torch.float16, "bf16": torch.bfloat16, "f32": torch.float32}


def rng_t(seed):
    return torch.Generator().manual_seed(seed)


def to_np_f32(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().to(torch.float32).numpy()


def ulp_f16(ref: np.ndarray) -> np.ndarray:
    """Size of one fp16 ULP at |ref| (2^-24 in the subnormal range)."""
    a = np.maximum(np.abs(ref.astype(np.float64)), 2.0 ** -14)
    return np.exp2(np.floor(np.log2(a)) - 10)


def assert_close_tol(got: np.ndarray, ref: np.ndarray, what: str = "", abs_floor=None):
    """The tolerance stated by the task: |d| <= 1e-2*|ref|  OR  |d| <= 2 fp16 ULP at |ref|.

    abs_floor (optional, per element): an extra absolute allowance for kernels whose fp32
    summation order is free (FP8 GEMM): a few fp32 ULPs of the sum of |terms|, the error any
    fp32 accumulation has when the terms cancel to a result near zero."""
    got = got.astype(np.float64)
    ref64 = ref.astype(np.float64)
    d = np.abs(got - ref64)
    ok = (d <= 1e-2 * np.abs(ref64)) | (d <= 2 * ulp_f16(ref))
    if abs_floor is not None:
        ok |= d <= abs_floor
    bad = int((~ok).sum())
    assert bad == 0, f"{what}: {bad} of {ok.size} outside 1e-2 rel / 2 fp16 ULP; max abs diff {d.max():.4g}"


def make_outlier_acts(m, k, n_out, mag, dtype, seed):
    g = rng_t(seed)
    x = torch.randn(m, k, generator=g)
    cols = torch.randperm(k, generator=g)[:n_out]
    x[:, cols] = torch.randn(m, n_out, generator=g) * mag
    return x.to(dtype)
