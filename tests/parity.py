"""Shared helpers for the parity tests: tolerances, seeded inputs and conversions."""
import numpy as np
import torch

# Normwise bar max|a-b| / max|b| per tensor: fp32 <= 1e-5; bf16/fp16 <= 1e-2 against the
# float64 oracle evaluated on identically rounded inputs.
TOL = {torch.float32: 1e-5, torch.float16: 1e-2, torch.bfloat16: 1e-2}


def rel_err(got, ref):
    got = got.detach().double().cpu().numpy() if isinstance(got, torch.Tensor) else np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    if ref.size == 0:
        return 0.0
    assert np.all(np.isfinite(got)), "non-finite values in device result"
    return float(np.max(np.abs(got - ref)) / max(np.max(np.abs(ref)), 1e-30))


def assert_close(got, ref, dtype, what="", scale=1.0):
    e = rel_err(got, ref)
    assert e <= TOL[dtype] * scale, f"{what}: normwise error {e:.3e} > {TOL[dtype] * scale:.1e} ({dtype})"
    return e


def rounded(t, dtype):
    """fp32 CPU draw -> rounded to dtype; returns (device-ready tensor of dtype, float64 numpy of the rounded values)."""
    r = t.to(dtype)
    return r, r.double().numpy()


def randn(gen, *shape):
    return torch.randn(*shape, generator=gen, dtype=torch.float32)
