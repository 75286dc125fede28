"""Helpers shared by the GPU parity tests."""

import numpy as np
import torch

# Stated tolerances: max abs error against the fp32 oracle for values of
# magnitude <= 1, the same figure relative to |value| above 1 (a stored bf16 of
# magnitude 4 cannot be closer than 2^-7 to an arbitrary real).
TOL = {torch.float32: 1e-6, torch.float16: 2e-3, torch.bfloat16: 2e-3}
DTYPES = [torch.float32, torch.float16, torch.bfloat16]
IDS = {torch.float32: "fp32", torch.float16: "fp16", torch.bfloat16: "bf16"}


def randn(shape, dtype, seed, std=1.0):
    """Seeded N(0, std^2) values rounded to `dtype`, as a CPU tensor."""
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g, dtype=torch.float32) * std).to(dtype)


def f32(t):
    """Exact fp32 numpy view of a tensor's values."""
    return t.detach().to("cpu", torch.float32).numpy()


def assert_close(got, want, dtype, what=""):
    got = f32(got) if isinstance(got, torch.Tensor) else np.asarray(got, dtype=np.float32)
    want = np.asarray(want, dtype=np.float32)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    assert np.isfinite(got).all(), f"{what}: non-finite values in the kernel output"
    err = np.abs(got.astype(np.float64) - want.astype(np.float64)) / np.maximum(1.0, np.abs(want))
    worst = float(err.max()) if err.size else 0.0
    assert worst <= TOL[dtype], f"{what}: max error {worst:.3e} > {TOL[dtype]:.1e} ({IDS[dtype]})"
    return worst
