"""Helpers shared by the GPU parity tests."""

import numpy as np
import torch

# Stated tolerances: max abs error against the fp32 oracle for values of
# magnitude <= 1 (softmax outputs, most gradients). Above magnitude 1 the same
# figure is taken relative to |value|, except for bf16, where even the
# correctly rounded result is up to half an ulp = 2^-8 relative away: there the
# bar is that half ulp (plus 0.1 % slack for the fp32 evaluation error).
TOL = {torch.float32: 1e-6, torch.float16: 2e-3, torch.bfloat16: 2e-3}
REL_ABOVE_ONE = {torch.float32: 1e-6, torch.float16: 2e-3, torch.bfloat16: 2.0 ** -8 * 1.001}
DTYPES = [torch.float32, torch.float16, torch.bfloat16]
IDS = {torch.float32: "fp32", torch.float16: "fp16", torch.bfloat16: "bf16"}


def oracle_dtype(dtype):
    """Precision the GeLU-gradient oracle is evaluated in. Everywhere else the
    oracle runs in fp32 with the reference's own order of operations (which is
    what decides, e.g., a fully masked softmax row, where scale*x - 10000 is
    rounded at magnitude 1e4). The GeLU gradient is the exception: the
    reference's formula forms 1 - tanh^2, which in fp32 loses two digits to
    cancellation, so its fp32 evaluation is itself up to 4e-6 away from the
    value of the expression. fp32 kernels are therefore compared with the
    float64 evaluation of that expression; 16-bit kernels with the fp32 one."""
    return np.float64 if dtype == torch.float32 else np.float32


def bf16_half_ulps(want):
    """Sum over the last axis of half an ulp of each value's bf16 neighbourhood:
    what storing a row in bf16 can move its sum by."""
    w = np.abs(np.asarray(want, dtype=np.float64))
    e = np.floor(np.log2(np.maximum(w, 2.0 ** -126)))
    return np.where(w > 0, 2.0 ** (e - 8), 0.0).sum(-1)


def assert_colsum_close(got, want, l1_mass, dtype, what="dbias"):
    """Bias gradient: an fp32 sum over rows stored in `dtype`. Bar: the storage
    bar of assert_close on the value plus 1e-6 of the column's L1 mass (the
    error scale of fp32 summation)."""
    got = f32(got).astype(np.float64)
    want = np.asarray(want, dtype=np.float64)
    bound = np.maximum(TOL[dtype], REL_ABOVE_ONE[dtype] * np.abs(want)) + 1e-6 * np.asarray(l1_mass, dtype=np.float64)
    ratio = np.abs(got - want) / bound
    assert ratio.max() <= 1.0, f"{what}: {ratio.max():.2f}x the bar ({IDS[dtype]})"


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
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    bound = np.maximum(TOL[dtype], REL_ABOVE_ONE[dtype] * np.abs(want.astype(np.float64)))
    ratio = err / bound
    worst = float(ratio.max()) if ratio.size else 0.0
    assert worst <= 1.0, (f"{what}: error {float(err.max()):.3e} is {worst:.2f}x the bar "
                          f"({TOL[dtype]:.1e} abs / {REL_ABOVE_ONE[dtype]:.2e} rel, {IDS[dtype]})")
    return worst
