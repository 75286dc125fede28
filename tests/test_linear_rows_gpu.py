"""The few-row linear layer (a decoding step's projections), called through
the C ABI, against the CPU oracle in float64. Bar: the output is one rounding
of the exact sum, so |err| <= eps(dtype)*|y| plus 1e-6 of sum |x*w| (fp32
accumulation in another order than the oracle's); fp32 storage meets the
second term alone."""

import numpy as np
import pytest
import torch

from oracle import oslo_oracle as orc
from oslo_amd import kernels
from tests.util import DTYPES, IDS, f32, randn

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
EPS = {torch.float32: 2.0 ** -23, torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}


def check(out, x, w, b, gelu, dtype, what):
    xd, wd = f32(x).astype(np.float64), f32(w).astype(np.float64)
    want = orc.linear_rows(xd, wd, None if b is None else f32(b), gelu)
    mass = np.abs(xd)[:, None, :] @ np.abs(wd).T[None]          # sum |x*w| per output
    mass = mass.reshape(want.shape)
    tol = EPS[dtype] * np.abs(want) + 1e-6 * mass + 1e-30
    got = f32(out).astype(np.float64).reshape(want.shape)
    worst = np.max(np.abs(got - want) / tol)
    assert worst <= 1.0, f"{what}: error {worst:.2f} x the bar"


# (m, n, k): every row count, ragged n, k below / at / past one chunk of 64 lanes, k not a
# multiple of the unrolled span, n not a multiple of the rows of a block
SHAPES = [(1, 1, 8), (1, 5, 64), (2, 17, 520), (3, 64, 512), (4, 33, 1032), (5, 130, 4096), (7, 9, 8200),
          (8, 257, 2048), (1, 4096, 4096), (8, 1000, 768)]


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS.get)
@pytest.mark.parametrize("m,n,k", SHAPES)
def test_linear_rows_matches_oracle(m, n, k, dtype):
    x = randn((m, k), dtype, seed=m * 11 + k)
    w = randn((n, k), dtype, seed=n * 13 + k, std=0.05)
    b = randn((n,), dtype, seed=n, std=0.5)
    for bias, gelu in ((None, False), (b, False), (b, True)):
        out = kernels.linear_rows_forward(x.to(DEV), w.to(DEV), None if bias is None else bias.to(DEV), gelu)
        assert out.shape == (m, n) and out.dtype == dtype
        check(out, x, w, bias, gelu, dtype, f"{m}x{n}x{k} bias={bias is not None} gelu={gelu}")


# weight stored [k, n] (Conv1D): n and k multiples of the vector; ragged strips (n not a multiple of
# 8 vectors), k below / past what 16 waves cover in one step
KN_SHAPES = [(1, 8, 8), (2, 24, 64), (3, 2304, 768), (5, 768, 3072), (8, 136, 1032), (4, 3072, 768), (7, 40, 4104)]


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS.get)
@pytest.mark.parametrize("m,n,k", KN_SHAPES)
def test_linear_rows_conv1d_layout_matches_oracle(m, n, k, dtype):
    x = randn((m, k), dtype, seed=m * 11 + k)
    w = randn((k, n), dtype, seed=n * 13 + k, std=0.05)       # [in, out]
    b = randn((n,), dtype, seed=n, std=0.5)
    for bias, gelu in ((None, False), (b, False), (b, True)):
        out = kernels.linear_rows_kn_forward(x.to(DEV), w.to(DEV), None if bias is None else bias.to(DEV), gelu)
        assert out.shape == (m, n) and out.dtype == dtype
        check(out, x, w.t().contiguous(), bias, gelu, dtype, f"kn {m}x{n}x{k} bias={bias is not None} gelu={gelu}")
    if n != k:
        with pytest.raises(RuntimeError):
            kernels.linear_rows_kn_forward(x.to(DEV), w.t().contiguous().to(DEV))   # the other layout


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS.get)
@pytest.mark.parametrize("m,n,k", [(1, 64, 512), (3, 130, 1032), (8, 4096, 1024)])
def test_linear_rows_three_layers_in_one_launch(m, n, k, dtype):
    """The multi-layer launch gives, bit for bit, what three single launches give."""
    x = randn((m, k), dtype, seed=1).to(DEV)
    ws = [randn((n, k), dtype, seed=10 + j, std=0.05).to(DEV) for j in range(3)]
    bs = [randn((n,), dtype, seed=20, std=0.5).to(DEV), None, randn((n,), dtype, seed=22, std=0.5).to(DEV)]
    outs = kernels.linear_rows_forward_multi(x, ws, bs)
    for w, b, out in zip(ws, bs, outs):
        assert torch.equal(out, kernels.linear_rows_forward(x, w, b))
    two = kernels.linear_rows_forward_multi(x, ws[:2], None, gelu=True)
    assert torch.equal(two[1], kernels.linear_rows_forward(x, ws[1], None, gelu=True))
    with pytest.raises(RuntimeError):
        kernels.linear_rows_forward_multi(x, ws + ws[:1])
    with pytest.raises(RuntimeError):
        kernels.linear_rows_forward_multi(x, [ws[0], ws[1][:-1]])


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS.get)
@pytest.mark.parametrize("m,n,k", [(1, 72, 512), (3, 136, 1032), (8, 264, 2048)])
def test_linear_rows_residual_epilogue(m, n, k, dtype):
    """act(x.w + b) + residual in one launch, both weight layouts: one rounding
    of the float64 value; in place over the residual too."""
    x = randn((m, k), dtype, seed=1)
    w = randn((n, k), dtype, seed=2, std=0.05)
    b = randn((n,), dtype, seed=3, std=0.5)
    res = randn((m, n), dtype, seed=4, std=2.0)
    for gelu in (False, True):
        want = orc.linear_rows(f32(x), f32(w), f32(b), gelu) + f32(res).astype(np.float64)
        mass = (np.abs(f32(x)).astype(np.float64) @ np.abs(f32(w)).astype(np.float64).T) + np.abs(f32(res))
        tol = EPS[dtype] * np.abs(want) + 1e-6 * mass + 1e-30
        nk = kernels.linear_rows_forward(x.to(DEV), w.to(DEV), b.to(DEV), gelu, res.to(DEV))
        kn = kernels.linear_rows_kn_forward(x.to(DEV), w.t().contiguous().to(DEV), b.to(DEV), gelu, res.to(DEV))
        for out in (nk, kn):
            assert np.max(np.abs(f32(out).astype(np.float64) - want) / tol) <= 1.0
    with pytest.raises(RuntimeError):
        kernels.linear_rows_forward(x.to(DEV), w.to(DEV), None, False, res[:, :-1].to(DEV))
    with pytest.raises(RuntimeError):
        kernels.linear_rows_forward_multi(x.to(DEV), [w.to(DEV), w.to(DEV)], None, False, res.to(DEV))


def test_linear_rows_leading_dims_and_torch_agreement():
    """[B, 1, K] inputs as the modules pass them; against torch's own linear +
    gelu on the device, within bf16 rounding of the two-step path."""
    dtype = torch.bfloat16
    x = randn((4, 1, 1024), dtype, seed=1).to(DEV)
    w = randn((3072, 1024), dtype, seed=2, std=0.03).to(DEV)
    b = randn((3072,), dtype, seed=3, std=0.1).to(DEV)
    out = kernels.linear_rows_forward(x, w, b, gelu=True)
    assert out.shape == (4, 1, 3072)
    ref = torch.nn.functional.gelu(torch.nn.functional.linear(x.float(), w.float(), b.float()), approximate="tanh")
    assert (out.float() - ref).abs().max() <= 2.0 ** -7 * ref.abs().max()


def test_linear_rows_errors():
    x = torch.zeros(2, 64, device=DEV)
    w = torch.zeros(8, 64, device=DEV)
    with pytest.raises(RuntimeError):
        kernels.linear_rows_forward(torch.zeros(9, 64, device=DEV), w)          # too many rows
    with pytest.raises(RuntimeError):
        kernels.linear_rows_forward(x, torch.zeros(8, 32, device=DEV))          # k mismatch
    with pytest.raises(RuntimeError):
        kernels.linear_rows_forward(x, w.half())                                # dtype mismatch
    with pytest.raises(RuntimeError):
        kernels.linear_rows_forward(x, w, torch.zeros(7, device=DEV))           # bias length
    with pytest.raises(RuntimeError):
        kernels.linear_rows_forward(x.cpu(), w.cpu())                           # no CPU path
    with pytest.raises(RuntimeError):
        kernels.linear_rows_forward(torch.zeros(2, 6, device=DEV), torch.zeros(8, 6, device=DEV))  # ragged rows
    assert kernels.linear_rows_forward(torch.zeros(0, 64, device=DEV), w).shape == (0, 8)
