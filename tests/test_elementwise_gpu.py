"""Parity of the bias-GeLU and bias-dropout(-residual) kernels, called through
the C ABI, with the CPU oracle. fp32 <= 1e-6, fp16/bf16 <= 2e-3 (relative above
magnitude 1). The dropout keep mask must equal the oracle's bit for bit."""

import numpy as np
import pytest
import torch

from oracle import oslo_oracle as orc
from oslo_amd import kernels
from tests.util import DTYPES, IDS, assert_close, assert_colsum_close, f32, oracle_dtype, randn

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
# (rows, cols): vector path, ragged tails, narrow and wide, column counts that
# are not a multiple of the vector width, more rows than one block range
SHAPES = [(1, 8), (3, 1), (5, 7), (33, 768), (129, 3072), (300, 4096), (257, 1000), (64, 16384), (2, 20000), (1025, 24)]


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS.get)
@pytest.mark.parametrize("rows,cols", SHAPES)
def test_bias_gelu_forward(rows, cols, dtype):
    y = randn((rows, cols), dtype, seed=rows * 7 + cols, std=2.0)
    b = randn((cols,), dtype, seed=cols, std=0.5)
    want = orc.bias_gelu_fwd(f32(y), f32(b))
    out = kernels.bias_gelu_forward(y.to(DEV), b.to(DEV))
    assert out.dtype == dtype and out.shape == y.shape
    assert_close(out, want, dtype, f"bias_gelu fwd {rows}x{cols}")


def test_bias_gelu_forward_extremes_and_leading_dims():
    y = torch.tensor([[0.0, 30.0, -30.0, 1e4, -1e4, 1e-8, -1e-8, 5.0]], dtype=torch.float32)
    b = torch.zeros(8)
    out = kernels.bias_gelu_forward(y.to(DEV), b.to(DEV))
    assert_close(out, orc.bias_gelu_fwd(y.numpy(), b.numpy(), dtype=np.float64), torch.float32)
    assert abs(f32(out)[0, 4]) < 1e-30 and f32(out)[0, 3] == 1e4
    y3 = randn((4, 6, 64), torch.bfloat16, seed=1)
    b3 = randn((64,), torch.bfloat16, seed=2)
    out3 = kernels.bias_gelu_forward(y3.to(DEV), b3.to(DEV))
    assert out3.shape == y3.shape
    assert_close(out3, orc.bias_gelu_fwd(f32(y3), f32(b3)), torch.bfloat16)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS.get)
@pytest.mark.parametrize("rows,cols", SHAPES)
def test_bias_gelu_backward(rows, cols, dtype):
    y = randn((rows, cols), dtype, seed=rows * 7 + cols, std=2.0)
    b = randn((cols,), dtype, seed=cols, std=0.5)
    g = randn((rows, cols), dtype, seed=rows + cols)
    want_dy, want_db = orc.bias_gelu_bwd(f32(g), f32(y), f32(b), dtype=oracle_dtype(dtype))
    dy, db = kernels.bias_gelu_backward(g.to(DEV), y.to(DEV), b.to(DEV))
    assert_close(dy, want_dy, dtype, f"bias_gelu bwd {rows}x{cols}")
    assert_colsum_close(db, want_db, np.abs(want_dy).sum(0), dtype)
    dy2, none = kernels.bias_gelu_backward(g.to(DEV), y.to(DEV), b.to(DEV), want_dbias=False)
    assert none is None and torch.equal(dy2, dy)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS.get)
@pytest.mark.parametrize("rows,cols", SHAPES)
@pytest.mark.parametrize("p", [0.1, 0.5])
def test_bias_dropout_add_forward_backward(rows, cols, dtype, p):
    seed, offset = 1234, 8
    x = randn((rows, cols), dtype, seed=rows * 3 + cols)
    res = randn((rows, cols), dtype, seed=rows * 5 + cols)
    b = randn((cols,), dtype, seed=cols, std=0.02)
    keep = orc.dropout_keep_mask(seed, offset, rows * cols, p).reshape(rows, cols)
    od = np.float32
    want = orc.bias_dropout_add_fwd(f32(x), f32(b), f32(res), p, keep, dtype=od)
    out = kernels.bias_dropout_add_forward(x.to(DEV), b.to(DEV), res.to(DEV), p, seed, offset)
    assert_close(out, want, dtype, f"bias_dropout_add fwd {rows}x{cols}")
    # the mask itself, bit for bit: without bias/residual a dropped element is exactly 0
    ones = torch.ones((rows, cols), dtype=dtype, device=DEV)
    m = kernels.bias_dropout_add_forward(ones, None, None, p, seed, offset)
    assert np.array_equal(f32(m) != 0, keep)
    # no residual
    out2 = kernels.bias_dropout_add_forward(x.to(DEV), b.to(DEV), None, p, seed, offset)
    assert_close(out2, orc.bias_dropout_add_fwd(f32(x), f32(b), None, p, keep, dtype=od), dtype)
    # backward regenerates the same mask
    g = randn((rows, cols), dtype, seed=rows + cols + 1)
    want_dx, want_db, _ = orc.bias_dropout_add_bwd(f32(g), p, keep, dtype=od)
    dx, db = kernels.bias_dropout_add_backward(g.to(DEV), p, seed, offset)
    assert_close(dx, want_dx, dtype, "bias_dropout_add bwd")
    assert np.array_equal(f32(dx) != 0, keep & (f32(g) != 0))
    assert_colsum_close(db, want_db, np.abs(want_dx).sum(0), dtype)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS.get)
@pytest.mark.parametrize("rows,cols", [(1, 8), (37, 264), (64, 1000), (129, 4096), (5, 7)])
def test_bias_dropout_add_two_residuals(rows, cols, dtype):
    """out = dropout(x + bias) + residual + residual2 in one pass (GPT-J's block
    sum): against the oracle with the kernel's keep mask; at p = 0 the exact
    fp32 sum of the four terms rounded once; without a bias; and through the
    operator under autograd, where both residuals receive the gradient itself."""
    from oslo_amd import FusedBiasDropoutResidual

    seed, offset, p = 99, 4, 0.25
    x, res, res2 = (randn((rows, cols), dtype, seed=rows + cols + i) for i in range(3))
    b = randn((cols,), dtype, seed=cols, std=0.02)
    keep = orc.dropout_keep_mask(seed, offset, rows * cols, p).reshape(rows, cols)
    dev = [t.to(DEV) for t in (x, b, res, res2)]
    out = kernels.bias_dropout_add_forward(dev[0], dev[1], dev[2], p, seed, offset, dev[3])
    want = orc.bias_dropout_add_fwd(f32(x), f32(b), f32(res), p, keep, residual2=f32(res2))
    assert_close(out, want, dtype, f"two residuals {rows}x{cols}")
    out = kernels.bias_dropout_add_forward(dev[0], None, dev[2], p, seed, offset, dev[3])
    assert_close(out, orc.bias_dropout_add_fwd(f32(x), None, f32(res), p, keep, residual2=f32(res2)), dtype)
    exact = kernels.bias_dropout_add_forward(dev[0], dev[1], dev[2], 0.0, 0, 0, dev[3])
    if dtype == torch.float32:
        want0 = ((x + b) + res) + res2                       # the kernel's order of fp32 additions
    else:
        want0 = (x.double() + b.double() + res.double() + res2.double())
        # (the fp32 sum of four 16-bit values may be off the exact sum by an fp32 ulp before its one rounding)
        assert (exact.cpu().double() - want0).abs().max() <= (2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11) * \
            want0.abs().max() + 1e-6
        want0 = None
    if want0 is not None:
        assert torch.equal(exact.cpu(), want0)
    with pytest.raises(RuntimeError):
        kernels.bias_dropout_add_forward(dev[0], dev[1], None, p, seed, offset, dev[3])   # second without first
    # the operator: reference signature plus the optional second residual
    xs = [t.clone().requires_grad_(True) for t in dev]
    torch.manual_seed(5)
    y = FusedBiasDropoutResidual.apply(xs[0], xs[1], xs[2], True, p, xs[3])
    go = randn((rows, cols), dtype, seed=7).to(DEV)
    y.backward(go)
    assert torch.equal(xs[2].grad, go) and torch.equal(xs[3].grad, go)
    dropped = f32(xs[0].grad) == 0
    assert_close(xs[0].grad, np.where(dropped, 0.0, f32(go) / (1 - p)), dtype, "dx")
    assert abs(dropped.mean() - p) <= 0.2 or rows * cols < 200
    # in eval mode the operator is the plain four-term sum
    y0 = FusedBiasDropoutResidual.apply(dev[0], dev[1], dev[2], False, p, dev[3])
    assert torch.equal(y0, exact)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS.get)
def test_bias_dropout_add_p0_is_exact(dtype):
    x = randn((37, 264), dtype, seed=1)
    res = randn((37, 264), dtype, seed=2)
    b = randn((264,), dtype, seed=3)
    out = kernels.bias_dropout_add_forward(x.to(DEV), b.to(DEV), res.to(DEV), 0.0, 0, 0)
    want = (x.float() + b.float() + res.float()).to(dtype)   # one rounding of the exact fp32 sum
    assert torch.equal(out.cpu(), want)
    g = randn((37, 264), dtype, seed=4)
    dx, db = kernels.bias_dropout_add_backward(g.to(DEV), 0.0, 0, 0)
    assert torch.equal(dx.cpu(), g)


def test_dropout_keep_rate_and_seed_offset_semantics():
    n_rows, n_cols, p = 4096, 1024, 0.1
    ones = torch.ones((n_rows, n_cols), dtype=torch.bfloat16, device=DEV)
    a = kernels.bias_dropout_add_forward(ones, None, None, p, 1234, 0)
    rate = float((a != 0).float().mean())
    sigma = (p * (1 - p) / (n_rows * n_cols)) ** 0.5
    assert abs(rate - (1 - p)) < 4 * sigma
    assert torch.equal(a, kernels.bias_dropout_add_forward(ones, None, None, p, 1234, 0))
    assert not torch.equal(a, kernels.bias_dropout_add_forward(ones, None, None, p, 1234, 4))
    assert not torch.equal(a, kernels.bias_dropout_add_forward(ones, None, None, p, 1235, 0))
    kept = a[a != 0].float()
    assert float((kept - 1 / (1 - p)).abs().max()) < 5e-3       # survivors scaled by 1/(1-p)
    # 64-bit seed and offset are honoured
    big = kernels.bias_dropout_add_forward(ones[:8], None, None, 0.5, 0xDEADBEEFCAFEF00D, (1 << 40) + 4)
    keep = orc.dropout_keep_mask(0xDEADBEEFCAFEF00D, (1 << 40) + 4, 8 * n_cols, 0.5).reshape(8, n_cols)
    assert np.array_equal(f32(big) != 0, keep)


def test_elementwise_errors():
    x = torch.zeros(4, 8, device=DEV)
    with pytest.raises(RuntimeError):
        kernels.bias_gelu_forward(x, torch.zeros(7, device=DEV))
    with pytest.raises(RuntimeError):
        kernels.bias_gelu_forward(x.cpu(), torch.zeros(8))
    with pytest.raises(RuntimeError):
        kernels.bias_dropout_add_forward(x, None, None, 1.0, 0, 0)
    with pytest.raises(RuntimeError):
        kernels.bias_dropout_add_forward(x, torch.zeros(8, device=DEV, dtype=torch.half), None, 0.1, 0, 0)


def test_full_size_bias_gelu_and_dropout_properties():
    """The benchmark shapes: [16384,16384] bias-GeLU and [16384,4096] dropout-add in
    bf16; oracle on a band of rows, structural properties on the whole."""
    dtype = torch.bfloat16
    g = torch.Generator(device=DEV).manual_seed(0)
    rows, cols = 16384, 16384
    y = torch.randn((rows, cols), generator=g, device=DEV, dtype=torch.float32).to(dtype)
    b = (torch.randn((cols,), generator=g, device=DEV, dtype=torch.float32) * 0.02).to(dtype)
    out = kernels.bias_gelu_forward(y, b)
    for r0 in (0, 8000, 16380):
        assert_close(out[r0:r0 + 4], orc.bias_gelu_fwd(f32(y[r0:r0 + 4]), f32(b)), dtype, f"rows {r0}")
    go = torch.randn((rows, cols), generator=g, device=DEV, dtype=torch.float32).to(dtype)
    dy, db = kernels.bias_gelu_backward(go, y, b)
    want_dy, _ = orc.bias_gelu_bwd(f32(go[5000:5004]), f32(y[5000:5004]), f32(b))
    assert_close(dy[5000:5004], want_dy, dtype, "bwd band")
    # dbias against the column sum of the kernel's own dy, summed in float64 on
    # the device. dy is stored rounded (each entry up to 2^-9 relative off, so
    # the sum of `rows` of them moves by up to 2^-9 of the column's L1 mass)
    # while dbias sums the unrounded products: that is added to the bar.
    colsum = dy.double().sum(0).cpu().numpy()
    l1 = dy.double().abs().sum(0).cpu().numpy()
    assert_colsum_close(db, colsum, l1 * (2.0 ** -9) * 1e6, dtype)
    del y, out, go, dy
    rows, cols, p = 16384, 4096, 0.1
    x = torch.randn((rows, cols), generator=g, device=DEV, dtype=torch.float32).to(dtype)
    res = torch.randn((rows, cols), generator=g, device=DEV, dtype=torch.float32).to(dtype)
    b = b[:cols].contiguous()
    o = kernels.bias_dropout_add_forward(x, b, res, p, 1234, 0)
    keep = orc.dropout_keep_mask(1234, 0, rows * cols, p).reshape(rows, cols)
    band = slice(9000, 9008)
    assert_close(o[band], orc.bias_dropout_add_fwd(f32(x[band]), f32(b), f32(res[band]), p, keep[band]), dtype)
    dropped = torch.from_numpy(~keep).to(DEV)
    assert torch.equal(o[dropped], res[dropped])                # dropped elements are the residual, exactly
    dx, db = kernels.bias_dropout_add_backward(x, p, 1234, 0)
    assert torch.count_nonzero(dx[dropped]) == 0


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS.get)
@pytest.mark.parametrize("conv1d", [False, True], ids=["linear", "conv1d"])
def test_linear_bias_gelu_in_the_products_launch(dtype, conv1d):
    """FusedLinearBiasActivation (bias and GeLU applied by the matrix product
    itself, where autograd records nothing) against the float64 oracle of
    tanh-GeLU(x . W + b), beside product + bias-GeLU kernel on the same inputs:
    it is the tanh form (the error form differs from it by up to 2e-4 at
    these magnitudes) and, rounded once, it is at least as close."""
    from oslo_amd.fused_kernels_utils import FusedBiasActivation, FusedLinearBiasActivation

    m, k, n = 48, 256, 384
    x = randn((2, m // 2, k), dtype, seed=3)
    w = randn((n, k), dtype, seed=4, std=1.0 / 16)
    b = randn((n,), dtype, seed=5, std=0.5)
    want = orc.linear_rows(f32(x).reshape(m, k), f32(w), f32(b), gelu=True)
    weight = (w.t().contiguous() if conv1d else w).to(DEV)
    xd, bd = x.to(DEV), b.to(DEV)
    assert FusedLinearBiasActivation.is_available(xd, weight, bd, "gelu_new")
    out = FusedLinearBiasActivation.apply(xd, weight, bd, "gelu_new", conv1d=conv1d)
    assert out.shape == (2, m // 2, n) and out.dtype == dtype
    two = FusedBiasActivation.apply(xd @ (weight if conv1d else weight.t()), bd, "gelu_new")
    err = np.abs(f32(out).reshape(m, n).astype(np.float64) - want)
    err_two = np.abs(f32(two).reshape(m, n).astype(np.float64) - want)
    if dtype == torch.float32:
        assert err.max() <= 2e-5, err.max()      # fp32 sums of 256 products of magnitude up to 1
    else:
        assert_close(out.reshape(m, n), want, dtype, "linear + bias + gelu")
        assert err.mean() <= err_two.mean() * 1.02, (err.mean(), err_two.mean())
    # recorded by autograd: not available, the callers keep the kernel with its backward
    assert not FusedLinearBiasActivation.is_available(xd.requires_grad_(), weight, bd, "gelu_new")
    assert not FusedLinearBiasActivation.is_available(xd.detach(), weight, bd, "relu")
    assert not FusedLinearBiasActivation.is_available(xd.detach(), weight, None, "gelu_new")
