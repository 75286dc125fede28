"""The benchmark configurations at their real shapes, checked rather than only
timed: the GPT-J-6B-shaped and GPT-2-small models fused against unfused (and
against the same weights in fp32), the fp32 causal softmax at [8,16,2048,2048],
bias-GeLU at [16384,4096] and bias-dropout(+residual) at [16384,16384] with its
bias gradient. Size-independent properties on the whole tensors, the oracle on
slabs and row bands."""

import copy

import numpy as np
import pytest
import torch

from oracle import oslo_oracle as orc
from oslo_amd import GPT2Config, GPT2LMHeadModel, GPTJConfig, GPTJForCausalLM, kernels
from tests.util import assert_close, assert_colsum_close, f32

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def test_gptj_6b_widths_fused_against_unfused_and_fp32():
    """GPT-J-6B's block (d_model 4096, 16 heads of 256, rotary 64, d_ff 16384,
    vocab 50400) at batch 8 x 2048 tokens in bf16, four layers. Fused and
    unfused bf16 logits are both compared with the unfused model run in fp32 on
    the same weights: the fused model must be no further from it than the
    unfused bf16 model is (their mutual difference is then rounding placement,
    not an error of the kernels)."""
    old = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        with torch.device(DEV):
            torch.manual_seed(0)
            model = GPTJForCausalLM(GPTJConfig(n_layer=4)).eval()
    finally:
        torch.set_default_dtype(old)
    ids = torch.randint(0, 50400, (8, 2048), device=DEV, generator=torch.Generator(device=DEV).manual_seed(0))
    with torch.no_grad():
        ref = copy.deepcopy(model).float()(ids)["logits"]
        unfused = model(ids)["logits"].float()
        model.fuse()
        fused = model(ids)["logits"].float()
    assert torch.isfinite(fused).all()
    err_u, err_f = (unfused - ref).abs(), (fused - ref).abs()
    mutual = (fused - unfused).abs().max().item()
    print(f"gptj widths: |logit| max {ref.abs().max().item():.3f}; unfused-fp32 max {err_u.max().item():.4f} "
          f"mean {err_u.mean().item():.5f}; fused-fp32 max {err_f.max().item():.4f} mean {err_f.mean().item():.5f}; "
          f"fused-unfused max {mutual:.4f}")
    assert err_f.mean().item() <= 1.05 * err_u.mean().item()
    assert err_f.max().item() <= 1.25 * err_u.max().item()
    # and the argmax token agrees with the fp32 model at least as often as the unfused bf16 model's
    top = ref.argmax(-1)
    assert (fused.argmax(-1) == top).float().mean().item() >= (unfused.argmax(-1) == top).float().mean().item() - 1e-3


def test_gpt2_small_fused_on_gpu_against_unfused_on_cpu():
    """GPT-2 small (12 layers, 768, 12 heads, vocab 50257), fp32, batch 4 x 512:
    the unfused model on the host against the same weights after fuse() on the
    GPU."""
    torch.manual_seed(0)
    model = GPT2LMHeadModel(GPT2Config()).eval()
    ids = torch.randint(0, 50257, (4, 512), generator=torch.Generator().manual_seed(0))
    with torch.no_grad():
        want = model(ids)["logits"]
        got = model.to(DEV).fuse()(ids.to(DEV))["logits"].cpu()
    assert torch.isfinite(got).all()
    err = (got - want).abs().max().item()
    assert err <= 2e-4, f"GPT-2 small fp32: fused GPU and unfused CPU logits differ by {err}"


def test_causal_fp32_full_size_properties():
    """fp32 [8,16,2048,2048]: zeros above the diagonal, row sums, determinism,
    the oracle on slabs; backward: zeros above the diagonal, rows of dx sum to
    zero against their own mass, the oracle on a slab, in place."""
    b, h, s = 8, 16, 2048
    g = torch.Generator(device=DEV).manual_seed(0)
    x = torch.randn((b, h, s, s), generator=g, device=DEV, dtype=torch.float32) * 8
    y = kernels.causal_softmax_forward(x, None, 0.125)
    assert torch.count_nonzero(torch.triu(y[::3, ::5], 1)) == 0
    assert float((y.sum(-1, dtype=torch.float64) - 1).abs().max()) <= 1e-5
    for bi, hi in [(0, 0), (5, 9), (7, 15)]:
        want = orc.softmax_causal(f32(x[bi:bi + 1, hi:hi + 1]), 0.125)
        assert_close(y[bi:bi + 1, hi:hi + 1], want, torch.float32, f"slab {bi},{hi}")
    assert torch.equal(y, kernels.causal_softmax_forward(x, None, 0.125))
    del x
    go = torch.randn((b * h, s, s), generator=g, device=DEV, dtype=torch.float32)
    yv = y.view(-1, s, s)
    want = orc.softmax_bwd(f32(go[101]), f32(yv[101]), 0.125, causal=True)
    go_slab = go[101].clone()
    dx = kernels.scaled_upper_triang_masked_softmax_backward(go, yv, 0.125)
    assert dx.data_ptr() == go.data_ptr()                        # the reference's contract: written over the gradient
    assert_close(dx[101], want, torch.float32, "bwd slab 101")
    assert torch.count_nonzero(torch.triu(dx[::9], 1)) == 0
    # sum_k dx = scale * (sum gy - sum y * sum gy) = 0 up to the rounding of the row's mass
    mass = (go_slab.tril().abs() * yv[101]).sum(-1, dtype=torch.float64)
    rowsum = dx.sum(-1, dtype=torch.float64)
    assert float(rowsum.abs().max()) <= 1e-4
    assert float((rowsum[101].abs() / (mass + 1e-3)).max()) <= 1e-5


def test_bias_gelu_16384x4096_forward_backward():
    dtype = torch.bfloat16
    rows, cols = 16384, 4096
    g = torch.Generator(device=DEV).manual_seed(0)
    y = torch.randn((rows, cols), generator=g, device=DEV, dtype=torch.float32).to(dtype)
    b = (torch.randn((cols,), generator=g, device=DEV, dtype=torch.float32) * 0.02).to(dtype)
    go = torch.randn((rows, cols), generator=g, device=DEV, dtype=torch.float32).to(dtype)
    out = kernels.bias_gelu_forward(y, b)
    dy, db = kernels.bias_gelu_backward(go, y, b)
    for r0 in (0, 4093, 16376):
        band = slice(r0, r0 + 8)
        assert_close(out[band], orc.bias_gelu_fwd(f32(y[band]), f32(b)), dtype, f"fwd rows {r0}")
        want_dy, _ = orc.bias_gelu_bwd(f32(go[band]), f32(y[band]), f32(b))
        assert_close(dy[band], want_dy, dtype, f"bwd rows {r0}")
    assert torch.equal(out, kernels.bias_gelu_forward(y, b))
    # dbias from the unrounded products: the float64 expression on the device
    x64 = y.double() + b.double()
    t = torch.tanh(0.79788456 * x64 * (1 + 0.044715 * x64 * x64))
    ff = 0.5 * x64 * ((1 - t * t) * (0.79788456 + 0.1070322243 * x64 * x64)) + 0.5 * (1 + t)
    prod = ff * go.double()
    assert_colsum_close(db, prod.sum(0).cpu().numpy(), prod.abs().sum(0).cpu().numpy(), dtype)
    dy2, db2 = kernels.bias_gelu_backward(go, y, b)
    assert torch.equal(db, db2) and torch.equal(dy, dy2)             # deterministic


def test_bias_dropout_residual_16384x16384_forward_backward():
    dtype = torch.bfloat16
    rows, cols, p, seed, offset = 16384, 16384, 0.1, 1234, 0
    g = torch.Generator(device=DEV).manual_seed(0)
    x = torch.randn((rows, cols), generator=g, device=DEV, dtype=torch.float32).to(dtype)
    res = torch.randn((rows, cols), generator=g, device=DEV, dtype=torch.float32).to(dtype)
    b = (torch.randn((cols,), generator=g, device=DEV, dtype=torch.float32) * 0.02).to(dtype)
    go = torch.randn((rows, cols), generator=g, device=DEV, dtype=torch.float32).to(dtype)
    out = kernels.bias_dropout_add_forward(x, b, res, p, seed, offset)
    dx, db = kernels.bias_dropout_add_backward(go, p, seed, offset)
    for r0 in (0, 8191, 16376):
        r0 -= r0 % 8
        band = slice(r0, r0 + 8)
        keep = orc.dropout_keep_mask(seed, offset, 8 * cols, p, start=r0 * cols).reshape(8, cols)
        assert_close(out[band], orc.bias_dropout_add_fwd(f32(x[band]), f32(b), f32(res[band]), p, keep), dtype,
                     f"fwd rows {r0}")
        want_dx, _, _ = orc.bias_dropout_add_bwd(f32(go[band]), p, keep)
        assert_close(dx[band], want_dx, dtype, f"bwd rows {r0}")
        dropped = torch.from_numpy(~keep).to(DEV)
        assert torch.equal(out[band][dropped], res[band][dropped])   # a dropped element is the residual, exactly
        assert torch.count_nonzero(dx[band][dropped]) == 0
    # the mask of the whole tensor, read off a forward over ones: forward and backward used it everywhere
    mask = kernels.bias_dropout_add_forward(torch.ones_like(x), None, None, p, seed, offset) != 0
    rate = mask.double().mean().item()
    assert abs(rate - (1 - p)) < 4 * (p * (1 - p) / (rows * cols)) ** 0.5
    assert torch.equal(torch.where(mask, res, out), res)             # dropped elements are the residual, exactly
    assert torch.equal(dx != 0, mask & (go != 0))
    # dbias: the unrounded products are g / (1 - p) where kept; the mask is read off dx
    scale = 1.0 / (1.0 - float(np.float32(p)))
    prod = torch.where(mask, go.double() * scale, torch.zeros((), dtype=torch.float64, device=DEV))
    assert_colsum_close(db, prod.sum(0).cpu().numpy(), prod.abs().sum(0).cpu().numpy(), dtype)
    dx2, db2 = kernels.bias_dropout_add_backward(go, p, seed, offset)
    assert torch.equal(db, db2) and torch.equal(dx, dx2)
