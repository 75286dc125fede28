"""oslo_rotary_qkv through the C ABI against the numpy oracle: the kernel does
the oracle's fp32 operations on the same tables, so results are compared bit
for bit (after the one rounding to the storage type)."""

import numpy as np
import pytest
import torch

from oracle import oslo_oracle as orc

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [torch.float32, torch.float16, torch.bfloat16]
IDS = {torch.float32: "fp32", torch.float16: "fp16", torch.bfloat16: "bf16"}


def rounded(a, dtype):
    """fp32 numpy array rounded to dtype (RNE), back as fp32 numpy."""
    return torch.from_numpy(np.ascontiguousarray(a)).to(dtype).float().numpy()


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS.get)
@pytest.mark.parametrize("shape", [
    # B, S, H, D, rotary_dim, offset
    (2, 37, 3, 64, 16, 0),
    (1, 5, 2, 8, 8, 3),          # one vector per head row (16-bit), full rotary
    (2, 130, 4, 256, 64, 0),     # GPT-J head
    (1, 9, 5, 96, 32, 7),        # lanes per row not a power of two
    (3, 16, 2, 32, 0, 0),        # nothing to rotate: transposition only
    (1, 64, 16, 128, 128, 100),
    (1, 3, 1, 16, 6, 0),         # rotary_dim not a multiple of the vector
])
def test_forward_and_inverse_match_the_oracle(shape, dtype):
    from oslo_amd import kernels

    b, s, h, d, rot, off = shape
    g = torch.Generator().manual_seed(sum(shape))
    q, k, v = (torch.randn(b, s, h, d, generator=g).to(dtype) for _ in range(3))
    sin, cos = orc.rotary_tables(max(rot, 2), s + off)
    sin_d, cos_d = torch.from_numpy(sin).to(DEV), torch.from_numpy(cos).to(DEV)
    if rot == 0:
        sin_d = cos_d = None
    qo, ko, vo = kernels.rotary_qkv_forward(q.to(DEV), k.to(DEV), v.to(DEV), sin_d, cos_d, rot, off)
    for got, x, rotate in ((qo, q, True), (ko, k, True), (vo, v, False)):
        want = orc.rotary_split_heads(x.float().numpy(), sin, cos, rot, offset=off, rotate=rotate)
        assert got.shape == (b, h, s, d) and got.is_contiguous()
        assert np.array_equal(got.float().cpu().numpy(), rounded(want, dtype)), "forward"
    # the inverse (backward) map on fresh gradients
    gq, gk, gv = (torch.randn(b, h, s, d, generator=g).to(dtype) for _ in range(3))
    dq, dk, dv = kernels.rotary_qkv_backward(gq.to(DEV), gk.to(DEV), gv.to(DEV), sin_d, cos_d, rot, off)
    for got, x, rotate in ((dq, gq, True), (dk, gk, True), (dv, gv, False)):
        want = orc.rotary_split_heads(x.float().numpy(), sin, cos, rot, offset=off, rotate=rotate, inverse=True)
        assert got.shape == (b, s, h, d)
        assert np.array_equal(got.float().cpu().numpy(), rounded(want, dtype)), "inverse"
    # a subset of the tensors
    only_k = kernels.rotary_qkv_forward(None, k.to(DEV), None, sin_d, cos_d, rot, off)
    assert only_k[0] is None and only_k[2] is None and torch.equal(only_k[1], ko)


def test_full_size_gptj_shape_properties():
    """[8, 2048, 16, 256] bf16, rotary 64: pass-through features and v are moved
    bit for bit, pair norms are preserved, a sampled slab matches the oracle."""
    from oslo_amd import kernels

    b, s, h, d, rot = 8, 2048, 16, 256, 64
    gen = torch.Generator(device=DEV).manual_seed(0)
    q = torch.randn(b, s, h, d, generator=gen, device=DEV).to(torch.bfloat16)
    v = torch.randn(b, s, h, d, generator=gen, device=DEV).to(torch.bfloat16)
    sin, cos = orc.rotary_tables(rot, s)
    qo, _, vo = kernels.rotary_qkv_forward(q, None, v, torch.from_numpy(sin).to(DEV),
                                           torch.from_numpy(cos).to(DEV), rot, 0)
    assert torch.equal(vo, v.permute(0, 2, 1, 3))
    assert torch.equal(qo[..., rot:], q.permute(0, 2, 1, 3)[..., rot:])
    n_in = torch.hypot(q[..., 0:rot:2].float(), q[..., 1:rot:2].float()).permute(0, 2, 1, 3)
    n_out = torch.hypot(qo[..., 0:rot:2].float(), qo[..., 1:rot:2].float())
    assert (n_out - n_in).abs().max().item() <= 2.0 ** -7 * n_in.max().item()
    for bi, hi in ((0, 0), (7, 15), (3, 8)):
        want = orc.rotary_split_heads(q[bi:bi + 1, :, hi:hi + 1].float().cpu().numpy(), sin, cos, rot)
        assert np.array_equal(qo[bi, hi].float().cpu().numpy(), rounded(want, torch.bfloat16)[0, 0])


def test_operator_autograd_matches_the_unfused_torch_path():
    from oslo_amd import FusedRotaryPositionEmbedding
    from oslo_amd.modeling_gptj import apply_rotary, rotary_tables

    torch.manual_seed(1)
    b, s, h, d, rot, off = 2, 33, 4, 64, 32, 2
    q, k, v = (torch.randn(b, s, h, d, device=DEV, requires_grad=True) for _ in range(3))
    sincos = rotary_tables(rot, s + off, DEV)
    outs = FusedRotaryPositionEmbedding.apply(q, k, v, sincos, rot, off)

    def unfused(x, rotate):
        if rotate:
            x = torch.cat([apply_rotary(x[..., :rot], *sincos, off), x[..., rot:]], dim=-1)
        return x.permute(0, 2, 1, 3)

    wants = (unfused(q, True), unfused(k, True), unfused(v, False))
    gos = [torch.randn(b, h, s, d, device=DEV) for _ in range(3)]
    for got, want in zip(outs, wants):
        assert torch.equal(got, want)
    grads = torch.autograd.grad(outs, (q, k, v), gos)
    grads_want = torch.autograd.grad(wants, (q, k, v), gos)
    for got, want in zip(grads, grads_want):
        assert (got - want).abs().max().item() <= 1e-6


def test_argument_errors():
    from oslo_amd import kernels

    x = torch.randn(1, 4, 2, 16, device=DEV)
    sin = torch.zeros(4, 4, device=DEV)
    with pytest.raises(RuntimeError, match="rotary_dim"):
        kernels.rotary_qkv_forward(x, None, None, torch.zeros(4, 1, device=DEV), torch.zeros(4, 1, device=DEV), 3)
    with pytest.raises(RuntimeError, match="exceed the table"):
        kernels.rotary_qkv_forward(x, None, None, sin, sin, 8, offset=1)
    with pytest.raises(RuntimeError, match="head_dim"):
        kernels.rotary_qkv_forward(torch.randn(1, 4, 2, 6, device=DEV), None, None, sin[:, :1], sin[:, :1], 2)
    with pytest.raises(RuntimeError, match="no CPU path"):
        kernels.rotary_qkv_forward(x.cpu(), None, None, sin, sin, 8)


def test_merge_heads_operator():
    from oslo_amd import FusedMergeHeads

    torch.manual_seed(4)
    x = torch.randn(2, 3, 17, 32, device=DEV, dtype=torch.bfloat16, requires_grad=True)
    got = FusedMergeHeads.apply(x)
    want = x.permute(0, 2, 1, 3).contiguous().view(2, 17, 96)
    assert got.is_contiguous() and torch.equal(got, want)
    go = torch.randn_like(want)
    (gx,) = torch.autograd.grad(got, x, go)
    (gw,) = torch.autograd.grad(want, x, go)
    assert torch.equal(gx, gw)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS.get)
def test_split_heads_of_a_packed_projection(dtype):
    """GPT-2's c_attn output [B, S, 3E]: the three slices are read in place
    (row stride 3E) and come out as [B, H, S, D]; the backward writes the three
    gradients back into one [B, S, 3E] tensor."""
    from oslo_amd import FusedSplitHeads

    torch.manual_seed(6)
    b, s, h, d = 2, 19, 3, 16
    e = h * d
    qkv = torch.randn(b, s, 3 * e, device=DEV).to(dtype).requires_grad_(True)
    outs = FusedSplitHeads.apply(qkv, h)
    wants = [t.view(b, s, h, d).permute(0, 2, 1, 3) for t in qkv.split(e, dim=2)]
    for got, want in zip(outs, wants):
        assert got.is_contiguous() and torch.equal(got, want)
    gos = [torch.randn(b, h, s, d, device=DEV).to(dtype) for _ in range(3)]
    (g_got,) = torch.autograd.grad(outs, qkv, gos)
    (g_want,) = torch.autograd.grad(wants, qkv, gos)
    assert torch.equal(g_got, g_want)
