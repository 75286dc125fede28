"""Score tensors of 2^31 elements and more. The softmax entry points index
elements with 64 bits; what a launch is limited by is the number of rows
(batch * heads * S < 2^31), so [32,16,2048,2048] (2^31 elements) and
[4,16,8192,8192] (2^32) are single calls. The reference launches any number of
attention batches (oslo/fused_kernels/fused_triang_softmax.cu:44-60).
Size-independent properties on the whole tensors, the oracle on the first slab
and on slabs that lie wholly behind element 2^31 (and 2^32 - one slab)."""

import numpy as np
import pytest
import torch

from oracle import oslo_oracle as orc
from oslo_amd import FusedScaleMaskSoftmax, kernels
from tests.util import assert_close, f32

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _slab_checks(y, x, scale, slabs, dtype):
    for bi, hi in slabs:
        want = orc.softmax_causal(f32(x[bi:bi + 1, hi:hi + 1]), scale)
        assert_close(y[bi:bi + 1, hi:hi + 1], want, dtype, f"slab {bi},{hi}")


def test_causal_bf16_4x16x8192x8192():
    dtype = torch.bfloat16
    b, h, s = 4, 16, 8192
    assert b * h * s * s == 2 ** 32
    assert FusedScaleMaskSoftmax.is_available(dtype, b, h, s, s, True)
    g = torch.Generator(device=DEV).manual_seed(0)
    x = torch.randn((b, h, s, s), generator=g, device=DEV, dtype=dtype)
    y = FusedScaleMaskSoftmax.apply(x, None, 1.0 / 16, True)
    for bi in range(b):  # properties head by head: a slab in fp64 is 512 MiB
        for hi in range(bi % 3, h, 5):
            assert torch.count_nonzero(torch.triu(y[bi, hi], 1)) == 0
            sums = y[bi, hi].sum(-1, dtype=torch.float64)
            assert float((sums - 1).abs().max()) <= 1e-3 + 2.0 ** -9 * 2  # plus the half-ulps of the stored row
    _slab_checks(y, x, 1.0 / 16, [(0, 0), (2, 0), (3, 15)], dtype)  # (2, 0) starts at element 2^31
    # backward over the same tensor, in place over the gradient
    go = torch.randn((b * h, s, s), generator=g, device=DEV, dtype=dtype)
    last = go[-1].clone()
    want = orc.softmax_bwd(f32(last), f32(y[3, 15]), 1.0 / 16, causal=True)
    dx = kernels.scaled_upper_triang_masked_softmax_backward(go, y.view(-1, s, s), 1.0 / 16)
    assert dx.data_ptr() == go.data_ptr()
    assert_close(dx[-1], want, dtype, "bwd last slab")
    for i in range(0, b * h, 5):
        assert torch.count_nonzero(torch.triu(dx[i], 1)) == 0


def test_causal_fp16_32x16x2048x2048_with_padding_mask():
    dtype = torch.float16
    b, h, s = 32, 16, 2048
    assert b * h * s * s == 2 ** 31
    g = torch.Generator(device=DEV).manual_seed(1)
    x = torch.randn((b, h, s, s), generator=g, device=DEV, dtype=dtype) * 8
    lens = torch.randint(s // 2, s + 1, (b,), generator=torch.Generator().manual_seed(2))
    pad = torch.where(torch.arange(s)[None, :] < lens[:, None], 0.0, -10000.0).view(b, 1, 1, s)
    y = FusedScaleMaskSoftmax.apply(x, pad.to(DEV), 0.125, True)
    assert torch.count_nonzero(torch.triu(y[::5, ::3], 1)) == 0
    assert float((y[::3].sum(-1, dtype=torch.float32) - 1).abs().max()) <= 1e-3
    for bi, hi in [(0, 0), (16, 0), (31, 15)]:
        want = orc.softmax_causal(f32(x[bi:bi + 1, hi:hi + 1]), 0.125, pad[bi:bi + 1].view(1, s).numpy())
        assert_close(y[bi:bi + 1, hi:hi + 1], want, dtype, f"slab {bi},{hi}")


def test_key_mask_bf16_64x16x2048x1024():
    dtype = torch.bfloat16
    b, h, sq, sk = 64, 16, 2048, 1024
    assert b * h * sq * sk == 2 ** 31
    g = torch.Generator(device=DEV).manual_seed(3)
    x = torch.randn((b, h, sq, sk), generator=g, device=DEV, dtype=dtype) * 3
    lens = torch.randint(128, sk + 1, (b,), generator=torch.Generator().manual_seed(4))
    mask = (torch.arange(sk)[None, :] >= lens[:, None]).view(b, 1, 1, sk)
    y = FusedScaleMaskSoftmax.apply(x, mask.to(DEV), 0.125, False)
    assert float((y[::7].sum(-1, dtype=torch.float32) - 1).abs().max()) <= 1e-3 + 2.0 ** -9 * 2
    for bi, hi in [(0, 0), (32, 0), (63, 15)]:
        want = orc.softmax_masked(f32(x[bi:bi + 1, hi:hi + 1]), mask[bi:bi + 1].numpy(), 0.125, "add")
        assert_close(y[bi:bi + 1, hi:hi + 1], want, dtype, f"slab {bi},{hi}")
        assert torch.count_nonzero(y[bi, hi, :, int(lens[bi]):]) == 0
    go = torch.randn((b, h, sq, sk), generator=g, device=DEV, dtype=dtype)
    want = orc.softmax_bwd(f32(go[63, 15]), f32(y[63, 15]), 0.125)
    dx = kernels.scaled_masked_softmax_backward(go, y, 0.125)
    assert_close(dx[63, 15], want, dtype, "bwd last slab")
    assert np.isfinite(f32(dx[::9, ::5])).all()
