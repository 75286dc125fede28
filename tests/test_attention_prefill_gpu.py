"""Causal attention over a whole prompt in one kernel, called through the C
ABI, against the CPU oracle in float64 (small cases) and against the same
formula in float64 on the device (large ones). Tolerance: the result is an fp32
sum rounded once to the storage type (at most REL * |ref|, REL = 2^-8 for bf16,
2^-11 for fp16), and the probabilities are rounded to the storage type before
they multiply the values, as the unfused path casts them (at most REL * max|v|
over a row, whose probabilities sum to one):
|err| <= REL * (|ref| + max|v|) + 1e-4."""

import math

import numpy as np
import pytest
import torch

from oracle import oslo_oracle as orc
from oslo_amd import FusedMergeHeads, FusedPrefillAttention, kernels
from tests.util import IDS, f32, randn

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
HALVES = [torch.float16, torch.bfloat16]
REL = {torch.float16: 2.0 ** -11, torch.bfloat16: 2.0 ** -8}


def device_reference(q, k, v, scale, pad=None, window=0):
    q, k, v = q.double(), k.double(), v.double()
    s = q.shape[2]
    w = q @ k.transpose(-1, -2) * scale
    if pad is not None:
        w = w + pad.double()[:, None, None, :]
    i = torch.arange(s, device=q.device)
    hidden = i[None, :] > i[:, None]
    if window:
        hidden = hidden | (i[None, :] <= i[:, None] - window)
    return torch.softmax(w.masked_fill(hidden, float("-inf")), -1) @ v


def check(out, want, dtype, what, vmax=4.0):
    """``vmax``: the largest value magnitude (4.0 covers the unit-normal inputs here)."""
    out, want = out.double(), want.double() if isinstance(want, torch.Tensor) else torch.from_numpy(want).to(out.device)
    excess = ((out - want).abs() - REL[dtype] * (want.abs() + vmax)).max().item()
    assert excess <= 1e-4, (excess, what)


def padding(b, s, seed):
    g = torch.Generator().manual_seed(seed)
    lens = torch.randint(max(1, s // 2), s + 1, (b,), generator=g)
    return torch.where(torch.arange(s)[None, :] < lens[:, None], 0.0, -10000.0).float()


# prompts shorter than a key tile, ragged against the 64-key tiles and the 128-query blocks, several blocks
@pytest.mark.parametrize("dtype", HALVES, ids=IDS.get)
@pytest.mark.parametrize("d", [64, 128, 256])
@pytest.mark.parametrize("s", [1, 8, 63, 64, 65, 128, 200, 332])
def test_prefill_matches_oracle(s, d, dtype):
    b, h = 2, 3
    q, k, v = (randn((b, h, s, d), dtype, seed=7 * s + i) for i in range(3))
    scale = 1.0 / math.sqrt(d)
    out = kernels.attention_prefill_forward(q.to(DEV), k.to(DEV), v.to(DEV), scale)
    assert out.shape == (b, h, s, d) and out.dtype == dtype
    assert out.permute(0, 2, 1, 3).is_contiguous()  # merged-heads memory
    want = orc.attention_prefill(f32(q).reshape(b * h, s, d), f32(k).reshape(b * h, s, d),
                                 f32(v).reshape(b * h, s, d), scale).reshape(b, h, s, d)
    check(out, want, dtype, (s, d))
    if s % 4 == 0:
        pad = padding(b, s, s)
        out = kernels.attention_prefill_forward(q.to(DEV), k.to(DEV), v.to(DEV), scale, pad.to(DEV))
        want = orc.attention_prefill(f32(q).reshape(b * h, s, d), f32(k).reshape(b * h, s, d),
                                     f32(v).reshape(b * h, s, d), scale,
                                     pad.numpy().repeat(h, axis=0)).reshape(b, h, s, d)
        check(out, want, dtype, (s, d, "pad"))


@pytest.mark.parametrize("dtype", HALVES, ids=IDS.get)
@pytest.mark.parametrize("b,h,s,d", [(2, 16, 1024, 64), (1, 9, 1000, 128), (2, 4, 2048, 256), (1, 2, 4100, 128)])
def test_prefill_long_prompts(b, h, s, d, dtype):
    q, k, v = (randn((b, h, s, d), dtype, seed=s + i).to(DEV) for i in range(3))
    pad = padding(b, s, 3).to(DEV)
    for p in (None, pad):
        out = kernels.attention_prefill_forward(q, k, v, 0.1, p)
        check(out, device_reference(q, k, v, 0.1, p), dtype, (b, h, s, d, p is not None))


# windows shorter than a step of 32 keys, ragged against steps and tiles, longer than a query block,
# and at least the prompt (no window at all)
@pytest.mark.parametrize("dtype", HALVES, ids=IDS.get)
@pytest.mark.parametrize("window", [1, 5, 32, 33, 64, 100, 256, 300, 700])
def test_prefill_sliding_window(window, dtype):
    for (b, h, s, d) in ((2, 3, 520, 64), (1, 2, 700, 256)):
        q, k, v = (randn((b, h, s, d), dtype, seed=window + i).to(DEV) for i in range(3))
        pad = padding(b, s, window).to(DEV)
        for p in (None, pad):
            out = kernels.attention_prefill_forward(q, k, v, 0.1, p, window)
            check(out, device_reference(q, k, v, 0.1, p, window), dtype, (b, h, s, d, window, p is not None))
    # small enough for the oracle: its causal softmax with a window, composed with a matmul
    b, h, s, d = 1, 2, 96, 64
    q, k, v = (randn((b, h, s, d), dtype, seed=3 * window + i) for i in range(3))
    scores = np.einsum("bhid,bhjd->bhij", f32(q).astype(np.float64), f32(k).astype(np.float64))
    probs = orc.softmax_causal(scores, 0.1, dtype=np.float64, window=window)
    want = np.einsum("bhij,bhjd->bhid", probs, f32(v).astype(np.float64))
    out = kernels.attention_prefill_forward(q.to(DEV), k.to(DEV), v.to(DEV), 0.1, None, window)
    check(out, want, dtype, ("oracle", window))


@pytest.mark.parametrize("dtype", HALVES, ids=IDS.get)
def test_prefill_large_scores_and_size_independent_properties(dtype):
    """Scores of several hundred (the maximum is subtracted in fp32: nothing
    overflows); row 0 is the first value; equal scores give the running mean
    of the values; the output is linear in the values."""
    b, h, s, d = 1, 4, 512, 128
    q, k, v = (randn((b, h, s, d), dtype, seed=20 + i).to(DEV) for i in range(3))
    out = kernels.attention_prefill_forward(q * 6, k * 6, v, 1.0)
    assert torch.isfinite(out).all()
    check(out, device_reference(q * 6, k * 6, v, 1.0), dtype, "large scores")
    assert torch.equal(out[:, :, 0], v[:, :, 0])
    flat = kernels.attention_prefill_forward(torch.zeros_like(q), k, v, 1.0)
    mean = v.double().cumsum(2) / torch.arange(1, s + 1, device=DEV)[None, None, :, None]
    check(flat, mean, dtype, "running mean")
    two = kernels.attention_prefill_forward(q, k, v * 2, 0.1)
    one = kernels.attention_prefill_forward(q, k, v, 0.1)
    if dtype == torch.bfloat16:
        assert torch.equal(two, one * 2)  # a power of two: exact
    else:  # fp16 values under 2^-14 are subnormal and their doubles are not: equal to an ulp
        assert torch.allclose(two.float(), one.float() * 2, rtol=2.0 ** -10, atol=1e-6)


@pytest.mark.parametrize("dtype", HALVES, ids=IDS.get)
@pytest.mark.parametrize("d", [64, 128, 256])
def test_prefill_scores_that_keep_rising(d, dtype):
    """Every tile of keys scores far above the ones before it (by 46 in log2
    units per tile, the slack of the reference maximum being 8), so that O is
    rescaled in every tile; then scores that fall (nothing is ever rescaled
    after the first tile), and a rise only at the very end."""
    b, h, s = 1, 2, 700
    pos = torch.arange(s, dtype=torch.float32)
    v = randn((b, h, s, d), dtype, seed=d).to(DEV)
    q = torch.full((b, h, s, d), 0.25).to(dtype).to(DEV)
    for slope in (lambda j: j / 64.0, lambda j: -j / 64.0, lambda j: (j >= s - 3).float() * 40.0):
        k = (slope(pos)[None, None, :, None] * torch.ones(d) * (8.0 / d)).to(dtype).to(DEV)  # q.k = 2 * slope
        k = k.expand(b, h, s, d).contiguous()
        out = kernels.attention_prefill_forward(q, k, v, 16.0)
        assert torch.isfinite(out).all()
        check(out, device_reference(q, k, v, 16.0), dtype, ("slope", d))


@pytest.mark.parametrize("dtype", HALVES, ids=IDS.get)
@pytest.mark.parametrize("d", [64, 128, 256])
def test_prefill_isolated_large_scores(d, dtype):
    """A few queries score far above their running maximum at a few scattered
    keys, the others never: the reference maximum has to rise for single lanes
    of single waves in the middle of a block (where the tiles otherwise run
    without looking at the maxima), with and without a padding mask."""
    b, h, s = 2, 3, 900
    q, k, v = (randn((b, h, s, d), dtype, seed=7 * d + i) for i in range(3))
    q, k = q * 0.5, k * 0.5
    rows = torch.arange(s)[torch.arange(s) % 37 == 5]
    q[:, :, rows] += 3.0
    for j, key in enumerate((70, 200, 333, 515, 640, 801)):
        k[:, (j % h):, key] += 1.0 + j  # q.k rises by 3 (1 + j) d, times the scale
    q, k, v = q.to(DEV), k.to(DEV), v.to(DEV)
    pad = padding(b, s, d).to(DEV)
    for p in (None, pad):
        out = kernels.attention_prefill_forward(q, k, v, d ** -0.5, p)
        assert torch.isfinite(out).all()
        check(out, device_reference(q, k, v, d ** -0.5, p), dtype, ("isolated", d, p is not None), vmax=5.0)


def test_prefill_full_size_properties():
    """The GPT-J shape of the benchmark, [8, 16, 2048, 256] bf16, where the oracle
    would take hours: the first row is the first value exactly, equal scores
    (q = 0) give the running mean of the values, and the result agrees with the
    library's attention (an independent implementation) within the bound for two
    bf16 results."""
    dtype = torch.bfloat16
    b, h, s, d = 8, 16, 2048, 256
    g = torch.Generator(device=DEV).manual_seed(0)
    q, k, v = (torch.randn((b, h, s, d), generator=g, device=DEV).to(dtype) for _ in range(3))
    out = kernels.attention_prefill_forward(q, k, v, d ** -0.5)
    assert torch.isfinite(out).all()
    assert torch.equal(out[:, :, 0], v[:, :, 0])
    lib = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True)
    excess = ((out.float() - lib.float()).abs() - 2 * REL[dtype] * (lib.float().abs() + 4.0)).max().item()
    assert excess <= 1e-4, excess
    flat = kernels.attention_prefill_forward(torch.zeros_like(q), k, v, 1.0)
    for bb in range(0, b, 3):  # in slices: float64 of the whole tensor is 1 GiB
        mean = v[bb].double().cumsum(1) / torch.arange(1, s + 1, device=DEV)[None, :, None]
        check(flat[bb], mean, dtype, "running mean", vmax=6.0)


@pytest.mark.parametrize("dtype", HALVES, ids=IDS.get)
def test_prefill_takes_strided_views(dtype):
    """Merged-heads memory ([B, S, H, D] viewed as [B, H, S, D]) and the slices of
    a packed q|k|v projection are read where they lie."""
    b, h, s, d = 2, 4, 160, 64
    packed = randn((b, s, 3 * h * d), dtype, seed=5).to(DEV)
    q, k, v = (packed[:, :, i * h * d:(i + 1) * h * d].view(b, s, h, d).permute(0, 2, 1, 3) for i in range(3))
    assert not q.is_contiguous()
    out = kernels.attention_prefill_forward(q, k, v, 0.125)
    want = kernels.attention_prefill_forward(q.contiguous(), k.contiguous(), v.contiguous(), 0.125)
    assert torch.equal(out, want)
    check(out, device_reference(q, k, v, 0.125), dtype, "strided")
    merged = FusedMergeHeads.apply(out)
    assert merged.shape == (b, s, h * d) and merged.data_ptr() == out.data_ptr()  # no copy
    assert torch.equal(merged, out.permute(0, 2, 1, 3).reshape(b, s, h * d))


def test_prefill_operator_gate_and_errors():
    q = randn((1, 2, 256, 64), torch.float16, seed=1).to(DEV)
    mask = padding(1, 256, 1).to(DEV).view(1, 1, 1, 256).half()
    assert FusedPrefillAttention.is_available(q, q)
    assert FusedPrefillAttention.is_available(q, q, mask)
    assert FusedPrefillAttention.is_available(q, q, training=True, dropout_p=0.1)       # dropout inside the kernel
    assert not FusedPrefillAttention.is_available(q[:, :, :250], q[:, :, :250], training=True, dropout_p=0.1)  # S % 8
    assert not FusedPrefillAttention.is_available(q.float(), q.float())
    assert FusedPrefillAttention.is_available(q[:, :, :5], q[:, :, :5])            # short prompts too
    assert not FusedPrefillAttention.is_available(q[:, :, :1], q[:, :, :1])        # one query: a decoding step
    assert not FusedPrefillAttention.is_available(q[:, :, :128], q)                # a cache longer than the prompt
    assert not FusedPrefillAttention.is_available(q[..., :32], q[..., :32])        # head size
    assert FusedPrefillAttention.is_available(q.clone().requires_grad_(), q)             # it has a backward
    out = FusedPrefillAttention.apply(q, q, q, mask, 0.125)
    check(out, device_reference(q, q, q, 0.125, mask.view(1, 256).float()), torch.float16, "operator")
    with pytest.raises(RuntimeError):
        kernels.attention_prefill_forward(q.float(), q.float(), q.float(), 1.0)
    with pytest.raises(RuntimeError):
        kernels.attention_prefill_forward(q[..., :32], q[..., :32], q[..., :32], 1.0)
    with pytest.raises(RuntimeError):
        kernels.attention_prefill_forward(q, q[:, :, :128], q, 1.0)
    with pytest.raises(RuntimeError):
        kernels.attention_prefill_forward(q[:, :, :254], q[:, :, :254], q[:, :, :254], 1.0,
                                          torch.zeros(1, 254, device=DEV))
    empty = kernels.attention_prefill_forward(q[:0], q[:0], q[:0], 1.0)
    assert empty.shape == (0, 2, 256, 64)
