"""The attention of a decoding step (one query over a key/value cache), called
through the C ABI, against the CPU oracle in float64: fp32 <= 1e-6 absolute on
values of unit scale, fp16/bf16 <= 2e-3 relative to the largest value (one
rounding of an fp32 result)."""

import numpy as np
import pytest
import torch

from oracle import oslo_oracle as orc
from oslo_amd import kernels
from tests.util import DTYPES, IDS, f32, randn

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
TOL = {torch.float32: 2e-6, torch.float16: 2e-3, torch.bfloat16: 8e-3}


def run_case(b, h, cap, d, last, window, dtype, scale=0.25, pos_on_device=False):
    q = randn((b, h, 1, d), dtype, seed=d + last)
    k = randn((b, h, cap, d), dtype, seed=cap + 1)
    v = randn((b, h, cap, d), dtype, seed=cap + 2)
    pos = torch.tensor([last], dtype=torch.int64, device=DEV) if pos_on_device else last
    out = kernels.attention_decode_forward(q.to(DEV), k.to(DEV), v.to(DEV), pos, scale, window)
    assert out.shape == (b, h, 1, d) and out.dtype == dtype
    want = orc.attention_decode(f32(q).reshape(b * h, d), f32(k).reshape(b * h, cap, d),
                                f32(v).reshape(b * h, cap, d), last, scale, window)
    err = np.abs(f32(out).reshape(b * h, d).astype(np.float64) - want).max()
    assert err <= TOL[dtype] * max(1.0, np.abs(want).max()), (err, b, h, cap, d, last, window)


# head sizes of 128 / 256 / 512 / 1024 bytes in every dtype; caches shorter than one split, ragged,
# several splits; the query at the first, a middle and the last slot
@pytest.mark.parametrize("dtype", DTYPES, ids=IDS.get)
@pytest.mark.parametrize("d", [32, 64, 128, 256])
@pytest.mark.parametrize("cap,last", [(1, 0), (5, 4), (64, 0), (64, 63), (100, 37), (257, 256), (1152, 1023)])
def test_attention_decode_matches_oracle(cap, last, d, dtype):
    es = 4 if dtype == torch.float32 else 2
    if d * es not in (128, 256, 512, 1024):
        with pytest.raises(RuntimeError):
            run_case(1, 2, cap, d, last, 0, dtype)
        return
    run_case(2, 3, cap, d, last, 0, dtype)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS.get)
@pytest.mark.parametrize("window", [1, 3, 16, 64, 500])
def test_attention_decode_sliding_window_and_device_position(window, dtype):
    for last in (0, 10, 200, 299):
        run_case(1, 4, 300, 64, last, window, dtype, pos_on_device=(last % 2 == 0))


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS.get)
def test_attention_decode_many_heads_several_tiles_per_block(dtype):
    """With many heads a block walks several tiles of keys with a running
    maximum; the query early, in the middle of a tile, and at the end."""
    for last in (2, 150, 299):
        run_case(8, 64, 300, 64, last, 0, dtype)
    run_case(8, 64, 300, 64, 299, 100, dtype, pos_on_device=True)


def test_attention_decode_follows_a_device_position_and_large_scores():
    """The same launch arguments, another position in device memory; scores of
    several hundred (no overflow: the maximum is subtracted in fp32)."""
    dtype = torch.float16
    b, h, cap, d = 1, 2, 256, 128
    q = (randn((b, h, 1, d), dtype, seed=1) * 6).to(DEV)
    k = (randn((b, h, cap, d), dtype, seed=2) * 6).to(DEV)
    v = randn((b, h, cap, d), dtype, seed=3).to(DEV)
    pos = torch.zeros(1, dtype=torch.int64, device=DEV)
    for last in (3, 77, 255):
        pos.fill_(last)
        out = kernels.attention_decode_forward(q, k, v, pos, 1.0)
        want = orc.attention_decode(f32(q).reshape(h, d), f32(k).reshape(h, cap, d), f32(v).reshape(h, cap, d),
                                    last, 1.0)
        assert np.isfinite(f32(out)).all()
        assert np.abs(f32(out).reshape(h, d) - want).max() <= 2e-3 * max(1.0, np.abs(want).max())


def test_attention_decode_against_the_three_step_path():
    """matmul -> fused key-mask softmax -> matmul on the device, bf16 at the GPT-J head shape."""
    dtype = torch.bfloat16
    b, h, cap, d, last = 2, 16, 1152, 256, 1023
    q = randn((b, h, 1, d), dtype, seed=1).to(DEV)
    k = randn((b, h, cap, d), dtype, seed=2).to(DEV)
    v = randn((b, h, cap, d), dtype, seed=3).to(DEV)
    hidden = (torch.arange(cap, device=DEV) > last).view(1, 1, 1, cap)
    scores = torch.matmul(q, k.transpose(-1, -2))
    probs = kernels.masked_softmax_forward(scores, hidden, 1 / 16.0, kernels.MASK_ADD)
    want = torch.matmul(probs, v)
    out = kernels.attention_decode_forward(q, k, v, last, 1 / 16.0)
    assert (out.float() - want.float()).abs().max() <= 2e-2 * want.float().abs().max()


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS.get)
@pytest.mark.parametrize("cap,last,window", [(64, 0, 0), (100, 37, 0), (300, 299, 0), (300, 150, 16)])
def test_attention_decode_appends_the_new_key(cap, last, window, dtype):
    """The key and value of the query's position handed over outside the cache:
    same result, bit for bit, as with them in the cache, and afterwards they
    are in their slot and no other slot has changed."""
    b, h, d = 2, 3, 64
    q = randn((b, h, 1, d), dtype, seed=1).to(DEV)
    k = randn((b, h, cap, d), dtype, seed=2).to(DEV)
    v = randn((b, h, cap, d), dtype, seed=3).to(DEV)
    want = kernels.attention_decode_forward(q, k, v, last, 0.25, window)
    k2, v2 = k.clone(), v.clone()
    k2[:, :, last] = 7.0            # the slot holds something else until the kernel fills it
    v2[:, :, last] = -7.0
    pos = torch.tensor([last], dtype=torch.int64, device=DEV)
    got = kernels.attention_decode_forward(q, k2, v2, pos, 0.25, window,
                                           k[:, :, last:last + 1].contiguous(), v[:, :, last:last + 1].contiguous())
    assert torch.equal(got, want)
    assert torch.equal(k2, k) and torch.equal(v2, v)
    # the same from the slices of a packed q|k|v row per sequence (GPT-2's c_attn output)
    packed = torch.zeros((b, 1, 3 * h * d), dtype=dtype, device=DEV)
    packed[:, 0, h * d:2 * h * d] = k[:, :, last].reshape(b, h * d)
    packed[:, 0, 2 * h * d:] = v[:, :, last].reshape(b, h * d)
    nk = packed[:, :, h * d:2 * h * d].reshape(b, h, 1, d)
    nv = packed[:, :, 2 * h * d:].reshape(b, h, 1, d)
    assert not nk.is_contiguous()
    k3, v3 = k.clone(), v.clone()
    k3[:, :, last] = 7.0
    v3[:, :, last] = -7.0
    assert torch.equal(kernels.attention_decode_forward(q, k3, v3, pos, 0.25, window, nk, nv), want)
    assert torch.equal(k3, k) and torch.equal(v3, v)


def test_attention_decode_errors():
    q = torch.zeros(1, 2, 1, 64, device=DEV)
    kv = torch.zeros(1, 2, 16, 64, device=DEV)
    with pytest.raises(RuntimeError):
        kernels.attention_decode_forward(torch.zeros(1, 2, 2, 64, device=DEV), kv, kv, 3, 1.0)   # two queries
    with pytest.raises(RuntimeError):
        kernels.attention_decode_forward(q, kv, kv, 16, 1.0)                                       # past the cache
    with pytest.raises(RuntimeError):
        kernels.attention_decode_forward(q, kv, kv.half(), 3, 1.0)
    with pytest.raises(RuntimeError):
        kernels.attention_decode_forward(q, kv[:, :1], kv[:, :1], 3, 1.0)
    with pytest.raises(RuntimeError):
        kernels.attention_decode_forward(q.cpu(), kv.cpu(), kv.cpu(), 3, 1.0)
    with pytest.raises(RuntimeError):
        kernels.attention_decode_forward(q, kv, kv, torch.zeros(1, dtype=torch.int32, device=DEV), 1.0)
