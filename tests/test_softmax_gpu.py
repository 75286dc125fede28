"""Parity of the HIP softmax kernels, called through the C ABI, with the CPU
oracle on the same seeded inputs. Bars: fp32 max abs error <= 1e-6; fp16/bf16
<= 2e-3 against the fp32 oracle; row sums within 1e-3 of 1."""

import ctypes

import numpy as np
import pytest
import torch

from oracle import oslo_oracle as orc
from oslo_amd import _lib, kernels
from tests.util import DTYPES, IDS, assert_close, bf16_half_ulps, f32, randn

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
# row lengths around every vector / wave / tile edge of the kernels
SIZES = [1, 2, 3, 4, 5, 8, 63, 64, 65, 127, 128, 129, 256, 504, 512, 520, 1000, 1024, 1032, 2040, 2047, 2048]
LONG = [2056, 4096, 5000, 8192]


def check_rowsums(y, dtype, want):
    """Row sums within 1e-3 of 1 (1e-5 for fp32). bf16 keeps 8 significant
    bits, so storing a row can by itself move its sum by the half-ulps of its
    entries (2^-9 for a single entry above 0.5): that much is added to the bar
    for bf16, computed from the oracle's row."""
    s = f32(y).astype(np.float64).sum(-1)
    bar = {torch.float32: 1e-5, torch.float16: 1e-3, torch.bfloat16: 1e-3}[dtype]
    if dtype == torch.bfloat16:
        bar = bar + bf16_half_ulps(want)
    assert (np.abs(s - 1.0) <= bar).all(), float(np.abs(s - 1.0).max())


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS.get)
@pytest.mark.parametrize("s", SIZES + LONG)
@pytest.mark.parametrize("with_pad", [False, True], ids=["nopad", "pad"])
def test_causal_forward(s, dtype, with_pad):
    b, h = (2, 3) if s <= 2048 else (1, 1)
    x = randn((b, h, s, s), dtype, seed=s, std=8.0)
    pad = None
    if with_pad:  # right padding: the tail keys of each sample are masked
        lens = torch.randint(1, s + 1, (b,), generator=torch.Generator().manual_seed(2))
        pad = torch.where(torch.arange(s)[None, :] < lens[:, None], 0.0, -10000.0).float()
    want = orc.softmax_causal(f32(x), 0.125, None if pad is None else pad.numpy())
    y = kernels.causal_softmax_forward(x.to(DEV), None if pad is None else pad.to(DEV), 0.125)
    assert y.dtype == dtype and y.shape == x.shape
    assert_close(y, want, dtype, f"causal fwd S={s}")
    assert torch.count_nonzero(torch.triu(y, 1)) == 0       # exactly zero above the diagonal
    assert torch.all(y[:, :, 0, 0] == 1)                     # row 0 is [1, 0, ...]
    check_rowsums(y, dtype, want)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS.get)
@pytest.mark.parametrize("s", SIZES + LONG)
def test_causal_backward(s, dtype):
    bh = 5 if s <= 2048 else 1
    y = torch.from_numpy(orc.softmax_causal(f32(randn((1, bh, s, s), dtype, seed=s, std=8.0)), 0.125)[0]).to(dtype)
    g = randn((bh, s, s), dtype, seed=s + 1)
    want = orc.softmax_bwd(f32(g), f32(y), 0.125, causal=True)
    # poison what must not be read: the upper triangles of g and y
    upper = torch.triu(torch.ones(s, s, dtype=torch.bool), 1)
    gd = torch.where(upper, torch.tensor(float("nan"), dtype=dtype), g).to(DEV)
    yd = torch.where(upper, torch.tensor(float("nan"), dtype=dtype), y).to(DEV)
    g_ptr = gd.data_ptr()
    dx = kernels.scaled_upper_triang_masked_softmax_backward(gd, yd, 0.125)
    assert dx.data_ptr() == g_ptr                            # written over the incoming gradient
    assert_close(dx, want, dtype, f"causal bwd S={s}")
    assert torch.count_nonzero(torch.triu(dx, 1)) == 0
    if dtype == torch.float32:                               # a softmax row's gradient sums to zero
        assert np.abs(f32(dx).astype(np.float64).sum(-1)).max() <= 1e-5


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS.get)
@pytest.mark.parametrize("sk", SIZES + LONG)
@pytest.mark.parametrize("mode", ["add", "replace"])
def test_masked_forward_key_mask(sk, dtype, mode):
    b, h, sq = (3, 2, 5) if sk <= 2048 else (2, 1, 3)
    x = randn((b, h, sq, sk), dtype, seed=sk, std=2.8)
    lens = torch.randint(1, sk + 1, (b,), generator=torch.Generator().manual_seed(2))
    mask = (torch.arange(sk)[None, :] >= lens[:, None]).view(b, 1, 1, sk)
    want = orc.softmax_masked(f32(x), mask.numpy(), 0.125, mode)
    y = kernels.masked_softmax_forward(x.to(DEV), mask.to(DEV), 0.125,
                                       kernels.MASK_ADD if mode == "add" else kernels.MASK_REPLACE)
    assert_close(y, want, dtype, f"masked fwd Sk={sk} {mode}")
    for i in range(b):                                       # padded keys get exactly 0
        assert torch.count_nonzero(y[i, :, :, int(lens[i]):]) == 0
    check_rowsums(y, dtype, want)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS.get)
@pytest.mark.parametrize("mode", ["add", "replace"])
@pytest.mark.parametrize("sq,sk", [(7, 40), (16, 1024), (3, 1001)])
def test_masked_forward_full_mask_with_fully_masked_rows(sq, sk, dtype, mode):
    # the reference's mask layout [B,1,Sq,Sk] (and [1,1,Sq,Sk]), with query rows
    # whose every key is masked: "replace" gives 1/Sk, "add" the softmax of the
    # raw scores, as the oracle spells out
    b, h = 2, 3
    x = randn((b, h, sq, sk), dtype, seed=sq * sk, std=2.8)
    g = torch.Generator().manual_seed(5)
    for mb in (b, 1):
        mask = torch.rand((mb, 1, sq, sk), generator=g) < 0.3
        mask[:, :, sq - 1, :] = True
        mask[0, :, 0, :] = True
        want = orc.softmax_masked(f32(x), mask.numpy(), 0.125, mode)
        fn_mode = kernels.MASK_ADD if mode == "add" else kernels.MASK_REPLACE
        y = kernels.masked_softmax_forward(x.to(DEV), mask.to(DEV), 0.125, fn_mode)
        assert_close(y, want, dtype, f"masked fwd full mask {mode}")
        if mode == "replace":
            assert_close(y[:, :, sq - 1], np.full((b, h, sk), 1.0 / sk, dtype=np.float32), dtype)
    # the reference-named symbol takes exactly this layout and replaces
    y2 = kernels.scaled_masked_softmax_forward(x.to(DEV), mask.to(DEV), 0.125)
    assert_close(y2, orc.softmax_masked(f32(x), mask.numpy(), 0.125, "replace"), dtype)


def test_masked_forward_no_mask_is_plain_softmax():
    x = randn((2, 2, 9, 333), torch.float32, seed=3, std=3.0)
    y = kernels.masked_softmax_forward(x.to(DEV), None, 1.0)
    assert_close(y, torch.softmax(x, -1).numpy(), torch.float32)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS.get)
@pytest.mark.parametrize("sk", SIZES + LONG)
def test_masked_backward(sk, dtype):
    b, h, sq = (2, 2, 3) if sk <= 2048 else (1, 2, 3)
    y = torch.from_numpy(orc.softmax_masked(f32(randn((b, h, sq, sk), dtype, seed=sk, std=2.8)), None, 0.125)).to(dtype)
    g = randn((b, h, sq, sk), dtype, seed=sk + 1)
    want = orc.softmax_bwd(f32(g), f32(y), 0.125)
    gd = g.to(DEV)
    dx = kernels.scaled_masked_softmax_backward(gd, y.to(DEV), 0.125)
    assert dx.data_ptr() == gd.data_ptr()
    assert_close(dx, want, dtype, f"masked bwd Sk={sk}")


def test_forward_in_place_and_unaligned_pointers():
    lib = _lib.load()
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    # y aliases x
    x = randn((2, 2, 512, 512), torch.float16, seed=1, std=8.0)
    want = orc.softmax_causal(f32(x), 0.125)
    xd = x.to(DEV)
    p = ctypes.c_void_p(xd.data_ptr())
    assert lib.oslo_softmax_causal_fwd(p, p, None, 0.125, 2, 2, 512, 1, st) == 0
    assert_close(xd, want, torch.float16, "in-place causal")
    # a base pointer that is only 2-byte aligned takes the element-wise path
    buf = torch.zeros(2 * 64 * 64 + 1, dtype=torch.float16, device=DEV)
    src = randn((2, 64, 64), torch.float16, seed=2, std=8.0)
    buf[1:] = src.reshape(-1).to(DEV)
    out = torch.empty_like(buf)
    assert lib.oslo_softmax_causal_fwd(ctypes.c_void_p(out.data_ptr() + 2), ctypes.c_void_p(buf.data_ptr() + 2),
                                       None, 0.125, 1, 2, 64, 1, st) == 0
    assert_close(out[1:].view(1, 2, 64, 64), orc.softmax_causal(f32(src)[None], 0.125), torch.float16, "unaligned")


def test_reference_symbol_names_and_errors():
    x = randn((4, 128, 128), torch.float16, seed=9, std=8.0)
    y = kernels.scaled_upper_triang_masked_softmax_forward(x.to(DEV), torch.tensor([0.125])[0])
    assert_close(y, orc.softmax_causal(f32(x)[None], 0.125)[0], torch.float16)
    with pytest.raises(RuntimeError):
        kernels.scaled_upper_triang_masked_softmax_forward(x.view(2, 2, 128, 128).to(DEV), 1.0)  # not 3-D
    with pytest.raises(RuntimeError):
        kernels.scaled_upper_triang_masked_softmax_forward(x, 1.0)                               # CPU tensor
    with pytest.raises(RuntimeError):
        kernels.scaled_upper_triang_masked_softmax_forward(x.to(DEV).double(), 1.0)               # dtype
    with pytest.raises(RuntimeError):
        kernels.causal_softmax_forward(torch.zeros(1, 1, 8, 16, device=DEV), None, 1.0)           # not square
    with pytest.raises(RuntimeError):
        kernels.masked_softmax_forward(torch.zeros(1, 1, 2, 8200, device=DEV), None, 1.0)         # too long


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=IDS.get)
def test_causal_full_size_properties(dtype):
    """The benchmark configuration [8,16,2048,2048]: size-independent properties on
    the whole tensor, the oracle on three slabs."""
    b, h, s = 8, 16, 2048
    g = torch.Generator(device=DEV).manual_seed(0)
    x = (torch.randn((b, h, s, s), generator=g, device=DEV, dtype=torch.float32) * 8).to(dtype)
    y = kernels.causal_softmax_forward(x, None, 0.125)
    assert torch.count_nonzero(torch.triu(y[::3, ::5], 1)) == 0
    sums = y.sum(-1, dtype=torch.float32)
    # bf16: a row's storage rounding alone can reach 2^-8 (see check_rowsums,
    # which applies the exact per-row figure to the slabs below)
    assert float((sums - 1).abs().max()) <= (1e-3 if dtype == torch.float16 else 1e-3 + 2.0 ** -8)
    for (bi, hi) in [(0, 0), (4, 13), (7, 15)]:
        want = orc.softmax_causal(f32(x[bi:bi + 1, hi:hi + 1]), 0.125)
        assert_close(y[bi:bi + 1, hi:hi + 1], want, dtype, f"slab {bi},{hi}")
        check_rowsums(y[bi:bi + 1, hi:hi + 1], dtype, want)
    y2 = kernels.causal_softmax_forward(x, None, 0.125)
    assert torch.equal(y, y2)                                 # deterministic
    # backward at full size: rows of dx sum to ~0, upper triangle zero, oracle on one slab
    go = torch.randn((b * h, s, s), generator=g, device=DEV, dtype=torch.float32).to(dtype)
    want = orc.softmax_bwd(f32(go[77]), f32(y.view(-1, s, s)[77]), 0.125, causal=True)
    dx = kernels.scaled_upper_triang_masked_softmax_backward(go, y.view(-1, s, s), 0.125)
    assert_close(dx[77], want, dtype, "bwd slab 77")
    assert torch.count_nonzero(torch.triu(dx[::9], 1)) == 0


def test_padded_full_size_properties():
    """The padded benchmark configuration, bf16 [16,16,1024,1024] with valid
    lengths uniform in [128,1024]: properties on the whole tensor, the oracle on
    slabs; then the same scores under a [B,1,Sq,Sk] mask whose query rows past
    the length are fully masked (additive semantics: such a row is the plain
    softmax of its scores), forward and backward."""
    dtype = torch.bfloat16
    b, h, s = 16, 16, 1024
    g = torch.Generator(device=DEV).manual_seed(0)
    x = (torch.randn((b, h, s, s), generator=g, device=DEV, dtype=torch.float32) * 8 ** 0.5).to(dtype)
    g.manual_seed(2)
    lens = torch.randint(128, 1025, (b,), generator=g, device=DEV)
    key_mask = (torch.arange(s, device=DEV)[None, :] >= lens[:, None]).view(b, 1, 1, s)
    y = kernels.masked_softmax_forward(x, key_mask, 0.125, kernels.MASK_ADD)
    assert torch.count_nonzero(y * key_mask) == 0                       # masked keys get exactly 0
    sums = y.sum(-1, dtype=torch.float32)
    assert float((sums - 1).abs().max()) <= 1e-3 + 2.0 ** -8
    assert torch.equal(y, kernels.masked_softmax_forward(x, key_mask, 0.125, kernels.MASK_ADD))
    for bi, hi in [(0, 0), (9, 7), (15, 15)]:
        want = orc.softmax_masked(f32(x[bi:bi + 1, hi:hi + 1]), key_mask[bi:bi + 1].cpu().numpy(), 0.125, "add")
        assert_close(y[bi:bi + 1, hi:hi + 1], want, dtype, f"slab {bi},{hi}")
        check_rowsums(y[bi:bi + 1, hi:hi + 1], dtype, want)
    full_mask = key_mask | (torch.arange(s, device=DEV)[None, :] >= lens[:, None]).view(b, 1, s, 1)
    yf = kernels.masked_softmax_forward(x, full_mask, 0.125, kernels.MASK_ADD)
    bi = int(torch.argmin(lens))                                        # the sample with the longest masked tail
    n = int(lens[bi])
    assert torch.equal(yf[bi, :, :n], y[bi, :, :n])                     # rows inside the length: as under the key mask
    plain = orc.softmax_masked(f32(x[bi:bi + 1, 3:4, n:]), None, 0.125, "add")
    assert_close(yf[bi:bi + 1, 3:4, n:], plain, dtype, "fully masked rows")
    go = torch.randn((b, h, s, s), generator=g, device=DEV, dtype=torch.float32).to(dtype)
    want_dx = orc.softmax_bwd(f32(go[bi, 3]), f32(yf[bi, 3]), 0.125)
    dx = kernels.scaled_masked_softmax_backward(go, yf, 0.125)
    assert_close(dx[bi, 3], want_dx, dtype, "bwd slab")
    assert torch.count_nonzero(dx[bi, :, :n] * key_mask[bi]) == 0       # no gradient into masked keys


def test_long_row_full_size_properties():
    """The long-row benchmark configuration, bf16 [1,16,8192,8192], scale 1/16:
    zeros above the diagonal, row sums, determinism on the whole tensor, the
    oracle on one head."""
    dtype = torch.bfloat16
    h, s = 16, 8192
    g = torch.Generator(device=DEV).manual_seed(0)
    x = torch.randn((1, h, s, s), generator=g, device=DEV, dtype=torch.float32).to(dtype)
    y = kernels.causal_softmax_forward(x, None, 1 / 16)
    assert torch.count_nonzero(torch.triu(y[0, ::5], 1)) == 0
    sums = y.sum(-1, dtype=torch.float32)
    assert float((sums - 1).abs().max()) <= 1e-3 + 2.0 ** -8
    assert torch.equal(y, kernels.causal_softmax_forward(x, None, 1 / 16))
    want = orc.softmax_causal(f32(x[:, 11:12]), 1 / 16)
    assert_close(y[:, 11:12], want, dtype, "head 11")
    check_rowsums(y[:, 11:12], dtype, want)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS.get)
@pytest.mark.parametrize("s", [5, 64, 520, 1024, 2048, 2050, 4096])
@pytest.mark.parametrize("with_pad", [False, True], ids=["nopad", "pad"])
def test_causal_softmax_with_fused_dropout(s, dtype, with_pad):
    """Softmax + attention dropout in one pass: the output is y*keep/(1-p) with
    the oracle's Philox mask bit for bit, the row statistics are the row's
    maximum and reciprocal sum, and the backward (which regenerates the mask and
    recomputes y from the scores and the statistics) matches the oracle."""
    b, h = (2, 2) if s <= 2048 else (1, 1)
    p, seed, offset = 0.1, 4321, 12
    x = randn((b, h, s, s), dtype, seed=s, std=8.0)
    pad = None
    if with_pad:
        lens = torch.randint(1, s + 1, (b,), generator=torch.Generator().manual_seed(2))
        pad = torch.where(torch.arange(s)[None, :] < lens[:, None], 0.0, -10000.0).float()
    want_y = orc.softmax_causal(f32(x), 0.125, None if pad is None else pad.numpy())
    keep = orc.dropout_keep_mask(seed, offset, b * h * s * s, p).reshape(b, h, s, s)
    ks = np.float32(1.0 / (1.0 - float(np.float32(p))))
    pad_dev = None if pad is None else pad.to(DEV)
    x_dev = x.to(DEV)
    yd, stats = kernels.causal_softmax_dropout_forward(x_dev, pad_dev, 0.125, p, seed, offset)
    assert_close(yd, np.where(keep, want_y * ks, np.float32(0)), dtype, f"softmax+dropout S={s}")
    lower = np.tril(np.ones((s, s), dtype=bool))
    nz = f32(yd) != 0
    assert not nz[..., ~lower].any()
    y = f32(kernels.causal_softmax_forward(x_dev, pad_dev, 0.125))
    assert np.array_equal(nz & (y != 0), keep & (y != 0))   # the mask itself, where y is non-zero
    # row statistics: the reciprocal of sum_k exp(e_k - max)
    e = f32(x).astype(np.float64) * 0.125
    if pad is not None:
        e = e + pad.numpy().astype(np.float64)[:, None, None, :]
    e = np.where(lower, e, -np.inf)
    inv = 1.0 / np.exp(e - e.max(-1, keepdims=True)).sum(-1)
    got = stats.cpu().numpy()
    assert got.shape == (b, h, s, 2)
    np.testing.assert_allclose(got[..., 1], inv, rtol=2e-6)
    unit = np.log2(np.e) if pad is None else 1.0
    np.testing.assert_allclose(got[..., 0], e.max(-1) * unit, rtol=1e-6, atol=1e-6)
    # backward: probabilities recomputed from x and the statistics
    g = randn((b, h, s, s), dtype, seed=s + 1)
    gk = np.where(keep, f32(g) * ks, np.float32(0))
    want_dx = orc.softmax_bwd(gk, want_y, 0.125, causal=True)
    dx = kernels.causal_softmax_dropout_backward(g.to(DEV), x_dev, stats, pad_dev, 0.125, p, seed, offset)
    assert_close(dx, want_dx, dtype, f"softmax+dropout bwd S={s}")
    # in place over the scores
    x2 = x_dev.clone()
    dx2 = torch.empty_like(x2)
    from oslo_amd import _lib
    with torch.cuda.device(DEV):
        _lib.check(_lib.load().oslo_softmax_causal_dropout_bwd(
            x2.data_ptr(), g.to(DEV).data_ptr(), x2.data_ptr(), stats.data_ptr(),
            None if pad_dev is None else pad_dev.data_ptr(), 0.125, p, seed, offset, b, h, s,
            kernels._dtype_code(x2, "x"), torch.cuda.current_stream().cuda_stream))
    assert torch.equal(x2, dx)
    # p == 0: the plain probabilities
    yd0, _ = kernels.causal_softmax_dropout_forward(x_dev, pad_dev, 0.125, 0.0, 0, 0)
    assert torch.equal(yd0, kernels.causal_softmax_forward(x_dev, pad_dev, 0.125))


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS.get)
@pytest.mark.parametrize("s,window", [(5, 2), (64, 1), (64, 64), (130, 7), (512, 256), (1000, 256), (1001, 33),
                                      (2048, 256), (2048, 2047), (4096, 256), (8192, 256)])
@pytest.mark.parametrize("with_pad", [False, True], ids=["nopad", "pad"])
def test_window_softmax_forward_backward(s, window, dtype, with_pad):
    """Sliding-window causal softmax (GPT-Neo's local attention) against the
    oracle, forward and backward; zero outside the band; NaNs outside the band
    are never read."""
    b, h = (2, 2) if s <= 2048 else (1, 1)
    x = randn((b, h, s, s), dtype, seed=s + window, std=8.0)
    band = np.tril(np.ones((s, s), dtype=bool)) & ~np.tril(np.ones((s, s), dtype=bool), -window)
    pad = None
    if with_pad:
        lens = torch.randint(1, s + 1, (b,), generator=torch.Generator().manual_seed(3))
        pad = torch.where(torch.arange(s)[None, :] < lens[:, None], 0.0, -10000.0).float()
    want = orc.softmax_causal(f32(x), 0.125, None if pad is None else pad.numpy(), window=window)
    poisoned = x.clone()
    poisoned[..., torch.from_numpy(~band)] = float("nan")
    y = kernels.causal_window_softmax_forward(poisoned.to(DEV), None if pad is None else pad.to(DEV), 0.125, window)
    assert_close(y, want, dtype, f"window softmax S={s} W={window}")
    assert (f32(y)[..., ~band] == 0).all()
    check_rowsums(y, dtype, want)
    g = randn((b, h, s, s), dtype, seed=s + window + 1)
    want_dx = orc.softmax_bwd(f32(g), f32(y), 0.125, causal=True, window=window)
    gp = g.clone()
    gp[..., torch.from_numpy(~band)] = float("nan")
    dx = kernels.causal_window_softmax_backward(gp.to(DEV), y, 0.125, window)
    assert_close(dx, want_dx, dtype, f"window softmax bwd S={s} W={window}")
    assert (f32(dx)[..., ~band] == 0).all()
    if window >= s:   # the plain causal kernel
        assert torch.equal(y, kernels.causal_softmax_forward(x.to(DEV), None if pad is None else pad.to(DEV), 0.125))
