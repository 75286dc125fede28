"""Backward of the one-kernel prompt attention, called through the C ABI,
against the CPU oracle in float64 (small cases) and the same formulas in
float64 on the device (large ones).

Tolerance. With REL the half-ulp of the storage type (2^-8 bf16, 2^-11 fp16),
every rounding moves a value by at most REL of its magnitude:
  * each gradient is an fp32 sum rounded once:                REL * |ref|
  * P and dS are rounded before the products that sum them:   REL * (P^T |dO|),
    REL * scale * (|dS| |K|), REL * scale * (|dS|^T |Q|)
  * delta is formed from the forward's *rounded* output, so it is off by up
    to REL * sum_d |dO| |O| =: e_delta, which moves dS by scale * P * e_delta.
The bar is twice the sum of these bounds (they are computed in float64 for the
case at hand) plus 1e-4."""

import math

import numpy as np
import pytest
import torch

from oracle import oslo_oracle as orc
from oslo_amd import kernels
from tests.util import IDS, f32, randn

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
HALVES = [torch.float16, torch.bfloat16]
REL = {torch.float16: 2.0 ** -11, torch.bfloat16: 2.0 ** -8}


def reference(q, k, v, do, scale, pad=None, window=0, keep=None, p_drop=0.0):
    """float64 gradients and the error bounds described above, on the inputs' device."""
    q, k, v, do = q.double(), k.double(), v.double(), do.double()
    s = q.shape[2]
    w = q @ k.transpose(-1, -2) * scale
    if pad is not None:
        w = w + pad.double()[:, None, None, :]
    i = torch.arange(s, device=q.device)
    hidden = i[None, :] > i[:, None]
    if window:
        hidden = hidden | (i[None, :] <= i[:, None] - window)
    p = torch.softmax(w.masked_fill(hidden, float("-inf")), -1)
    m = torch.ones_like(p) if keep is None else keep.double() / (1.0 - p_drop)   # the dropout factor on P
    o = (m * p) @ v
    dv = (m * p).transpose(-1, -2) @ do
    dp = m * (do @ v.transpose(-1, -2))
    delta = (do * o).sum(-1, keepdim=True)
    ds = p * (dp - delta)
    dq = scale * (ds @ k)
    dk = scale * (ds.transpose(-1, -2) @ q)
    e_delta = (do.abs() * o.abs()).sum(-1, keepdim=True)
    ds_mag = ds.abs() + p * e_delta
    bounds = {
        "dq": dq.abs() + scale * (ds_mag @ k.abs()),
        "dk": dk.abs() + scale * (ds_mag.transpose(-1, -2) @ q.abs()),
        "dv": dv.abs() + (m * p).transpose(-1, -2) @ do.abs(),
    }
    return o, {"dq": dq, "dk": dk, "dv": dv}, bounds


def backward_both_ways(do, q, k, v, out, lse, scale, pad=None, window=0, p=0.0, seed=0, offset=0):
    """The backward with every pass computing its scores and with the
    probabilities handed from the dQ pass to the dK/dV pass through the tile
    store: the same bits (the same products, rounded and summed in the same
    order), whatever the head size."""
    plain = kernels.attention_prefill_backward(do, q, k, v, out, lse, scale, pad, window, p, seed, offset, store=False)
    stored = kernels.attention_prefill_backward(do, q, k, v, out, lse, scale, pad, window, p, seed, offset, store=True)
    for name, a, b in zip(("dq", "dk", "dv"), plain, stored):
        assert torch.equal(a, b), (name, tuple(q.shape), window, p, (a.float() - b.float()).abs().max().item())
    return stored


def run(q, k, v, do, scale, pad=None, window=0):
    out, lse = kernels.attention_prefill_forward(q, k, v, scale, pad, window, want_lse=True)
    dq, dk, dv = backward_both_ways(do, q, k, v, out, lse, scale, pad, window)
    return out, lse, {"dq": dq, "dk": dk, "dv": dv}


def check(got, want, bounds, dtype, what):
    for name in ("dq", "dk", "dv"):
        assert torch.isfinite(got[name]).all(), (name, what)
        excess = ((got[name].double() - want[name]).abs() - 2 * REL[dtype] * bounds[name]).max().item()
        assert excess <= 1e-4, (name, excess, what)


def padding(b, s, seed):
    g = torch.Generator().manual_seed(seed)
    lens = torch.randint(max(1, s // 2), s + 1, (b,), generator=g)
    return torch.where(torch.arange(s)[None, :] < lens[:, None], 0.0, -10000.0).float()


@pytest.mark.parametrize("dtype", HALVES, ids=IDS.get)
@pytest.mark.parametrize("d", [64, 128, 256])
@pytest.mark.parametrize("s", [1, 8, 31, 64, 65, 128, 200, 332])
def test_backward_matches_oracle(s, d, dtype):
    b, h = 2, 3
    q, k, v, do = (randn((b, h, s, d), dtype, seed=11 * s + i) for i in range(4))
    scale = 1.0 / math.sqrt(d)
    dev = [t.to(DEV) for t in (q, k, v, do)]
    for pad in ([None, padding(b, s, s)] if s % 4 == 0 else [None]):
        out, lse, got = run(*dev, scale, None if pad is None else pad.to(DEV))
        flat = [f32(t).reshape(b * h, s, d) for t in (q, k, v, do)]
        want = orc.attention_prefill_bwd(*flat, scale, None if pad is None else pad.numpy().repeat(h, axis=0))
        _, _, bounds = reference(*dev, scale, None if pad is None else pad.to(DEV))
        want = {n: torch.from_numpy(w.reshape(b, h, s, d)).to(DEV) for n, w in zip(("dq", "dk", "dv"), want)}
        check(got, want, bounds, dtype, (s, d, pad is not None))
        # the log-sum-exp the forward hands over: log2 of the sum of 2^(log2e * score) over the visible keys
        scores = np.einsum("bhid,bhjd->bhij", f32(q).astype(np.float64), f32(k).astype(np.float64)) * scale
        if pad is not None:
            scores = scores + pad.numpy().astype(np.float64)[:, None, None, :]
        scores = np.where(np.tril(np.ones((s, s), dtype=bool)), scores, -np.inf)
        m = scores.max(-1, keepdims=True)
        want_lse = (m[..., 0] + np.log(np.exp(scores - m).sum(-1))) * math.log2(math.e)
        assert np.abs(f32(lse).astype(np.float64) - want_lse).max() <= 2e-3 * (1 + np.abs(want_lse).max() * 1e-3)


@pytest.mark.parametrize("dtype", HALVES, ids=IDS.get)
@pytest.mark.parametrize("b,h,s,d", [(2, 8, 1024, 64), (1, 5, 1000, 128), (1, 4, 2048, 256), (1, 2, 2300, 128)])
def test_backward_long_prompts(b, h, s, d, dtype):
    q, k, v, do = (randn((b, h, s, d), dtype, seed=s + i).to(DEV) for i in range(4))
    pads = [None, padding(b, s, 3).to(DEV)] if s % 4 == 0 else [None]
    for p in pads:
        _, _, got = run(q, k, v, do, 0.1, p)
        _, want, bounds = reference(q, k, v, do, 0.1, p)
        check(got, want, bounds, dtype, (b, h, s, d, p is not None))


# windows shorter than a step of 32, ragged against steps, tiles and blocks, and at least the prompt
@pytest.mark.parametrize("dtype", HALVES, ids=IDS.get)
@pytest.mark.parametrize("window", [1, 5, 32, 33, 64, 100, 256, 300, 700])
def test_backward_sliding_window(window, dtype):
    for (b, h, s, d) in ((2, 3, 520, 64), (1, 2, 360, 128), (1, 2, 700, 256)):
        q, k, v, do = (randn((b, h, s, d), dtype, seed=window + i).to(DEV) for i in range(4))
        pad = padding(b, s, window).to(DEV)
        for p in (None, pad):
            _, _, got = run(q, k, v, do, 0.1, p, window)
            _, want, bounds = reference(q, k, v, do, 0.1, p, window)
            check(got, want, bounds, dtype, (b, h, s, d, window, p is not None))
    b, h, s, d = 1, 2, 96, 64
    q, k, v, do = (randn((b, h, s, d), dtype, seed=3 * window + i) for i in range(4))
    dev = [t.to(DEV) for t in (q, k, v, do)]
    _, _, got = run(*dev, 0.1, None, window)
    want = orc.attention_prefill_bwd(*[f32(t).reshape(b * h, s, d) for t in (q, k, v, do)], 0.1, None, window)
    want = {n: torch.from_numpy(w.reshape(b, h, s, d)).to(DEV) for n, w in zip(("dq", "dk", "dv"), want)}
    _, _, bounds = reference(*dev, 0.1, None, window)
    check(got, want, bounds, dtype, ("oracle", window))


@pytest.mark.parametrize("dtype", HALVES, ids=IDS.get)
def test_backward_strided_inputs_determinism_and_closed_forms(dtype):
    """q, k, v as slices of one packed projection and the gradient of the output
    in merged-heads memory (how a model hands them over); two runs give the same
    bits; with equal scores the probabilities are 1/(i+1), so dV is a weighted
    suffix sum of dO; a single position passes dO through to dV and gives
    (all but) no gradient to q and k."""
    b, h, s, d = 2, 4, 384, 64
    packed = randn((b, s, 3, h, d), dtype, seed=1).to(DEV)
    q, k, v = (packed[:, :, i].permute(0, 2, 1, 3) for i in range(3))
    do = randn((b, s, h, d), dtype, seed=2).to(DEV).permute(0, 2, 1, 3)
    _, _, got = run(q, k, v, do, 0.125)
    _, want, bounds = reference(q, k, v, do, 0.125)
    check(got, want, bounds, dtype, "strided")
    _, _, again = run(q, k, v, do, 0.125)
    assert all(torch.equal(got[n], again[n]) for n in got)
    zero = torch.zeros_like(q)
    _, _, flat = run(zero, k, v, do, 0.125)
    weights = 1.0 / torch.arange(1, s + 1, device=DEV, dtype=torch.float64)
    suffix = torch.flip(torch.cumsum(torch.flip(do.double() * weights[None, None, :, None], [2]), 2), [2])
    excess = ((flat["dv"].double() - suffix).abs() - 2 * REL[dtype] * (suffix.abs() + 8.0)).max().item()
    assert excess <= 1e-4
    one = [t[:, :, :1].contiguous() for t in (q, k, v, do)]
    _, _, single = run(*one, 0.125)
    # the one probability is exactly 1; dP and delta are the same dot product summed in two orders,
    # so dS (and with it dq, dk) is zero up to the rounding of an fp32 sum
    assert torch.equal(single["dv"], one[3])
    assert single["dq"].abs().max().item() <= 1e-4 and single["dk"].abs().max().item() <= 1e-4


def test_backward_full_size_properties():
    """The GPT-J shape of the benchmark, [8, 16, 2048, 256] bf16, where the oracle
    would take days: heads taken one at a time against the float64 formulas on
    the device; the same call twice gives the same bits; no gradient comes
    back for dO = 0; and the gradients are linear in dO (doubling it doubles
    them exactly: a power of two)."""
    dtype = torch.bfloat16
    b, h, s, d = 8, 16, 2048, 256
    g = torch.Generator(device=DEV).manual_seed(3)
    q, k, v, do = (torch.randn((b, h, s, d), generator=g, device=DEV).to(dtype) for _ in range(4))
    scale = d ** -0.5
    out, lse, got = run(q, k, v, do, scale)
    for bb, hh in ((0, 0), (3, 7), (7, 15)):
        one = [t[bb:bb + 1, hh:hh + 1] for t in (q, k, v, do)]
        _, want, bounds = reference(*one, scale)
        check({n: t[bb:bb + 1, hh:hh + 1] for n, t in got.items()}, want, bounds, dtype, ("full size", bb, hh))
    again = kernels.attention_prefill_backward(do, q, k, v, out, lse, scale)
    for t, n in zip(again, ("dq", "dk", "dv")):
        assert torch.equal(t, got[n]), n
    twice = kernels.attention_prefill_backward(do * 2, q, k, v, out, lse, scale)
    for t, n in zip(twice, ("dq", "dk", "dv")):
        assert torch.equal(t, got[n] * 2), n
    none = kernels.attention_prefill_backward(torch.zeros_like(do), q, k, v, out, lse, scale)
    for t in none:
        assert not t.any()


def keep_mask(b, h, s, p, seed, offset):
    """The mask of the softmax kernel with fused dropout: flat index over [B, H, S, S]."""
    return torch.from_numpy(orc.dropout_keep_mask(seed, offset, b * h * s * s, p).reshape(b, h, s, s))


@pytest.mark.parametrize("dtype", HALVES, ids=IDS.get)
@pytest.mark.parametrize("d", [64, 128, 256])
@pytest.mark.parametrize("s", [8, 64, 200, 328])
def test_attention_dropout_forward_and_backward(s, d, dtype):
    """Attention dropout inside the kernels: the forward equals the oracle's
    with the keep mask the softmax kernel with fused dropout draws for the same
    seed and offset, the log-sum-exp is that of the undropped probabilities,
    the backward regenerates the same mask."""
    b, h, p, seed, offset = 2, 3, 0.25, 1234, 8
    scale = 1.0 / math.sqrt(d)
    q, k, v, do = (randn((b, h, s, d), dtype, seed=13 * s + i) for i in range(4))
    dev = [t.to(DEV) for t in (q, k, v, do)]
    keep = keep_mask(b, h, s, p, seed, offset)
    for pad, window in ((None, 0), (padding(b, s, s), 0), (None, 40)):
        padd = None if pad is None else pad.to(DEV)
        out, lse = kernels.attention_prefill_forward(*dev[:3], scale, padd, window, want_lse=True, p=p, seed=seed,
                                                     offset=offset)
        plain, lse0 = kernels.attention_prefill_forward(*dev[:3], scale, padd, window, want_lse=True)
        assert torch.equal(lse, lse0)
        o_ref, want, bounds = reference(*dev, scale, padd, window, keep.to(DEV), p)
        vmax = 4.0 / (1 - p)
        excess = ((out.double() - o_ref).abs() - REL[dtype] * (o_ref.abs() + vmax)).max().item()
        assert excess <= 1e-4, (excess, s, d, "forward")
        dq, dk, dv = backward_both_ways(dev[3], *dev[:3], out, lse, scale, padd, window, p, seed, offset)
        check({"dq": dq, "dk": dk, "dv": dv}, want, bounds, dtype, (s, d, pad is not None, window))
        if pad is None and window == 0 and s <= 64:
            flat = [f32(t).reshape(b * h, s, d) for t in (q, k, v, do)]
            kf = keep.numpy().reshape(b * h, s, s)
            o_orc = orc.attention_prefill(*flat[:3], scale, keep=kf, p=p).reshape(b, h, s, d)
            assert np.abs(o_orc - o_ref.cpu().numpy()).max() <= 1e-9
            g_orc = orc.attention_prefill_bwd(*flat, scale, keep=kf, p=p)
            for n, g in zip(("dq", "dk", "dv"), g_orc):
                assert np.abs(g.reshape(b, h, s, d) - want[n].cpu().numpy()).max() <= 1e-9
    # another offset is another mask; the same one repeats bit for bit
    again = kernels.attention_prefill_forward(*dev[:3], scale, None, 0, want_lse=True, p=p, seed=seed, offset=offset)[0]
    other = kernels.attention_prefill_forward(*dev[:3], scale, None, 0, want_lse=True, p=p, seed=seed, offset=offset + 4)[0]
    first = kernels.attention_prefill_forward(*dev[:3], scale, None, 0, want_lse=True, p=p, seed=seed, offset=offset)[0]
    assert torch.equal(again, first) and not torch.equal(again, other)


def test_random_combinations_forward_and_backward():
    """Forty draws of (type, head size, length, scale, window, padding mask,
    dropout) that the tests above only take one or two at a time, forward and
    backward against the float64 formulas on the device."""
    import random

    rng = random.Random(5)
    for case in range(40):
        dt = rng.choice(HALVES)
        d = rng.choice([64, 128, 256])
        s = rng.choice([1, 2, 31, 32, 33, 64, 100, 128, 129, 200, 256, 300, 384, 500, 640, 777, 1024])
        b, h = rng.randint(1, 2), rng.randint(1, 3)
        scale = rng.choice([1.0 / math.sqrt(d), 0.1, 0.3])
        window = rng.choice([0, 0, 1, 3, 31, 32, 33, 64, 100, 128, 129, 200, 300, 511])
        pad = padding(b, s, case).to(DEV) if rng.random() < 0.4 and s % 4 == 0 else None
        p = rng.choice([0.0, 0.0, 0.1, 0.5]) if s % 8 == 0 else 0.0
        g = torch.Generator(device=DEV).manual_seed(case)
        q, k, v, do = (torch.randn((b, h, s, d), generator=g, device=DEV).to(dt) for _ in range(4))
        seed, offset = 99 + case, 4 * case
        keep = keep_mask(b, h, s, p, seed, offset).to(DEV) if p > 0 else None
        what = (case, dt, b, h, s, d, scale, window, pad is not None, p)
        out, lse = kernels.attention_prefill_forward(q, k, v, scale, pad, window, want_lse=True, p=p, seed=seed,
                                                     offset=offset)
        dq, dk, dv = backward_both_ways(do, q, k, v, out, lse, scale, pad, window, p, seed, offset)
        o_ref, want, bounds = reference(q, k, v, do, scale, pad, window, keep, p)
        excess = ((out.double() - o_ref).abs() - REL[dt] * (o_ref.abs() + 5.0 / (1 - p))).max().item()
        assert torch.isfinite(out).all() and excess <= 1e-4, (excess, what)
        check({"dq": dq, "dk": dk, "dv": dv}, want, bounds, dt, what)


def test_attention_dropout_long_prompt_and_operator():
    """At [2,4,1024,128]: against the float64 formulas with the regenerated mask;
    and through FusedPrefillAttention.apply, which takes seed and offset from the
    device generator and advances it like the softmax kernel with dropout."""
    from oslo_amd import FusedPrefillAttention
    dtype, b, h, s, d, p = torch.bfloat16, 2, 4, 1024, 128, 0.1
    q, k, v, do = (randn((b, h, s, d), dtype, seed=40 + i).to(DEV) for i in range(4))
    torch.manual_seed(77)
    gen = torch.cuda.default_generators[0]
    seed, off0 = gen.initial_seed(), gen.get_offset()
    qq, kk, vv = (t.clone().requires_grad_(True) for t in (q, k, v))
    out = FusedPrefillAttention.apply(qq, kk, vv, None, 0.1, None, p)
    assert gen.get_offset() == off0 + 4
    out.backward(do)
    keep = keep_mask(b, h, s, p, seed, off0).to(DEV)
    o_ref, want, bounds = reference(q, k, v, do, 0.1, None, 0, keep, p)
    assert ((out.detach().double() - o_ref).abs() - REL[dtype] * (o_ref.abs() + 4.0 / (1 - p))).max().item() <= 1e-4
    check({"dq": qq.grad, "dk": kk.grad, "dv": vv.grad}, want, bounds, dtype, "operator")
    # the fraction of (query, key) pairs dropped, read off a forward with v = identity-like columns:
    # with q = 0 the probabilities of row i are 1/(i+1), so out[i] = sum_s keep/(1-p)/(i+1) * v[s]
    ones = torch.ones_like(v)
    frac = kernels.attention_prefill_forward(torch.zeros_like(q), k, ones, 1.0, None, 0, want_lse=True, p=p,
                                             seed=seed, offset=off0)[0][..., 0].double()
    want_frac = (keep.double().tril().sum(-1) / (1 - p)) / torch.arange(1, s + 1, device=DEV)
    assert (frac - want_frac).abs().max().item() <= 2.0 ** -7 * 2


@pytest.mark.parametrize("d", [64, 256])
def test_tile_store_smaller_than_the_heads(d, monkeypatch):
    """A store that holds 8 heads (16 with the second limit) where the call has
    20: the heads go through it in launches of 8, 8 and 4 (16 and 4), with a
    window, a padding mask and dropout; the same bits as without a store,
    whatever the default picks for the head size."""
    dtype, b, h, s, p, seed, offset = torch.bfloat16, 4, 5, 264, 0.2, 5, 12
    q, k, v, do = (randn((b, h, s, d), dtype, seed=70 + i).to(DEV) for i in range(4))
    pad = padding(b, s, 9).to(DEV)
    lib = kernels._lib.load()
    least = lib.oslo_attention_prefill_bwd_store_bytes(1, 8, s)
    assert lib.oslo_attention_prefill_bwd_store_bytes(b, h, s) == 3 * least     # 20 heads: three groups of 8
    assert least == 8 * (12 * 13 // 2) * 4096                                    # 264 positions: 12 tiles of 32 (3 blocks of 128)
    for window in (0, 70):
        out, lse = kernels.attention_prefill_forward(q, k, v, 0.1, pad, window, want_lse=True, p=p, seed=seed, offset=offset)
        want = kernels.attention_prefill_backward(do, q, k, v, out, lse, 0.1, pad, window, p, seed, offset, store=False)
        for limit in (least, 2 * least + 100, 1 << 40):
            monkeypatch.setattr(kernels, "PREFILL_BWD_STORE_LIMIT", limit)
            got = kernels.attention_prefill_backward(do, q, k, v, out, lse, 0.1, pad, window, p, seed, offset, store=True)
            assert all(torch.equal(x, y) for x, y in zip(got, want)), (window, limit)
        auto = kernels.attention_prefill_backward(do, q, k, v, out, lse, 0.1, pad, window, p, seed, offset)
        assert all(torch.equal(x, y) for x, y in zip(auto, want))
    # a limit below 8 heads: the default does without a store
    monkeypatch.setattr(kernels, "PREFILL_BWD_STORE_LIMIT", least - 1)
    auto = kernels.attention_prefill_backward(do, q, k, v, out, lse, 0.1, pad, 70, p, seed, offset)
    assert all(torch.equal(x, y) for x, y in zip(auto, want))


def test_backward_rejects_what_it_cannot_take():
    q = torch.zeros(1, 2, 16, 48, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError):
        kernels.attention_prefill_forward(q, q, q, 1.0, want_lse=True)          # head size
    q = torch.zeros(1, 2, 16, 64, dtype=torch.float32, device=DEV)
    with pytest.raises(RuntimeError):
        kernels.attention_prefill_forward(q, q, q, 1.0, want_lse=True)          # fp32
    q = torch.zeros(1, 2, 16, 64, dtype=torch.bfloat16, device=DEV)
    out, lse = kernels.attention_prefill_forward(q, q, q, 1.0, want_lse=True)
    with pytest.raises(RuntimeError):
        kernels.attention_prefill_backward(q, q, q, q, out, lse[:, :1], 1.0)    # lse of another shape
