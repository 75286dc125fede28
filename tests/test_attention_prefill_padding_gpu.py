"""Left padding in the one-kernel prompt attention and its backward: the first
key tiles of a sequence masked in full, with the mask values callers build
(-10000, -1e10, -1e30, the most negative bf16 / fp32 number, -inf). A query
that is itself padding sees masked keys only, so its reference maximum starts
at a masked score and has to rise from there for the queries behind it; the
rows and keys of the valid part must match the float64 formulas (a padded
query only sees padded keys, so it contributes nothing to a valid key's
gradient), and nothing anywhere may be inf or NaN: the gradients of padded keys
flow on into the weight gradients.

Tolerances: those of tests/test_attention_prefill_gpu.py (forward) and
tests/test_attention_prefill_bwd_gpu.py (backward)."""

import math

import pytest
import torch

from oslo_amd import FusedPrefillAttention, kernels
from tests.test_attention_prefill_bwd_gpu import REL, keep_mask, reference
from tests.util import IDS, randn

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
HALVES = [torch.float16, torch.bfloat16]
MASKS = {
    "m1e4": -10000.0,
    "m1e10": -1e10,
    "m1e30": -1e30,
    "bf16min": float(torch.finfo(torch.bfloat16).min),
    "fp32min": float(torch.finfo(torch.float32).min),
    "inf": float("-inf"),
}


def left_padding(lengths, s, value):
    """fp32 [B, S]: the first lengths[b] keys of sequence b carry `value`."""
    pad = torch.zeros((len(lengths), s))
    for b, n in enumerate(lengths):
        pad[b, :n] = value
    return pad


def check_valid_part(got, want, bounds, lengths, dtype, what):
    """got / want: dicts of [B, H, S, D]; rows from lengths[b] on are compared."""
    for name, g in got.items():
        assert torch.isfinite(g).all(), (name, "not finite", what)
        for b, n in enumerate(lengths):
            err = (g[b, :, n:].double() - want[name][b, :, n:]).abs()
            excess = (err - bounds[name][b, :, n:]).max().item() if err.numel() else 0.0
            assert excess <= 1e-4, (name, b, excess, what)


@pytest.mark.parametrize("dtype", HALVES, ids=IDS.get)
@pytest.mark.parametrize("d", [64, 128, 256])
@pytest.mark.parametrize("value", list(MASKS), ids=list(MASKS))
def test_left_padding_forward_and_backward(value, d, dtype):
    b, h, s = 3, 2, 320
    lengths = [32, 160, 44]  # one tile; a whole block of queries and a tile more; ragged against the tiles
    scale = 1.0 / math.sqrt(d)
    q, k, v, do = (randn((b, h, s, d), dtype, seed=17 * d + i).to(DEV) for i in range(4))
    pad = left_padding(lengths, s, MASKS[value]).to(DEV)
    finite = left_padding(lengths, s, -1e5).to(DEV)  # what the float64 formulas take: exp(-1e5) is 0 there too
    for window, p in ((0, 0.0), (48, 0.0), (0, 0.25), (200, 0.25)):
        seed, offset = 77, 12
        keep = keep_mask(b, h, s, p, seed, offset).to(DEV) if p > 0 else None
        out, lse = kernels.attention_prefill_forward(q, k, v, scale, pad, window, want_lse=True, p=p, seed=seed,
                                                     offset=offset)
        dq, dk, dv = kernels.attention_prefill_backward(do, q, k, v, out, lse, scale, pad, window, p, seed, offset)
        o_ref, want, bounds = reference(q, k, v, do, scale, finite, window, keep, p)
        what = (value, d, window, p)
        assert torch.isfinite(lse).all(), what
        vmax = 5.0 / (1 - p)
        check_valid_part({"out": out}, {"out": o_ref}, {"out": REL[dtype] * (o_ref.abs() + vmax)}, lengths, dtype, what)
        check_valid_part({"dq": dq, "dk": dk, "dv": dv}, want, {n: 2 * REL[dtype] * bd for n, bd in bounds.items()},
                         lengths, dtype, what)
        if p == 0.0:  # the forward without the log-sum-exp is another entry point
            plain = kernels.attention_prefill_forward(q, k, v, scale, pad, window)
            assert torch.equal(plain, out), what


@pytest.mark.parametrize("dtype", HALVES, ids=IDS.get)
def test_every_key_masked_and_mixed_padding(dtype):
    """A sequence whose every key is masked (all of its rows are padding) beside
    a clean one and one padded on both sides: finite everywhere, the clean
    sequence bit-equal to a call without a mask, the valid middle as the
    formulas say."""
    b, h, s, d = 3, 2, 256, 128
    q, k, v, do = (randn((b, h, s, d), dtype, seed=5 + i).to(DEV) for i in range(4))
    for value in ("m1e4", "bf16min", "inf"):
        pad = torch.zeros((b, s))
        pad[0, :] = MASKS[value]
        pad[2, :70] = MASKS[value]
        pad[2, 200:] = MASKS[value]
        pad = pad.to(DEV)
        out, lse = kernels.attention_prefill_forward(q, k, v, 0.1, pad, 0, want_lse=True)
        grads = kernels.attention_prefill_backward(do, q, k, v, out, lse, 0.1, pad, 0)
        for t in (out, lse) + tuple(grads):
            assert torch.isfinite(t).all(), value
        clean, lse1 = kernels.attention_prefill_forward(q[1:2], k[1:2], v[1:2], 0.1, None, 0, want_lse=True)
        assert (out[1:2].float() - clean.float()).abs().max().item() <= 2 * REL[dtype] * 5.0
        finite = torch.where(pad < 0, -1e5, 0.0)
        o_ref, want, bounds = reference(q, k, v, do, 0.1, finite)
        got = dict(zip(("dq", "dk", "dv"), grads))
        # sequence 2: queries 70..199 see valid keys 70..199 (and masked ones, with probability 0); the
        # gradients of those keys also take the queries behind them, 200.., which are real rows
        err = (out[2, :, 70:].double() - o_ref[2, :, 70:]).abs() - REL[dtype] * (o_ref[2, :, 70:].abs() + 5.0)
        assert err.max().item() <= 1e-4, value
        for n in ("dq", "dk", "dv"):
            e = (got[n][2, :, 70:].double() - want[n][2, :, 70:]).abs() - 2 * REL[dtype] * bounds[n][2, :, 70:]
            assert e.max().item() <= 1e-4, (n, value)


def test_operator_takes_infinite_masks_in_training():
    """FusedPrefillAttention under autograd with a -inf / finfo.min mask of
    left padding: output and parameter-side gradients finite."""
    b, h, s, d = 2, 4, 192, 64
    for value in ("inf", "bf16min"):
        q, k, v = (randn((b, h, s, d), torch.bfloat16, seed=i).to(DEV).requires_grad_(True) for i in range(3))
        mask = left_padding([64, 0], s, MASKS[value]).view(b, 1, 1, s).to(DEV)
        assert FusedPrefillAttention.is_available(q, k, mask, training=True, dropout_p=0.0)
        out = FusedPrefillAttention.apply(q, k, v, mask, 0.125)
        out.float().square().sum().backward()
        for t in (out, q.grad, k.grad, v.grad):
            assert torch.isfinite(t).all(), value
