"""A randomized sweep over every kernel family: shapes, dtypes, masks, windows,
seeds and positions drawn from a seeded generator, each result compared on the
device with the same expression written in torch fp32 (float64 for the
attention of a decoding step). It complements the oracle tests, which pin
exact bars on chosen shapes, by covering shapes nobody chose: 250 draws here;
the same loop was run for 4500 draws with other seeds without a failure (the
attention over a whole prompt joined later, on a stream of draws of its own; a
loop of that family alone, with left and right padding, windows and strided
layouts, was run for 6900 draws without a failure)."""

import random

import pytest
import torch

from oslo_amd import kernels

pytestmark = pytest.mark.gpu

dev = "cuda:0"


def test_random_shapes_against_torch_expressions():
    rng = random.Random(0)
    N = 250
    failures = []

    def report(name, err, tol, desc):
        if not (err <= tol):
            failures.append((name, desc, err, tol))

    DT = [torch.float32, torch.float16, torch.bfloat16]
    TOL = {torch.float32: 2e-6, torch.float16: 2e-3, torch.bfloat16: 1.6e-2}
    def pick_len_from(r_):
        r = r_.random()
        if r < 0.3:
            return r_.randint(1, 70)
        if r < 0.6:
            return min(8192, r_.choice([64, 128, 256, 512, 1024, 2048, 4096, 8192]) + r_.choice([-8, -1, 0, 0, 1, 8]))
        return r_.randint(1, 8192)

    def pick_len():
        return pick_len_from(rng)

    rng_prompt = random.Random(1)
    for it in range(N):
        dt = rng.choice(DT)
        tol = TOL[dt]
        # causal softmax fwd/bwd (+pad, +window)
        S = max(1, min(pick_len(), 4096 if dt == torch.float32 else 8192))
        S = min(S, 2048) if rng.random() < 0.7 else S
        b, h = rng.randint(1, 3), rng.randint(1, 3)
        if b * h * S * S > 6e7:
            b = h = 1
        scale = rng.choice([1.0, 0.125, 0.3])
        x = (torch.randn(b, h, S, S, device=dev) * rng.choice([1, 4, 8])).to(dt)
        pad = None
        if rng.random() < 0.5:
            lens = torch.randint(1, S + 1, (b,), device=dev)
            pad = torch.where(torch.arange(S, device=dev)[None] < lens[:, None], 0.0, -10000.0).float().contiguous()
        window = rng.choice([0, 0, 1, 7, 64, 256])
        e = x.float() * scale
        if pad is not None:
            e = e + pad[:, None, None, :]
        i = torch.arange(S, device=dev)
        vis = i[None, :] <= i[:, None]
        if window:
            vis = vis & (i[None, :] > i[:, None] - window)
        ref = torch.softmax(e.masked_fill(~vis, float("-inf")), -1)
        y = kernels.causal_window_softmax_forward(x, pad, scale, window) if window else kernels.causal_softmax_forward(x, pad, scale)
        report("causal_fwd", (y.float() - ref).abs().max().item(), tol, (dt, b, h, S, scale, pad is not None, window))
        g = torch.randn(b * h, S, S, device=dev).to(dt)
        yf = y.float().view(b * h, S, S)
        want = scale * yf * (g.float() - (g.float() * yf).sum(-1, keepdim=True))
        if window:
            dx = kernels.causal_window_softmax_backward(g.clone().view(b, h, S, S), y, scale, window).view(b * h, S, S)
        else:
            dx = kernels.scaled_upper_triang_masked_softmax_backward(g.clone(), y.view(b * h, S, S), scale)
        report("causal_bwd", (dx.float() - want).abs().max().item(), tol * max(1.0, want.abs().max().item()), (dt, b, h, S, window))
        # masked softmax
        sq, sk = rng.randint(1, 40), pick_len()
        xm = (torch.randn(b, h, sq, sk, device=dev) * 3).to(dt)
        mq = rng.choice([1, sq])
        mb = rng.choice([1, b])
        mask = torch.rand(mb, 1, mq, sk, device=dev) < 0.3
        em = xm.float() * scale + mask.float() * -10000.0
        ym = kernels.masked_softmax_forward(xm, mask, scale, kernels.MASK_ADD)
        report("masked_fwd", (ym.float() - torch.softmax(em, -1)).abs().max().item(), tol, (dt, b, h, sq, sk))
        # epilogues
        rows, cols = rng.randint(1, 300), rng.choice([rng.randint(1, 300), rng.choice([256, 768, 1024, 4096]) + rng.choice([0, 0, 8, -8, 1])])
        a = torch.randn(rows, cols, device=dev).to(dt)
        bias = (torch.randn(cols, device=dev) * 0.5).to(dt)
        out = kernels.bias_gelu_forward(a, bias)
        refg = torch.nn.functional.gelu(a.float() + bias.float(), approximate="tanh")
        report("bias_gelu", ((out.float() - refg).abs() / refg.abs().clamp(min=1)).max().item(), tol, (dt, rows, cols))
        go = torch.randn(rows, cols, device=dev).to(dt)
        xa = (a.float() + bias.float()).requires_grad_(True)
        torch.nn.functional.gelu(xa, approximate="tanh").backward(go.float())
        dy, db = kernels.bias_gelu_backward(go, a, bias)
        report("bias_gelu_bwd", ((dy.float() - xa.grad).abs() / xa.grad.abs().clamp(min=1)).max().item(), max(tol, 1e-5), (dt, rows, cols))
        report("bias_gelu_dbias", ((db.float() - xa.grad.sum(0)).abs() / (xa.grad.abs().sum(0) + 1)).max().item(), max(tol, 1e-5), (dt, rows, cols))
        res = torch.randn(rows, cols, device=dev).to(dt)
        o0 = kernels.bias_dropout_add_forward(a, bias, res, 0.0, 0, 0)
        report("bda_p0", (o0.float() - (a.float() + bias.float() + res.float())).abs().max().item() / 8, tol, (dt, rows, cols))
        p = rng.choice([0.1, 0.5])
        seed, off = rng.randint(0, 2**40), 4 * rng.randint(0, 2**30)
        ones = torch.ones(rows, cols, device=dev, dtype=dt)
        keep = kernels.bias_dropout_add_forward(ones, None, None, p, seed, off) != 0
        o1 = kernels.bias_dropout_add_forward(a, bias, res, p, seed, off)
        want1 = (a.float() + bias.float()) * keep / (1 - p) + res.float()
        report("bda_p", ((o1.float() - want1).abs() / want1.abs().clamp(min=1)).max().item(), tol, (dt, rows, cols, p))
        # few-row linear, both layouts
        m = rng.randint(1, 8)
        vec = 4 if dt == torch.float32 else 8
        k = vec * rng.randint(1, 600)
        n = rng.randint(1, 700)
        xl = torch.randn(m, k, device=dev).to(dt)
        w = (torch.randn(n, k, device=dev) * 0.05).to(dt)
        bl = torch.randn(n, device=dev).to(dt)
        gelu = rng.random() < 0.5
        refl = xl.float() @ w.float().t() + bl.float()
        if gelu:
            refl = torch.nn.functional.gelu(refl, approximate="tanh")
        ol = kernels.linear_rows_forward(xl, w, bl, gelu)
        mass = xl.float().abs() @ w.float().abs().t() + 1
        report("linear_rows", ((ol.float() - refl).abs() / (refl.abs().clamp(min=1) * (tol if dt != torch.float32 else 0) + 2e-6 * mass)).max().item(), 1.0, (dt, m, n, k, gelu))
        n2 = vec * rng.randint(1, 100)
        w2 = (torch.randn(k, n2, device=dev) * 0.05).to(dt)
        b2 = torch.randn(n2, device=dev).to(dt)
        ref2 = xl.float() @ w2.float() + b2.float()
        o2 = kernels.linear_rows_kn_forward(xl, w2, b2, False)
        mass2 = xl.float().abs() @ w2.float().abs() + 1
        report("linear_rows_kn", ((o2.float() - ref2).abs() / (ref2.abs().clamp(min=1) * (tol if dt != torch.float32 else 0) + 2e-6 * mass2)).max().item(), 1.0, (dt, m, n2, k))
        # decode attention
        d = rng.choice([32, 64, 128, 256])
        es = 4 if dt == torch.float32 else 2
        if d * es in (128, 256, 512, 1024):
            cap = rng.randint(1, 1500)
            last = rng.randint(0, cap - 1)
            win = rng.choice([0, 0, 1, 5, 100])
            bb, hh = rng.randint(1, 3), rng.randint(1, 20)
            q = torch.randn(bb, hh, 1, d, device=dev).to(dt)
            kk = torch.randn(bb, hh, cap, d, device=dev).to(dt)
            vv = torch.randn(bb, hh, cap, d, device=dev).to(dt)
            first = max(0, last - win + 1) if win else 0
            sc = (q.double() @ kk.double()[:, :, first:last + 1].transpose(-1, -2)) * 0.2
            refa = (torch.softmax(sc, -1) @ vv.double()[:, :, first:last + 1]).float()
            pos = torch.tensor([last], device=dev) if rng.random() < 0.5 else last
            oa = kernels.attention_decode_forward(q, kk, vv, pos, 0.2, win)
            report("attention_decode", (oa.float() - refa).abs().max().item(), tol * max(1.0, refa.abs().max().item()), (dt, bb, hh, cap, d, last, win))
        # attention over a whole prompt (16-bit only; drawn from a stream of its own, so that the
        # draws of the other families are the ones the longer runs covered)
        if dt != torch.float32:
            pd = rng_prompt.choice([64, 128, 256])
            ps = max(1, min(pick_len_from(rng_prompt), 3000))
            pb, ph = rng_prompt.randint(1, 2), rng_prompt.randint(1, 5)
            pscale = rng_prompt.choice([1.0, 0.125, pd ** -0.5])
            pq, pk, pvv = (torch.randn(pb, ph, ps, pd, device=dev).to(dt) for _ in range(3))
            ppad = None
            if ps % 4 == 0 and rng_prompt.random() < 0.5:
                plens = torch.randint(1, ps + 1, (pb,), device=dev)
                ppad = torch.where(torch.arange(ps, device=dev)[None] < plens[:, None], 0.0, -10000.0).float()
            if rng_prompt.random() < 0.3:  # merged-heads memory viewed as [B, H, S, D]
                pq, pk, pvv = (t.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3) for t in (pq, pk, pvv))
            w = pq.double() @ pk.double().transpose(-1, -2) * pscale
            if ppad is not None:
                w = w + ppad.double()[:, None, None, :]
            ii = torch.arange(ps, device=dev)
            pwin = rng_prompt.choice([0, 0, 1, 7, 64, 256])
            hidden = ii[None, :] > ii[:, None]
            if pwin:
                hidden = hidden | (ii[None, :] <= ii[:, None] - pwin)
            refp = torch.softmax(w.masked_fill(hidden, float("-inf")), -1) @ pvv.double()
            op = kernels.attention_prefill_forward(pq, pk, pvv, pscale, ppad, pwin)
            rel = 2.0 ** -11 if dt == torch.float16 else 2.0 ** -8   # output rounding + rounding of the probabilities
            report("attention_prefill", ((op.double() - refp).abs() - rel * (refp.abs() + pvv.abs().max().item())).max().item(),
                   1e-4, (dt, pb, ph, ps, pd, pscale, ppad is not None, pwin))
        # softmax + dropout in one pass, forward and backward (the mask is read off the output)
        if S <= 2048:
            p_drop = rng.choice([0.1, 0.5])
            seed_s, off_s = rng.randint(0, 2 ** 40), 4 * rng.randint(0, 2 ** 30)
            yd, stats = kernels.causal_softmax_dropout_forward(x, pad, scale, p_drop, seed_s, off_s)
            plain = torch.softmax((x.float() * scale + (0 if pad is None else pad[:, None, None, :]))
                                  .masked_fill(~(i[None, :] <= i[:, None]), float("-inf")), -1)
            kept = yd != 0
            report("dropout_softmax_fwd", ((yd.float() - plain * kept / (1 - p_drop)).abs()).max().item(),
                   tol / (1 - p_drop), (dt, b, h, S, p_drop))
            # where the mask says "kept" the probability may still have rounded to 0: use the mask of ones
            ones_keep = kernels.bias_dropout_add_forward(torch.ones(b * h * S, S, device=dev, dtype=dt), None, None,
                                                         p_drop, seed_s, off_s).view(b, h, S, S) != 0
            gd = torch.randn(b, h, S, S, device=dev).to(dt)
            gy = gd.float() * ones_keep / (1 - p_drop)
            want_dx = scale * plain * (gy - (gy * plain).sum(-1, keepdim=True))
            dxd = kernels.causal_softmax_dropout_backward(gd.clone(), x, stats, pad, scale, p_drop, seed_s, off_s)
            report("dropout_softmax_bwd", (dxd.float() - want_dx).abs().max().item(),
                   2 * tol * max(1.0, want_dx.abs().max().item()), (dt, b, h, S, p_drop))
        # masked softmax backward and bias-dropout backward
        gm = torch.randn(b, h, sq, sk, device=dev).to(dt)
        ymf = ym.float()
        want_m = scale * ymf * (gm.float() - (gm.float() * ymf).sum(-1, keepdim=True))
        dxm = kernels.scaled_masked_softmax_backward(gm.clone(), ym, scale)
        report("masked_bwd", (dxm.float() - want_m).abs().max().item(), tol * max(1.0, want_m.abs().max().item()),
               (dt, b, h, sq, sk))
        dxb, dbb = kernels.bias_dropout_add_backward(go, p, seed, off)
        want_b = go.float() * keep / (1 - p)
        report("bda_bwd", ((dxb.float() - want_b).abs() / want_b.abs().clamp(min=1)).max().item(), tol, (dt, rows, cols, p))
        report("bda_dbias", ((dbb.float() - want_b.sum(0)).abs() / (want_b.abs().sum(0) + 1)).max().item(),
               max(tol, 1e-5), (dt, rows, cols, p))
        # rotary embedding + split heads against the torch operators
        from oslo_amd.modeling_gptj import apply_rotary, rotary_tables
        rb, rs, rh, rd = rng.randint(1, 3), rng.randint(1, 70), rng.randint(1, 5), rng.choice([32, 64, 128])
        rot = rng.choice([0, 8, 16, rd])
        roff = rng.randint(0, 20)
        qkv = [torch.randn(rb, rs, rh, rd, device=dev).to(dt) for _ in range(3)]
        sin, cos = rotary_tables(max(rot, 2), rs + roff, dev)
        outs = kernels.rotary_qkv_forward(qkv[0], qkv[1], qkv[2], sin if rot else None, cos if rot else None, rot, roff)
        for t_in, t_out, rotated in zip(qkv, outs, (True, True, False)):
            ref = t_in.float()
            if rotated and rot:
                ref = torch.cat([apply_rotary(ref[..., :rot], sin, cos, roff), ref[..., rot:]], dim=-1)
            report("rotary", (t_out.float() - ref.permute(0, 2, 1, 3)).abs().max().item(),
                   tol * max(1.0, ref.abs().max().item()), (dt, rb, rs, rh, rd, rot, roff))
    assert not failures, failures[:5]
