"""The library under HIP graph capture: every entry point only enqueues kernels
on the caller's stream and allocates nothing, so a sequence of calls can be
captured once and replayed. The graph is replayed several times, with new input
data and eager work between the replays, and every replay is compared with the
eager result of the same calls."""

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def test_captured_sequence_replays_like_eager():
    from oslo_amd import _lib

    lib = _lib.load()
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    BF16 = 2
    b, h, s = 2, 4, 512
    rows, cols = 256, 1024
    bs, hs, d, rot = 2, 4, 64, 32

    g = torch.Generator(device=DEV).manual_seed(0)
    x = torch.empty(b, h, s, s, device=DEV, dtype=torch.bfloat16)
    go = torch.empty_like(x)
    a = torch.empty(rows, cols, device=DEV, dtype=torch.bfloat16)
    ga = torch.empty_like(a)
    bias = (torch.randn(cols, device=DEV, generator=g) * 0.02).bfloat16()
    q = torch.empty(bs, s, hs, d, device=DEV, dtype=torch.bfloat16)
    from oslo_amd.modeling_gptj import rotary_tables
    sin, cos = rotary_tables(rot, s, DEV)
    inputs = (x, go, a, ga, q)

    def fresh_inputs(seed):
        g.manual_seed(seed)
        for t in inputs:
            t.copy_(torch.randn(t.shape, device=DEV, generator=g) * 2)

    def outputs():
        return dict(
            y=torch.empty_like(x), yd=torch.empty_like(x), stats=torch.empty(b, h, s, 2, device=DEV),
            dx=torch.empty_like(x), dxd=torch.empty_like(x), act=torch.empty_like(a), da=torch.empty_like(a),
            dbias=torch.empty_like(bias), drop=torch.empty_like(a), ddrop=torch.empty_like(a),
            dbias2=torch.empty_like(bias), qo=torch.empty(bs, hs, s, d, device=DEV, dtype=torch.bfloat16),
            ws=torch.empty(lib.oslo_colsum_workspace_bytes(rows, cols) // 4, device=DEV))

    def enqueue(o):
        st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        rc = [
            lib.oslo_softmax_causal_fwd(P(o["y"]), P(x), None, 0.125, b, h, s, BF16, st),
            lib.oslo_softmax_causal_bwd(P(o["dx"]), P(go), P(o["y"]), 0.125, b * h, s, BF16, st),
            lib.oslo_softmax_causal_dropout_fwd(P(o["yd"]), P(o["stats"]), P(x), None, 0.125, 0.1, 77, 8,
                                                b, h, s, BF16, st),
            lib.oslo_softmax_causal_dropout_bwd(P(o["dxd"]), P(go), P(x), P(o["stats"]), None, 0.125, 0.1, 77, 8,
                                                b, h, s, BF16, st),
            lib.oslo_bias_gelu_fwd(P(o["act"]), P(a), P(bias), rows, cols, BF16, st),
            lib.oslo_bias_gelu_bwd(P(o["da"]), P(o["dbias"]), P(o["ws"]), P(ga), P(a), P(bias), rows, cols, BF16, st),
            lib.oslo_bias_dropout_add_fwd(P(o["drop"]), P(a), P(bias), P(ga), 0.1, 77, 12, rows, cols, BF16, st),
            lib.oslo_bias_dropout_add_bwd(P(o["ddrop"]), P(o["dbias2"]), P(o["ws"]), P(ga), 0.1, 77, 12,
                                          rows, cols, BF16, st),
            lib.oslo_rotary_qkv(P(o["qo"]), None, None, P(q), None, None, P(sin), P(cos), s,
                                bs, s, hs, d, 0, rot, 0, 0, BF16, st),
        ]
        assert all(r == 0 for r in rc), lib.oslo_last_error().decode()

    fresh_inputs(1)
    captured = outputs()
    enqueue(captured)               # warm-up outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        enqueue(captured)

    for replay in range(4):
        fresh_inputs(100 + replay)
        for t in captured.values():
            t.fill_(float("nan")) if t.is_floating_point() else t.zero_()
        graph.replay()
        torch.cuda.synchronize()
        eager = outputs()
        enqueue(eager)              # the program's own eager work between replays
        torch.cuda.synchronize()
        for name in captured:
            if name == "ws":
                continue
            assert torch.equal(captured[name], eager[name]), f"replay {replay}: {name} differs from eager"
            assert not torch.isnan(captured[name].float()).any(), f"replay {replay}: {name} not written"


@pytest.mark.parametrize("d,padded", [(256, False), (64, True)])
def test_prompt_attention_captured(d, padded):
    """The one-kernel prompt attention under capture (at head_dim 256 its launcher
    also raises the kernel's LDS limit, a host-side setting): replays on new
    inputs equal the eager results."""
    from oslo_amd import kernels

    q, k, v = (torch.randn(2, 4, 300, d, device=DEV).bfloat16() for _ in range(3))
    pad = None
    if padded:
        pad = torch.zeros(2, 300, device=DEV)
        pad[1, 250:] = -10000.0
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = kernels.attention_prefill_forward(q, k, v, 0.0625, pad)
    for replay in range(3):
        for t in (q, k, v):
            t.copy_(torch.randn_like(t))
        out.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        eager = kernels.attention_prefill_forward(q, k, v, 0.0625, pad)   # eager work between replays
        assert torch.equal(out, eager), f"replay {replay} differs from eager"
        assert torch.isfinite(out).all()


@pytest.mark.parametrize("family", ["gpt2", "gptj", "gpt_neo"])
def test_graphed_forward_of_a_fused_model(family):
    """The whole fused forward captured once and replayed with new token ids and
    padding masks; every replay equals the eager forward bit for bit, with eager
    work between the replays."""
    from oslo_amd import (GPT2Config, GPT2LMHeadModel, GPTJConfig, GPTJForCausalLM, GPTNeoConfig,
                          GPTNeoForCausalLM, GraphedForward)

    torch.manual_seed(0)
    make = {
        "gpt2": lambda: GPT2LMHeadModel(GPT2Config(vocab_size=512, n_positions=128, n_embd=128, n_layer=2, n_head=4)),
        "gptj": lambda: GPTJForCausalLM(GPTJConfig(vocab_size=512, n_positions=128, n_embd=128, n_layer=2, n_head=4,
                                                   rotary_dim=16)),
        "gpt_neo": lambda: GPTNeoForCausalLM(GPTNeoConfig(vocab_size=512, max_position_embeddings=128,
                                                          hidden_size=128, num_layers=2, num_heads=4,
                                                          window_size=32)),
    }[family]
    model = make().half().to(DEV).eval().fuse()
    b, s = 3, 96

    def batch(seed):
        g = torch.Generator(device=DEV).manual_seed(seed)
        ids = torch.randint(0, 512, (b, s), device=DEV, generator=g)
        lens = torch.randint(s // 2, s + 1, (b,), device=DEV, generator=g)
        mask = (torch.arange(s, device=DEV)[None, :] < lens[:, None]).to(torch.int64)
        return ids, mask

    ids, mask = batch(1)
    graphed = GraphedForward(model, ids, attention_mask=mask)
    for replay in range(4):
        ids, mask = batch(10 + replay)
        got = graphed(ids, attention_mask=mask)["logits"].clone()
        with torch.no_grad():
            want = model(ids, attention_mask=mask)["logits"]      # eager work between replays
        assert torch.equal(got, want), f"{family} replay {replay}"
    with pytest.raises(RuntimeError, match="captured for"):
        graphed(ids[:, :50], attention_mask=mask[:, :50])
    with pytest.raises(RuntimeError, match="eval"):
        GraphedForward(model.train(), ids, attention_mask=mask)


def test_kernels_follow_torchs_current_stream():
    """Inside ``torch.cuda.stream(side)`` the launches go to ``side``: the
    stream handed to the library is the one torch reports, and work queued on
    that stream before the call (a fill of the input) is seen by the kernel."""
    from oslo_amd import kernels

    side = torch.cuda.Stream(device=DEV)
    x = torch.zeros(4, 8, 256, 256, device=DEV, dtype=torch.float16)
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        assert kernels._stream(x).value == torch.cuda.current_stream(x.device).cuda_stream == side.cuda_stream
        for _ in range(20):                       # keep the side stream busy ahead of the fill
            x.mul_(1.0)
        x.fill_(3.0)                              # equal scores: every visible key gets 1 / (row + 1)
        y = kernels.causal_softmax_forward(x, None, 1.0)
    side.synchronize()
    row = torch.arange(1, 257, device=DEV, dtype=torch.float32)
    want = torch.tril(torch.ones(256, 256, device=DEV)) / row[:, None]
    assert (y[2, 5].float() - want).abs().max() <= 2e-3
