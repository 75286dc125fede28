"""``model.generate``: the decoding loop against the installed transformers'
own ``generate`` on the same weights (CPU, unfused model), and on the GPU the
reference's kernel-fusion test (tests/gpt2/gpt2_test_kernel_fusion.py:26-49):
the same tokens before and after ``fuse()``, with the host and the fused
n-gram ban."""

import pytest
import torch

from oslo_amd import GPT2Config, GPT2LMHeadModel, GPTJConfig, GPTJForCausalLM, GPTNeoConfig, GPTNeoForCausalLM

VOCAB = 97


def tiny_gpt2(scale=8.0, seed=0):
    torch.manual_seed(seed)
    cfg = GPT2Config(vocab_size=VOCAB, n_positions=64, n_embd=32, n_layer=2, n_head=4,
                     resid_pdrop=0.0, embd_pdrop=0.0, attn_pdrop=0.0)
    model = GPT2LMHeadModel(cfg).eval()
    with torch.no_grad():  # larger weights: a peaked distribution, so that sequences end
        for p in model.parameters():
            if p.dim() > 1:
                p.mul_(scale)
    return model


def hf_twin(model):
    import transformers

    transformers.logging.set_verbosity_error()
    cfg = transformers.GPT2Config(vocab_size=VOCAB, n_positions=64, n_embd=32, n_layer=2, n_head=4,
                                  resid_pdrop=0.0, embd_pdrop=0.0, attn_pdrop=0.0, bos_token_id=0, eos_token_id=None)
    twin = transformers.GPT2LMHeadModel(cfg).eval()
    missing = twin.load_state_dict(model.state_dict(), strict=False)
    assert not missing.missing_keys
    return twin


# settings under which the installed transformers decodes by the same rule as the
# reference's (older) one; it differs where finished hypotheses of different
# lengths compete with length_penalty 1 (it normalises by generated length)
SETTINGS = [
    dict(max_length=30),
    dict(max_length=30, no_repeat_ngram_size=2),
    dict(max_length=30, num_beams=3),
    dict(max_length=30, min_length=30, num_beams=4, no_repeat_ngram_size=3),
    dict(max_length=30, eos_token_id=7, pad_token_id=0),
    dict(max_length=30, min_length=12, eos_token_id=7, pad_token_id=0, num_beams=4),
    dict(max_length=40, eos_token_id=11, pad_token_id=0, num_beams=2, length_penalty=2.0),
]


@pytest.mark.parametrize("kw", SETTINGS, ids=lambda kw: "-".join(f"{k}{v}" for k, v in kw.items()))
def test_generate_matches_transformers(kw):
    model = tiny_gpt2()
    twin = hf_twin(model)
    ids = torch.randint(1, VOCAB, (3, 5), generator=torch.Generator().manual_seed(1))
    with torch.no_grad():
        assert (twin(ids).logits - model(ids)["logits"]).abs().max() < 1e-4
    got = model.generate(ids, **kw)
    hf_kw = dict(kw)
    hf_kw.setdefault("pad_token_id", 0)
    want = twin.generate(ids, do_sample=False, early_stopping=False, **hf_kw)
    assert got.shape == want.shape and torch.equal(got, want)


def test_generate_without_cache_and_errors():
    model = tiny_gpt2()
    ids = torch.randint(1, VOCAB, (2, 4), generator=torch.Generator().manual_seed(2))
    for kw in (dict(max_length=20), dict(max_length=20, num_beams=3, no_repeat_ngram_size=2)):
        assert torch.equal(model.generate(ids, use_cache=True, **kw), model.generate(ids, use_cache=False, **kw))
    with pytest.raises(ValueError):
        model.generate(ids, max_length=4)
    with pytest.raises(ValueError):
        model.generate(ids[0], max_length=10)
    with pytest.raises(ValueError):
        model.generate(ids, max_length=10, num_beams=0)
    # on the host the "fused" processor takes its host branch, as the reference's does: the same tokens
    kw = dict(max_length=12, num_beams=2, no_repeat_ngram_size=2)
    assert torch.equal(model.generate(ids, fused_no_repeat_ngram_blocking=True, **kw), model.generate(ids, **kw))


def test_beam_search_finished_hypotheses():
    """A sequence that ends early is returned with its closing token and padding,
    and beats running beams by score / length."""
    model = tiny_gpt2()
    ids = torch.randint(1, VOCAB, (3, 5), generator=torch.Generator().manual_seed(1))
    out = model.generate(ids, max_length=40, min_length=8, eos_token_id=11, pad_token_id=0, num_beams=5,
                         no_repeat_ngram_size=2)
    assert out.shape[0] == 3 and out.shape[1] <= 40
    assert torch.equal(out[:, :5], ids)
    for row in out.tolist():
        if 11 in row[5:]:
            end = row.index(11, 5)
            assert end >= 8 and all(t == 0 for t in row[end + 1:])
        bigrams = list(zip(row, row[1:]))
        body = bigrams[: (row.index(11, 5) if 11 in row[5:] else len(row)) - 1]
        assert len(set(body)) == len(body)       # no bigram twice


FAMILIES = {
    "gpt2": lambda: GPT2LMHeadModel(GPT2Config(vocab_size=211, n_positions=128, n_embd=64, n_layer=2, n_head=4,
                                               resid_pdrop=0.0, embd_pdrop=0.0, attn_pdrop=0.0)),
    "gpt_neo": lambda: GPTNeoForCausalLM(GPTNeoConfig(vocab_size=211, max_position_embeddings=128, hidden_size=64,
                                                      num_layers=2, num_heads=4, window_size=16,
                                                      resid_dropout=0.0, embed_dropout=0.0, attention_dropout=0.0)),
    "gptj": lambda: GPTJForCausalLM(GPTJConfig(vocab_size=211, n_positions=128, n_embd=64, n_layer=2, n_head=4,
                                               rotary_dim=8, resid_pdrop=0.0, embd_pdrop=0.0, attn_pdrop=0.0)),
}


def family_model(family):
    torch.manual_seed(3)
    model = FAMILIES[family]().eval()
    with torch.no_grad():
        for p in model.parameters():
            if p.dim() > 1:
                p.mul_(4.0)
    return model


DECODING = [dict(max_length=50), dict(max_length=50, min_length=50, num_beams=3, no_repeat_ngram_size=2),
            dict(max_length=50, min_length=10, num_beams=3, eos_token_id=5)]


@pytest.mark.parametrize("family", sorted(FAMILIES))
def test_static_cache_decodes_the_same_tokens(family):
    """Preallocated caches under a key mask (GPT-Neo's window is longer than
    its local layers' 16 keys here) against caches grown by concatenation."""
    model = family_model(family)
    ids = torch.randint(1, 211, (2, 6), generator=torch.Generator().manual_seed(4))
    for kw in DECODING:
        want = model.generate(ids, **kw)
        got = model.generate(ids, static_cache=True, **kw)
        assert got.shape == want.shape and torch.equal(got, want), kw
    with pytest.raises(ValueError):
        model.generate(ids, max_length=20, static_cache=True, use_cache=False)
    with pytest.raises(RuntimeError):   # graphs are a device feature
        model.generate(ids, max_length=20, graph=True)


@pytest.mark.gpu
@pytest.mark.parametrize("family", sorted(FAMILIES))
def test_graphed_decoding_same_tokens(family):
    """One HIP graph replay per token (fused model) against the step-by-step
    decoding of the unfused model."""
    model = family_model(family).cuda()
    ids = torch.randint(1, 211, (2, 6), generator=torch.Generator().manual_seed(4)).cuda()
    want = [model.generate(ids, **kw) for kw in DECODING]
    model = model.fuse()
    for kw, w in zip(DECODING, want):
        for extra in (dict(static_cache=True), dict(graph=True)):
            got = model.generate(ids, **kw, **extra)
            assert got.shape == w.shape and torch.equal(got, w), (kw, extra)
    # a second prompt reuses the captured steps of the first (same shapes); another batch size does not
    kept = model._kept_decoder[1]
    ids2 = torch.randint(1, 211, (2, 6), generator=torch.Generator().manual_seed(5)).cuda()
    ids3 = torch.randint(1, 211, (3, 9), generator=torch.Generator().manual_seed(6)).cuda()
    for other in (ids2, ids3, ids):
        for kw in DECODING[:2]:
            assert torch.equal(model.generate(other, graph=True, **kw), model.generate(other, **kw)), kw
        assert model._kept_decoder[1] is kept
    # the step that is captured may carry any beam permutation: it is applied once
    from oslo_amd import DynamicDecoder, StaticDecoder
    rows = ids.repeat_interleave(3, dim=0)
    with torch.no_grad():
        dyn, sta = DynamicDecoder(model, True), StaticDecoder(model, 64, True)
        assert torch.allclose(dyn.step(rows), sta.step(rows), atol=1e-5)
        perm = torch.tensor([2, 0, 1, 5, 3, 4], device=rows.device)
        grown = torch.cat([rows[perm], rows[:, :1]], dim=1)
        for _ in range(3):
            want_logits, got_logits = dyn.step(grown, perm), sta.step(grown, perm)
            assert torch.allclose(want_logits, got_logits, atol=1e-4)
            grown = torch.cat([grown[perm], grown[:, :1]], dim=1)
    # the fused ban reads the growing token tensor outside the graph
    kw = dict(max_length=50, min_length=50, num_beams=3, no_repeat_ngram_size=2)
    assert torch.equal(model.generate(ids, graph=True, fused_no_repeat_ngram_blocking=True, **kw), want[1])
    model.release_decoder()
    assert "_kept_decoder" not in model.__dict__
    assert torch.equal(model.generate(ids, graph=True, **DECODING[1]), want[1])
    kept = model._kept_decoder[1]
    # new storage for the weights: the kept graph would read the old one, so it is dropped
    model = model.double().float()
    assert torch.equal(model.generate(ids, graph=True, **DECODING[1]), want[1])
    assert model._kept_decoder[1] is not kept
    model.train()
    with pytest.raises(RuntimeError):
        model.generate(ids, max_length=20, graph=True)


@pytest.mark.gpu
@pytest.mark.parametrize("family", sorted(FAMILIES))
def test_generate_same_tokens_before_and_after_fuse(family):
    model = family_model(family).cuda()
    ids = torch.randint(1, 211, (2, 6), generator=torch.Generator().manual_seed(4)).cuda()
    kw = dict(max_length=60, min_length=60, num_beams=5, no_repeat_ngram_size=4)
    before = model.generate(ids, **kw)
    greedy_before = model.generate(ids, max_length=40)
    model = model.fuse()
    after = model.generate(ids, **kw)
    after_fused_ban = model.generate(ids, fused_no_repeat_ngram_blocking=True, **kw)
    assert before.shape == (2, 60)
    assert torch.equal(before, after)
    assert torch.equal(before, after_fused_ban)
    assert torch.equal(greedy_before, model.generate(ids, max_length=40))
    # the switch can also come from the configuration (oslo/generation_utils.py:753-757)
    model.config.fused_no_repeat_ngram_blocking = True
    assert torch.equal(before, model.generate(ids, **kw))
