"""Host-side behaviour of the operator API and of model.fuse(), no GPU needed:
the availability gate, the class swap, argument errors, and the rule that
nothing computes on the CPU."""

import itertools

import pytest
import torch

import oslo_amd
from oracle import oslo_oracle as orc
from oracle import unfused_torch as ref
from oslo_amd import (FusedBiasActivation, FusedBiasDropout, FusedScaleMaskSoftmax, GPT2Config,
                      GPT2LMHeadModel, GPTJConfig, GPTJForCausalLM, GPTNeoConfig, GPTNeoForCausalLM)
from oslo_amd import modeling_gpt2, modeling_gpt_neo, modeling_gptj


def tiny_gpt2():
    return GPT2LMHeadModel(GPT2Config(vocab_size=97, n_positions=32, n_embd=32, n_layer=2, n_head=4))


def tiny_gptj():
    return GPTJForCausalLM(GPTJConfig(vocab_size=97, n_positions=32, n_embd=32, n_layer=2, n_head=4, rotary_dim=4))


def tiny_neo():
    return GPTNeoForCausalLM(GPTNeoConfig(vocab_size=97, max_position_embeddings=32, hidden_size=32,
                                           num_layers=2, num_heads=4, window_size=8))


def test_gate_is_a_superset_of_the_reference_gate():
    avail = FusedScaleMaskSoftmax.is_available
    for bsz, np_, sq, sk, tri in itertools.product((1, 2, 3, 8), (1, 3, 12, 16),
                                                   (1, 2, 6, 63, 64, 128, 1024, 2048),
                                                   (1, 63, 64, 66, 128, 1024, 2048), (True, False)):
        if orc.reference_is_available(True, bsz, np_, sq, sk, tri):
            assert avail(torch.half, bsz, np_, sq, sk, tri), (bsz, np_, sq, sk, tri)
    # and the widening: bf16, fp32, long rows, no divisibility rules
    assert avail(torch.bfloat16, 8, 16, 2048, 2048, True)
    assert avail(torch.float32, 1, 3, 1000, 1000, True)
    assert avail(torch.half, 1, 16, 8192, 8192, True)
    assert avail(torch.half, 2, 4, 5, 1024, False)
    # still refused
    assert not avail(torch.half, 1, 16, 8200, 8200, True)       # longer than the kernels hold
    assert not avail(torch.half, 8, 16, 1, 2048, True)          # decode step: causal needs sq == sk
    assert not avail(torch.float64, 8, 16, 128, 128, True)
    assert not avail(torch.half, 8, 16, 128, 0, False)


def test_get_custom_kernels_exposes_the_reference_symbols():
    k = oslo_amd.get_custom_kernels()
    for name in ("scaled_masked_softmax_forward", "scaled_masked_softmax_backward", "get_batch_per_block",
                 "scaled_upper_triang_masked_softmax_forward", "scaled_upper_triang_masked_softmax_backward"):
        assert callable(getattr(k, name))
    assert k.get_batch_per_block(2048, 2048, 8, 16) == 4


def test_nothing_computes_on_the_cpu():
    x = torch.randn(1, 2, 8, 8)
    with pytest.raises(RuntimeError, match="no CPU path"):
        FusedScaleMaskSoftmax.apply(x, None, 1.0, True)
    with pytest.raises(RuntimeError, match="no CPU path"):
        FusedScaleMaskSoftmax.apply(x, None, 1.0, False)
    with pytest.raises(RuntimeError, match="no CPU path"):
        FusedBiasActivation.apply(torch.randn(4, 8), torch.zeros(8), "gelu_new")
    with pytest.raises(RuntimeError, match="no CPU path"):
        FusedBiasDropout.apply(torch.randn(4, 8), torch.zeros(8), True, 0.1)
    # a fused model on the CPU fails the same way instead of silently running something else
    m = tiny_gpt2().fuse().eval()
    with pytest.raises(RuntimeError, match="no CPU path"):
        m(torch.randint(0, 97, (2, 8)))


def test_non_gelu_activation_is_the_unfused_expression():
    x, b = torch.randn(4, 8), torch.randn(8)
    torch.testing.assert_close(FusedBiasActivation.apply(x, b, "relu"), torch.relu(x + b))


def test_pad_mask_shape_is_checked():
    with pytest.raises(RuntimeError, match="pad_mask"):
        FusedScaleMaskSoftmax.apply(torch.randn(2, 2, 8, 8), torch.zeros(2, 1, 8, 8), 1.0, True)


def test_pad_mask_conversion_on_the_host():
    """The [B,1,1,Sk] -> fp32 [B,Sk] conversion needs no device: bool and float
    forms, broadcasting over the batch, reuse while the tensor is unchanged, a
    fresh conversion after an in-place change, and masks made under
    torch.inference_mode(), which have no version counter to consult."""
    from oslo_amd import fused_kernels_utils as fku
    m = torch.zeros(2, 1, 1, 8)
    m[1, :, :, 5:] = -10000.0
    a = fku._pad_additive_f32(m, 2, 8)
    assert a.dtype == torch.float32 and torch.equal(a, m.view(2, 8))
    assert fku._pad_additive_f32(m, 2, 8) is a
    m[0, :, :, 2:] = -10000.0
    b = fku._pad_additive_f32(m, 2, 8)
    assert b is not a and torch.equal(b, m.view(2, 8))
    bm = torch.zeros(1, 1, 1, 8, dtype=torch.bool)
    bm[..., 6:] = True
    c = fku._pad_additive_f32(bm, 3, 8)
    assert c.shape == (3, 8) and torch.equal(c[2], torch.tensor([0.0] * 6 + [-10000.0] * 2))
    with torch.inference_mode():
        im = torch.zeros(2, 1, 1, 8)
        im[0, :, :, 4:] = -10000.0
        d = fku._pad_additive_f32(im, 2, 8)
        assert torch.equal(d, im.view(2, 8))
        im[1, :, :, 1:] = -10000.0          # invisible to a version counter: must not be served from a cache
        assert torch.equal(fku._pad_additive_f32(im, 2, 8), im.view(2, 8))
    # a malformed mask is rejected even when a well-formed one was converted just before
    with pytest.raises(RuntimeError, match="pad_mask"):
        fku._pad_additive_f32(torch.zeros(2, 1, 8, 8), 2, 8)


@pytest.mark.parametrize("make,mods,fused", [
    (tiny_gpt2, (modeling_gpt2.GPT2Attention, modeling_gpt2.GPT2MLP),
     (modeling_gpt2.FusedGPT2Attention, modeling_gpt2.FusedGPT2MLP)),
    (tiny_gptj, (modeling_gptj.GPTJAttention, modeling_gptj.GPTJMLP),
     (modeling_gptj.FusedGPTJAttention, modeling_gptj.FusedGPTJMLP)),
    (tiny_neo, (modeling_gpt_neo.GPTNeoSelfAttention, modeling_gpt_neo.GPTNeoMLP),
     (modeling_gpt_neo.FusedGPTNeoSelfAttention, modeling_gpt_neo.FusedGPTNeoMLP)),
])
def test_fuse_swaps_classes_and_nothing_else(make, mods, fused):
    m = make()
    before = {k: v.clone() for k, v in m.state_dict().items()}
    n_attn = sum(type(x) is mods[0] for x in m.modules())
    n_mlp = sum(type(x) is mods[1] for x in m.modules())
    assert n_attn >= 1 and n_mlp == 2
    assert m.fuse() is m
    assert sum(type(x) is fused[0] for x in m.modules()) == n_attn
    assert sum(type(x) is fused[1] for x in m.modules()) == n_mlp
    assert not any(type(x) in mods for x in m.modules())
    after = m.state_dict()
    assert list(after) == list(before)
    for k in before:
        assert torch.equal(before[k], after[k]), k
    for x in m.modules():
        if type(x) in fused:
            assert x.config is m.config


def test_fuse_modules_filter_and_errors():
    m = tiny_gpt2().fuse(modules=[modeling_gpt2.GPT2MLP])
    assert sum(type(x) is modeling_gpt2.FusedGPT2MLP for x in m.modules()) == 2
    assert sum(type(x) is modeling_gpt2.GPT2Attention for x in m.modules()) == 2      # left alone
    with pytest.raises(AssertionError, match="List"):
        tiny_gpt2().fuse(modules=modeling_gpt2.GPT2MLP)
    with pytest.raises(AssertionError, match="can't be fused"):
        tiny_gpt2().fuse(modules=[torch.nn.LayerNorm])

    class Plain(oslo_amd.modeling_utils.PreTrainedModel):
        pass

    with pytest.raises(RuntimeError, match="doesn't support kernel fusion"):
        Plain(None).fuse()


def test_blocks_are_fused_unless_the_reference_selection_is_asked_for():
    """fuse() also swaps the blocks (their residual additions go into the fused
    modules); the reference's own selection leaves them alone, and so does a
    partial one, whose unfused child the fused block could not hand a residual."""
    for make, block, fused_block, selection in (
            (tiny_gpt2, modeling_gpt2.GPT2Block, modeling_gpt2.FusedGPT2Block,
             [modeling_gpt2.GPT2Attention, modeling_gpt2.GPT2MLP]),
            (tiny_gptj, modeling_gptj.GPTJBlock, modeling_gptj.FusedGPTJBlock,
             [modeling_gptj.GPTJAttention, modeling_gptj.GPTJMLP]),
            (tiny_neo, modeling_gpt_neo.GPTNeoBlock, modeling_gpt_neo.FusedGPTNeoBlock,
             [modeling_gpt_neo.GPTNeoSelfAttention, modeling_gpt_neo.GPTNeoMLP])):
        m = make().fuse()
        assert all(type(b) is fused_block for b in m.transformer.h) and m.fused_lm_head
        m = make().fuse(modules=selection)
        assert all(type(b) is block for b in m.transformer.h) and not m.fused_lm_head
        # a fused block may sit over an unfused child (it then runs the plain block's code)
        m = make().fuse(modules=[selection[1], block])
        assert all(type(b) is fused_block for b in m.transformer.h)
        assert not any(type(x) in (modeling_gpt2.FusedGPT2Attention, modeling_gptj.FusedGPTJAttention,
                                   modeling_gpt_neo.FusedGPTNeoSelfAttention) for x in m.modules())


def test_gpt_neo_local_attention_has_a_fused_class_of_its_own():
    m = tiny_neo().fuse()
    kinds = [type(b.attn.attention) for b in m.transformer.h]
    assert kinds == [modeling_gpt_neo.FusedGPTNeoSelfAttention, modeling_gpt_neo.FusedGPTNeoLocalSelfAttention]
    assert isinstance(m.transformer.h[1].attn.attention, modeling_gpt_neo.GPTNeoLocalSelfAttention)
    # the reference's behaviour (local layers left alone) is one filter away
    m = tiny_neo().fuse(modules=[modeling_gpt_neo.GPTNeoSelfAttention, modeling_gpt_neo.GPTNeoMLP])
    kinds = [type(b.attn.attention) for b in m.transformer.h]
    assert kinds == [modeling_gpt_neo.FusedGPTNeoSelfAttention, modeling_gpt_neo.GPTNeoLocalSelfAttention]


def test_unfused_models_run_on_cpu_and_use_the_reference_attention():
    torch.manual_seed(0)
    for make in (tiny_gpt2, tiny_gptj, tiny_neo):
        m = make().eval()
        ids = torch.randint(0, 97, (2, 16))
        mask = torch.ones(2, 16)
        mask[1, 10:] = 0
        out = m(ids, attention_mask=mask, labels=ids)
        assert out["logits"].shape == (2, 16, 97) and torch.isfinite(out["loss"])
    # GPT-2 attention probabilities equal the unfused restatement on the same scores
    att = tiny_gpt2().eval().transformer.h[0].attn
    q, k, v = (torch.randn(2, 4, 16, 8) for _ in range(3))
    add = torch.zeros(2, 1, 1, 16)
    add[1, :, :, 12:] = -10000.0
    _, w = att._attn(q, k, v, add)
    want = ref.attention_probs(q @ k.transpose(-1, -2), 1 / 8 ** 0.5, True, add, masked_bias=-1e4)
    torch.testing.assert_close(w, want)


def test_kv_cache_decode_matches_full_forward_unfused():
    torch.manual_seed(1)
    for make in (tiny_gpt2, tiny_gptj, tiny_neo):
        m = make().eval()
        ids = torch.randint(0, 97, (2, 12))
        full = m(ids)["logits"]
        first = m(ids[:, :11], use_cache=True)
        step = m(ids[:, 11:], past_key_values=first["past_key_values"], use_cache=True)
        torch.testing.assert_close(step["logits"][:, 0], full[:, 11], rtol=1e-4, atol=1e-4)
