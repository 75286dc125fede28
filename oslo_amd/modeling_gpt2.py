"""GPT-2 blocks with the reference's kernel-fusion hooks.

``GPT2Attention`` / ``GPT2MLP`` compute what the reference's unfused modules
compute (oslo/models/gpt2/modeling_gpt2.py:131-230, :385-399);
``FusedGPT2Attention`` / ``FusedGPT2MLP`` are the classes ``fuse()`` swaps in
(oslo/models/gpt2/modeling_gpt2.py:1434-1569). Sub-module and buffer names
(c_attn, c_proj, c_fc, attn_dropout, resid_dropout, bias, masked_bias) are the
reference's, so a state_dict moves between the two unchanged."""

from dataclasses import dataclass
from typing import Optional

import torch
from torch import nn

from .fused_kernels_utils import (FusedBiasActivation, FusedBiasDropout, FusedBiasDropoutResidual,
                                 FusedDecodeAttention, FusedLinearBiasActivation, FusedLinearRows, FusedPrefillAttention,
                                 FusedMergeHeads,
                                 FusedScaleMaskSoftmax,
                                 FusedScaleMaskSoftmaxDropout, FusedSplitHeads)
from .modeling_utils import (ACT2FN, Conv1D, LayerPolicy, PreTrainedModel, StaticKV, additive_attention_mask,
                             append_kv, causal_lm_loss, static_cache_mask)


@dataclass
class GPT2Config:
    vocab_size: int = 50257
    n_positions: int = 1024
    n_embd: int = 768
    n_layer: int = 12
    n_head: int = 12
    n_inner: Optional[int] = None
    activation_function: str = "gelu_new"
    resid_pdrop: float = 0.1
    embd_pdrop: float = 0.1
    attn_pdrop: float = 0.1
    layer_norm_epsilon: float = 1e-5
    scale_attn_weights: bool = True
    scale_attn_by_inverse_layer_idx: bool = False
    add_cross_attention: bool = False

    @property
    def hidden_size(self):
        return self.n_embd

    @property
    def num_attention_heads(self):
        return self.n_head

    @property
    def max_position_embeddings(self):
        return self.n_positions


class GPT2Attention(nn.Module):
    def __init__(self, config, is_cross_attention=False, layer_idx=None):
        super().__init__()
        n_pos = config.max_position_embeddings
        self.register_buffer(
            "bias", torch.tril(torch.ones((n_pos, n_pos), dtype=torch.uint8)).view(1, 1, n_pos, n_pos))
        self.register_buffer("masked_bias", torch.tensor(-1e4))
        self.embed_dim = config.hidden_size
        self.num_heads = config.num_attention_heads
        self.head_dim = self.embed_dim // self.num_heads
        self.split_size = self.embed_dim
        if self.head_dim * self.num_heads != self.embed_dim:
            raise ValueError("`embed_dim` must be divisible by num_heads")
        self.scale_attn_weights = config.scale_attn_weights
        self.scale_attn_by_inverse_layer_idx = config.scale_attn_by_inverse_layer_idx
        self.is_cross_attention = is_cross_attention
        self.layer_idx = layer_idx
        if is_cross_attention:
            self.c_attn = Conv1D(2 * self.embed_dim, self.embed_dim)
            self.q_attn = Conv1D(self.embed_dim, self.embed_dim)
        else:
            self.c_attn = Conv1D(3 * self.embed_dim, self.embed_dim)
        self.c_proj = Conv1D(self.embed_dim, self.embed_dim)
        self.attn_dropout = nn.Dropout(config.attn_pdrop)
        self.resid_dropout = nn.Dropout(config.resid_pdrop)

    def _split_heads(self, t, num_heads, head_dim):
        return t.view(t.size()[:-1] + (num_heads, head_dim)).permute(0, 2, 1, 3)

    def _merge_heads(self, t, num_heads, head_dim):
        t = t.permute(0, 2, 1, 3).contiguous()
        return t.view(t.size()[:-2] + (num_heads * head_dim,))

    def _attention_scale(self, value):
        scale = 1.0
        if self.scale_attn_weights:
            scale *= 1 / (float(value.size(-1)) ** 0.5)
        if self.scale_attn_by_inverse_layer_idx:
            scale *= 1 / float(self.layer_idx + 1)
        return scale

    def _attn(self, query, key, value, attention_mask=None, head_mask=None, causal=True):
        """The unfused path: scale, where(causal, w, -1e4), + mask, softmax, dropout."""
        w = torch.matmul(query, key.transpose(-1, -2))
        if self.scale_attn_weights:
            w = w / (float(value.size(-1)) ** 0.5)
        if self.scale_attn_by_inverse_layer_idx:
            w = w / float(self.layer_idx + 1)
        if causal and not self.is_cross_attention:
            sq, sk = query.size(-2), key.size(-2)
            causal = self.bias[:, :, sk - sq:sk, :sk].bool()
            w = torch.where(causal, w, self.masked_bias.to(w.dtype))
        if attention_mask is not None:
            w = w + attention_mask
        w = nn.functional.softmax(w, dim=-1)
        w = self.attn_dropout(w.type(value.dtype))
        if head_mask is not None:
            w = w * head_mask
        return torch.matmul(w, value), w

    def _project_qkv(self, hidden_states, layer_past, encoder_hidden_states, use_cache):
        if encoder_hidden_states is not None:
            if not hasattr(self, "q_attn"):
                raise ValueError("cross attention needs GPT2Attention(..., is_cross_attention=True)")
            query = self.q_attn(hidden_states)
            key, value = self.c_attn(encoder_hidden_states).split(self.split_size, dim=2)
        else:
            query, key, value = self.c_attn(hidden_states).split(self.split_size, dim=2)
        query = self._split_heads(query, self.num_heads, self.head_dim)
        key = self._split_heads(key, self.num_heads, self.head_dim)
        value = self._split_heads(value, self.num_heads, self.head_dim)
        key, value, present = append_kv(layer_past, key, value, use_cache)
        return query, key, value, present

    def forward(self, hidden_states, layer_past=None, attention_mask=None, head_mask=None,
                encoder_hidden_states=None, encoder_attention_mask=None, use_cache=False,
                output_attentions=False):
        query, key, value, present = self._project_qkv(hidden_states, layer_past, encoder_hidden_states, use_cache)
        if encoder_hidden_states is not None:
            attention_mask = encoder_attention_mask
        static = isinstance(layer_past, StaticKV)
        if static:
            attention_mask = static_cache_mask(layer_past, attention_mask, fused=False)
        out, w = self._attn(query, key, value, attention_mask, head_mask, causal=not static)
        out = self._merge_heads(out, self.num_heads, self.head_dim)
        out = self.resid_dropout(self.c_proj(out))
        return (out, present, w) if output_attentions else (out, present)


class FusedGPT2Attention(GPT2Attention):
    """oslo/models/gpt2/modeling_gpt2.py:1434-1542. The reference's fused
    attention leaves out attn_dropout, which its unfused attention applies
    (:222); here it is applied, inside the softmax kernel, so that fused and
    unfused training agree. Beyond the reference's fused class, the split of the
    packed c_attn projection with its three split-heads permutes, and the
    merge-heads permute, run through the transposition kernel instead of torch's
    strided copies."""

    def _project_qkv(self, hidden_states, layer_past, encoder_hidden_states, use_cache):
        if encoder_hidden_states is not None or not (
                hidden_states.is_cuda and FusedSplitHeads.is_available(hidden_states.dtype, self.head_dim)):
            return super()._project_qkv(hidden_states, layer_past, encoder_hidden_states, use_cache)
        # (a decoding step streams the weight in one pass, bias included)
        query, key, value = FusedSplitHeads.apply(FusedLinearRows.project_conv1d(self.c_attn, hidden_states),
                                                  self.num_heads)
        key, value, present = append_kv(layer_past, key, value, use_cache, defer=True)
        return query, key, value, present

    def _fused_attn(self, query, key, value, attention_mask=None, head_mask=None, causal=True):
        w = torch.matmul(query, key.transpose(-1, -2))
        w = FusedScaleMaskSoftmaxDropout.apply(w, attention_mask, self._attention_scale(value), causal,
                                               self.attn_dropout.p, self.training)
        if head_mask is not None:
            w = w * head_mask
        return torch.matmul(w, value), w

    def forward(self, hidden_states, layer_past=None, attention_mask=None, head_mask=None,
                encoder_hidden_states=None, encoder_attention_mask=None, use_cache=False,
                output_attentions=False, residual=None):
        """``residual``: added to the output (the residual connection of the
        block, which a decoding step takes into the projection's launch)."""
        query, key, value, present = self._project_qkv(hidden_states, layer_past, encoder_hidden_states, use_cache)
        if encoder_hidden_states is not None:
            attention_mask = encoder_attention_mask
        (bsz, np_, sq, _), sk = query.size(), key.size(-2)
        # a single query over a key/value cache (a decoding step) sees every key:
        # the causal mask is empty and the key-mask kernel applies
        causal = not self.is_cross_attention and sq > 1
        static = isinstance(layer_past, StaticKV)
        fused = FusedScaleMaskSoftmax.is_available(query.dtype, bsz, np_, sq, sk, use_triang_mask=causal)
        one_pass = (sq == 1 and not self.is_cross_attention and attention_mask is None and head_mask is None
                    and not output_attentions
                    and FusedDecodeAttention.is_available(query, key, self.training, self.attn_dropout.p))
        fresh = (None, None)  # the step's key and value, if not yet in a static cache
        if static and one_pass and layer_past.pending_is_dense():
            fresh = layer_past.take_pending()  # the kernel below writes them into their slot
        elif static:
            layer_past.flush()
        if static and not one_pass:
            attention_mask = static_cache_mask(layer_past, attention_mask, fused)
        prompt = (causal and not static and head_mask is None and not output_attentions
                  and FusedPrefillAttention.is_available(query, key, attention_mask, self.training,
                                                         self.attn_dropout.p))
        if one_pass:
            # a decoding step: scores, softmax and weighted sum in one pass over the cache
            out = FusedDecodeAttention.apply(query, key, value, layer_past.state.pos if static else sk - 1,
                                             self._attention_scale(value), None, *fresh)
            w = None
        elif prompt:
            # a whole prompt: one kernel, the scores stay on chip (in training too: it has a backward
            # and drops attention probabilities itself)
            out, w = FusedPrefillAttention.apply(query, key, value, attention_mask, self._attention_scale(value),
                                                 None, self.attn_dropout.p if self.training else 0.0), None
        elif fused:
            out, w = self._fused_attn(query, key, value, attention_mask, head_mask, causal)
        else:
            out, w = self._attn(query, key, value, attention_mask, head_mask, causal=not static)
        if out.is_cuda and FusedSplitHeads.is_available(out.dtype, self.head_dim):
            out = FusedMergeHeads.apply(out)
        else:
            out = self._merge_heads(out, self.num_heads, self.head_dim)
        if FusedLinearRows.is_available(out, self.c_proj.weight, self.c_proj.bias, conv1d=True) and not (
                self.training and self.resid_dropout.p > 0.0):
            out = FusedLinearRows.apply(out, self.c_proj.weight, self.c_proj.bias, conv1d=True,
                                        residual=residual)  # a decoding step
        else:
            out = out @ self.c_proj.weight  # projection without its bias, which is fused here:
            if residual is None:
                out = FusedBiasDropout.apply(out, self.c_proj.bias, self.training, self.resid_dropout.p)
            else:  # with the block's residual addition in the same pass
                out = FusedBiasDropoutResidual.apply(out, self.c_proj.bias, residual, self.training,
                                                     self.resid_dropout.p)
        return (out, present, w) if output_attentions else (out, present)


class GPT2MLP(nn.Module):
    def __init__(self, intermediate_size, config):
        super().__init__()
        self.c_fc = Conv1D(intermediate_size, config.hidden_size)
        self.c_proj = Conv1D(config.hidden_size, intermediate_size)
        self.act = ACT2FN[config.activation_function]
        self.dropout = nn.Dropout(config.resid_pdrop)

    def forward(self, hidden_states):
        return self.dropout(self.c_proj(self.act(self.c_fc(hidden_states))))


class FusedGPT2MLP(GPT2MLP):
    """oslo/models/gpt2/modeling_gpt2.py:1545-1569."""

    def forward(self, x, residual=None):
        """``residual``: added to the output (the residual connection of the block)."""
        if FusedLinearRows.is_available(x, self.c_fc.weight, self.c_fc.bias, conv1d=True) and \
                FusedLinearRows.is_available(None, self.c_proj.weight, self.c_proj.bias, conv1d=True, rows_of=x):
            # a decoding step: each projection is one pass over its weight with
            # the bias (and the activation, and the residual) applied to the fp32 sums
            x = FusedLinearRows.apply(x, self.c_fc.weight, self.c_fc.bias, self.config.activation_function,
                                      conv1d=True)
            if not (self.training and self.dropout.p > 0.0):
                return FusedLinearRows.apply(x, self.c_proj.weight, self.c_proj.bias, conv1d=True,
                                             residual=residual)
            x = FusedLinearRows.apply(x, self.c_proj.weight, conv1d=True)
        else:
            act = self.config.activation_function
            if FusedLinearBiasActivation.is_available(x, self.c_fc.weight, self.c_fc.bias, act):
                # bias and GeLU on the product's fp32 sums, in its own launch
                x = FusedLinearBiasActivation.apply(x, self.c_fc.weight, self.c_fc.bias, act, conv1d=True)
            else:
                x = x @ self.c_fc.weight
                x = FusedBiasActivation.apply(x, self.c_fc.bias, act)
            x = x @ self.c_proj.weight
        if residual is None:
            return FusedBiasDropout.apply(x, self.c_proj.bias, self.training, self.dropout.p)
        # bias, dropout and the block's residual addition in one pass
        return FusedBiasDropoutResidual.apply(x, self.c_proj.bias, residual, self.training, self.dropout.p)


class GPT2Block(nn.Module):
    def __init__(self, config, layer_idx=None):
        super().__init__()
        inner = config.n_inner if config.n_inner is not None else 4 * config.hidden_size
        self.ln_1 = nn.LayerNorm(config.hidden_size, eps=config.layer_norm_epsilon)
        self.attn = GPT2Attention(config, layer_idx=layer_idx)
        self.ln_2 = nn.LayerNorm(config.hidden_size, eps=config.layer_norm_epsilon)
        self.mlp = GPT2MLP(inner, config)

    def forward(self, hidden_states, layer_past=None, attention_mask=None, head_mask=None, use_cache=False):
        a = self.attn(self.ln_1(hidden_states), layer_past=layer_past, attention_mask=attention_mask,
                      head_mask=head_mask, use_cache=use_cache)
        hidden_states = a[0] + hidden_states
        hidden_states = hidden_states + self.mlp(self.ln_2(hidden_states))
        return hidden_states, a[1]


class FusedGPT2Block(GPT2Block):
    """The block with its two residual additions handed to the fused modules,
    which take them into their last projection's launch in a decoding step.
    No counterpart in the reference, which fuses attention and MLP only
    (oslo/models/gpt2/configuration_gpt2.py:272-284); the arithmetic is that
    of oslo/models/gpt2/modeling_gpt2.py:420-481."""

    def forward(self, hidden_states, layer_past=None, attention_mask=None, head_mask=None, use_cache=False):
        if not (isinstance(self.attn, FusedGPT2Attention) and isinstance(self.mlp, FusedGPT2MLP)):
            return super().forward(hidden_states, layer_past, attention_mask, head_mask, use_cache)
        a = self.attn(self.ln_1(hidden_states), layer_past=layer_past, attention_mask=attention_mask,
                      head_mask=head_mask, use_cache=use_cache, residual=hidden_states)
        hidden_states = self.mlp(self.ln_2(a[0]), residual=a[0])
        return hidden_states, a[1]


class GPT2LayerPolicy(LayerPolicy):
    """oslo/models/gpt2/configuration_gpt2.py:272-284."""

    @staticmethod
    def fused_modules():
        return {GPT2Attention: FusedGPT2Attention, GPT2MLP: FusedGPT2MLP, GPT2Block: FusedGPT2Block}


class GPT2Model(nn.Module):
    def __init__(self, config):
        super().__init__()
        self.wte = nn.Embedding(config.vocab_size, config.hidden_size)
        self.wpe = nn.Embedding(config.max_position_embeddings, config.hidden_size)
        self.drop = nn.Dropout(config.embd_pdrop)
        self.h = nn.ModuleList([GPT2Block(config, layer_idx=i) for i in range(config.n_layer)])
        self.ln_f = nn.LayerNorm(config.hidden_size, eps=config.layer_norm_epsilon)

    def forward(self, input_ids, attention_mask=None, past_key_values=None, use_cache=False):
        if past_key_values is not None and isinstance(past_key_values[0], StaticKV):
            pos = past_key_values[0].state.pos
        else:
            past_len = 0 if past_key_values is None else past_key_values[0][0].size(-2)
            pos = torch.arange(past_len, past_len + input_ids.size(-1), device=input_ids.device)
        h = self.drop(self.wte(input_ids) + self.wpe(pos)[None])
        mask = additive_attention_mask(attention_mask, h.dtype)
        presents = []
        for i, block in enumerate(self.h):
            h, present = block(h, layer_past=None if past_key_values is None else past_key_values[i],
                               attention_mask=mask, use_cache=use_cache)
            presents.append(present)
        return self.ln_f(h), (tuple(presents) if use_cache else None)


class GPT2LMHeadModel(PreTrainedModel):
    is_fusable = True

    def __init__(self, config):
        super().__init__(config)
        self.transformer = GPT2Model(config)
        self.lm_head = nn.Linear(config.hidden_size, config.vocab_size, bias=False)
        self.init_weights()
        self.lm_head.weight = self.transformer.wte.weight  # tied

    def get_layer_policies(self):
        return [GPT2LayerPolicy]

    def forward(self, input_ids, attention_mask=None, past_key_values=None, use_cache=False, labels=None):
        h, presents = self.transformer(input_ids, attention_mask, past_key_values, use_cache)
        fused_head = getattr(self, "fused_lm_head", False) and not self.training
        logits = FusedLinearRows.project(self.lm_head, h) if fused_head else self.lm_head(h)
        loss = causal_lm_loss(logits, labels) if labels is not None else None
        return {"loss": loss, "logits": logits, "past_key_values": presents}
