"""GPT-Neo blocks with the reference's kernel-fusion hooks.

``GPTNeoSelfAttention`` / ``GPTNeoMLP`` compute what the reference's unfused
modules compute (oslo/models/gpt_neo/modeling_gpt_neo.py:145-329): unscaled
scores, fp32 softmax, global or sliding-window ("local") causal masks.
``FusedGPTNeoSelfAttention`` / ``FusedGPTNeoMLP`` are what ``fuse()`` swaps in
(oslo/models/gpt_neo/modeling_gpt_neo.py:993-1102). As in the reference, local
attention layers are a separate class
(oslo/models/gpt_neo/modeling_gpt_neo.py:268-272); the reference leaves them
unfused because their mask is not a plain lower triangle, here they get a fused
class of their own on the sliding-window softmax kernel."""

from dataclasses import dataclass, field
from typing import List, Optional

import torch
from torch import nn

from .fused_kernels_utils import (FusedBiasActivation, FusedBiasDropout, FusedBiasDropoutResidual,
                                 FusedDecodeAttention, FusedLinearBiasActivation, FusedLinearRows, FusedPrefillAttention,
                                 FusedMergeHeads,
                                 FusedRotaryPositionEmbedding, FusedScaleMaskSoftmax,
                                 FusedScaleMaskSoftmaxDropout, FusedScaleMaskWindowSoftmax)
from .modeling_utils import (ACT2FN, LayerPolicy, PreTrainedModel, StaticKV, additive_attention_mask, append_kv,
                             causal_lm_loss, static_cache_mask)


@dataclass
class GPTNeoConfig:
    vocab_size: int = 50257
    max_position_embeddings: int = 2048
    hidden_size: int = 2048
    num_layers: int = 24
    num_heads: int = 16
    attention_layers: List[str] = field(default_factory=list)  # "global" / "local" per layer
    window_size: int = 256
    intermediate_size: Optional[int] = None
    activation_function: str = "gelu_new"
    resid_dropout: float = 0.0
    embed_dropout: float = 0.0
    attention_dropout: float = 0.0
    layer_norm_epsilon: float = 1e-5

    def __post_init__(self):
        if not self.attention_layers:
            self.attention_layers = ["global", "local"] * (self.num_layers // 2) + \
                                    ["global"] * (self.num_layers % 2)


class GPTNeoSelfAttention(nn.Module):
    def __init__(self, config, attention_type):
        super().__init__()
        n_pos = config.max_position_embeddings
        bias = torch.tril(torch.ones((n_pos, n_pos), dtype=torch.uint8)).view(1, 1, n_pos, n_pos)
        if attention_type == "local":  # keep only the last window_size keys of each row
            bias = torch.bitwise_xor(bias, torch.tril(bias, -config.window_size))
        self.register_buffer("bias", bias)
        self.register_buffer("masked_bias", torch.tensor(-1e9))
        self.attn_dropout = nn.Dropout(config.attention_dropout)
        self.resid_dropout = nn.Dropout(config.resid_dropout)
        self.embed_dim = config.hidden_size
        self.num_heads = config.num_heads
        self.head_dim = self.embed_dim // self.num_heads
        self.config_window = config.window_size
        if self.head_dim * self.num_heads != self.embed_dim:
            raise ValueError("embed_dim must be divisible by num_heads")
        self.k_proj = nn.Linear(self.embed_dim, self.embed_dim, bias=False)
        self.v_proj = nn.Linear(self.embed_dim, self.embed_dim, bias=False)
        self.q_proj = nn.Linear(self.embed_dim, self.embed_dim, bias=False)
        self.out_proj = nn.Linear(self.embed_dim, self.embed_dim, bias=True)

    def _split_heads(self, t):
        return t.view(t.size()[:-1] + (self.num_heads, self.head_dim)).permute(0, 2, 1, 3)

    def _merge_heads(self, t):
        t = t.permute(0, 2, 1, 3).contiguous()
        return t.view(t.size()[:-2] + (self.num_heads * self.head_dim,))

    def _attn(self, query, key, value, attention_mask=None, head_mask=None, causal=True):
        """The unfused path: fp32 scores (no scaling), where(mask, w, -1e9), + mask, softmax."""
        w = torch.matmul(query.to(torch.float32), key.to(torch.float32).transpose(-1, -2))
        if causal:
            sq, sk = query.size(-2), key.size(-2)
            w = torch.where(self.bias[:, :, sk - sq:sk, :sk].bool(), w, self.masked_bias.to(w.dtype))
        if attention_mask is not None:
            w = w + attention_mask
        w = nn.functional.softmax(w, dim=-1).to(value.dtype)
        w = self.attn_dropout(w)
        if head_mask is not None:
            w = w * head_mask
        return torch.matmul(w, value), w

    def _project_qkv(self, hidden_states, layer_past, use_cache):
        query = self._split_heads(self.q_proj(hidden_states))
        key = self._split_heads(self.k_proj(hidden_states))
        value = self._split_heads(self.v_proj(hidden_states))
        key, value, present = append_kv(layer_past, key, value, use_cache)
        return query, key, value, present

    def _window(self):
        """Keys a query sees counting back from itself; None: all of them."""
        return self.config_window if isinstance(self, GPTNeoLocalSelfAttention) else None

    def forward(self, hidden_states, attention_mask=None, layer_past=None, head_mask=None,
                use_cache=False, output_attentions=False):
        query, key, value, present = self._project_qkv(hidden_states, layer_past, use_cache)
        static = isinstance(layer_past, StaticKV)
        if static:
            attention_mask = static_cache_mask(layer_past, attention_mask, fused=False, window=self._window())
        out, w = self._attn(query, key, value, attention_mask, head_mask, causal=not static)
        out = self.resid_dropout(self.out_proj(self._merge_heads(out)))
        return (out, present, w) if output_attentions else (out, present)


class GPTNeoLocalSelfAttention(GPTNeoSelfAttention):
    """Sliding-window layers; a class of their own so that fusion skips them."""


class FusedGPTNeoSelfAttention(GPTNeoSelfAttention):
    """oslo/models/gpt_neo/modeling_gpt_neo.py:993-1075. Beyond the reference's
    fused class, the split-heads permutes of q, k, v and the merge-heads
    permute run through the transposition kernel (one launch for q, k and v)
    instead of torch's strided copies."""

    def _transposes_fused(self, t):
        return t.is_cuda and FusedRotaryPositionEmbedding.is_available(t.dtype, self.head_dim, 0)

    def _project_qkv(self, hidden_states, layer_past, use_cache):
        if not self._transposes_fused(hidden_states):
            return super()._project_qkv(hidden_states, layer_past, use_cache)
        b, s, _ = hidden_states.shape
        shape = (b, s, self.num_heads, self.head_dim)
        # (a decoding step streams the three weights in one launch)
        query, key, value = FusedLinearRows.project_many((self.q_proj, self.k_proj, self.v_proj), hidden_states)
        query, key, value = FusedRotaryPositionEmbedding.apply(
            query.view(shape), key.view(shape), value.view(shape), (None, None), 0)
        key, value, present = append_kv(layer_past, key, value, use_cache, defer=True)
        return query, key, value, present

    def _fused_attn(self, query, key, value, attention_mask=None, head_mask=None, causal=True):
        w = torch.matmul(query, key.transpose(-1, -2))
        # softmax and attn_dropout in one kernel (the reference runs nn.Dropout
        # as a second pass over the probabilities)
        w = FusedScaleMaskSoftmaxDropout.apply(w, attention_mask, None, causal,
                                               self.attn_dropout.p, self.training).to(value.dtype)
        if head_mask is not None:
            w = w * head_mask
        return torch.matmul(w, value), w

    def forward(self, hidden_states, attention_mask=None, layer_past=None, head_mask=None,
                use_cache=False, output_attentions=False, residual=None):
        """``residual``: added to the output (the residual connection of the
        block, which a decoding step takes into the projection's launch)."""
        query, key, value, present = self._project_qkv(hidden_states, layer_past, use_cache)
        (bsz, np_, sq, _), sk = query.size(), key.size(-2)
        # a single query over a key/value cache (a decoding step) sees every key
        # of a global layer: the causal mask is empty and the key-mask kernel
        # applies. A local layer still has its window and stays unfused then.
        # With a static cache the window, too, is part of the step's key mask.
        static = isinstance(layer_past, StaticKV)
        causal = not static and (sq > 1 or isinstance(self, GPTNeoLocalSelfAttention))
        fused = FusedScaleMaskSoftmax.is_available(query.dtype, bsz, np_, sq, sk, use_triang_mask=causal)
        one_pass = (sq == 1 and attention_mask is None and head_mask is None and not output_attentions
                    and FusedDecodeAttention.is_available(query, key, self.training, self.attn_dropout.p))
        fresh = (None, None)  # the step's key and value, if not yet in a static cache
        if static and one_pass and layer_past.pending_is_dense():
            fresh = layer_past.take_pending()  # the kernel below writes them into their slot
        elif static:
            layer_past.flush()
        if static and not one_pass:
            attention_mask = static_cache_mask(layer_past, attention_mask, fused, window=self._window())
        prompt = (causal and sq > 1 and head_mask is None and not output_attentions
                  and FusedPrefillAttention.is_available(query, key, attention_mask, self.training,
                                                         self.attn_dropout.p))
        if one_pass:
            # a decoding step: scores, softmax and weighted sum in one pass over the
            # cache, the window of a local layer included
            out = FusedDecodeAttention.apply(query, key, value, layer_past.state.pos if static else sk - 1,
                                             None, self._window(), *fresh)
            w = None
        elif prompt:
            # a whole prompt: one kernel, the scores stay on chip (in training too: it has a backward
            # and drops attention probabilities itself) (a local
            # layer's window included)
            out, w = FusedPrefillAttention.apply(query, key, value, attention_mask, None, self._window(),
                                                 self.attn_dropout.p if self.training else 0.0), None
        elif fused and static:
            out, w = FusedGPTNeoSelfAttention._fused_attn(self, query, key, value, attention_mask, head_mask, False)
        elif fused:
            out, w = self._fused_attn(query, key, value, attention_mask, head_mask, causal)
        else:
            out, w = self._attn(query, key, value, attention_mask, head_mask, causal=not static)
        out = FusedMergeHeads.apply(out) if self._transposes_fused(out) else self._merge_heads(out)
        if FusedLinearRows.is_available(out, self.out_proj.weight) and not (
                self.training and self.resid_dropout.p > 0.0):
            out = FusedLinearRows.apply(out, self.out_proj.weight, self.out_proj.bias, residual=residual)
        else:
            out = out @ self.out_proj.weight.t()
            if residual is None:
                out = FusedBiasDropout.apply(out, self.out_proj.bias, self.training, self.resid_dropout.p)
            else:  # bias, dropout and the block's residual addition in one pass
                out = FusedBiasDropoutResidual.apply(out, self.out_proj.bias, residual, self.training,
                                                     self.resid_dropout.p)
        return (out, present, w) if output_attentions else (out, present)


class FusedGPTNeoLocalSelfAttention(FusedGPTNeoSelfAttention, GPTNeoLocalSelfAttention):
    """The fused attention on the sliding-window kernel: row r attends the last
    ``window_size`` keys up to r. No counterpart in the reference."""

    def _fused_attn(self, query, key, value, attention_mask=None, head_mask=None, causal=True):
        w = torch.matmul(query, key.transpose(-1, -2))
        w = FusedScaleMaskWindowSoftmax.apply(w, attention_mask, None, self.config.window_size)
        w = self.attn_dropout(w.to(value.dtype))
        if head_mask is not None:
            w = w * head_mask
        return torch.matmul(w, value), w


class GPTNeoAttention(nn.Module):
    def __init__(self, config, layer_id=0):
        super().__init__()
        self.attention_type = config.attention_layers[layer_id]
        if self.attention_type == "local":
            self.attention = GPTNeoLocalSelfAttention(config, "local")
        elif self.attention_type == "global":
            self.attention = GPTNeoSelfAttention(config, "global")
        else:
            raise NotImplementedError(f"unknown attention layer type {self.attention_type!r}")

    def forward(self, hidden_states, layer_past=None, attention_mask=None, head_mask=None,
                use_cache=False, output_attentions=False):
        return self.attention(hidden_states, attention_mask=attention_mask, layer_past=layer_past,
                              head_mask=head_mask, use_cache=use_cache, output_attentions=output_attentions)


class GPTNeoMLP(nn.Module):
    def __init__(self, intermediate_size, config):
        super().__init__()
        self.c_fc = nn.Linear(config.hidden_size, intermediate_size)
        self.c_proj = nn.Linear(intermediate_size, config.hidden_size)
        self.act = ACT2FN[config.activation_function]
        self.dropout = nn.Dropout(config.resid_dropout)

    def forward(self, hidden_states):
        return self.dropout(self.c_proj(self.act(self.c_fc(hidden_states))))


class FusedGPTNeoMLP(GPTNeoMLP):
    """oslo/models/gpt_neo/modeling_gpt_neo.py:1078-1102."""

    def forward(self, x, residual=None):
        """``residual``: added to the output (the residual connection of the block)."""
        if FusedLinearRows.is_available(x, self.c_fc.weight, self.c_fc.bias) and \
                FusedLinearRows.is_available(None, self.c_proj.weight, self.c_proj.bias, rows_of=x):
            # a decoding step: each projection is one pass over its weight with
            # the bias (and the activation, and the residual) applied to the fp32 sums
            x = FusedLinearRows.apply(x, self.c_fc.weight, self.c_fc.bias, self.config.activation_function)
            if not (self.training and self.dropout.p > 0.0):
                return FusedLinearRows.apply(x, self.c_proj.weight, self.c_proj.bias, residual=residual)
            x = FusedLinearRows.apply(x, self.c_proj.weight)
        else:
            act = self.config.activation_function
            if FusedLinearBiasActivation.is_available(x, self.c_fc.weight, self.c_fc.bias, act):
                # bias and GeLU on the product's fp32 sums, in its own launch
                x = FusedLinearBiasActivation.apply(x, self.c_fc.weight, self.c_fc.bias, act)
            else:
                x = x @ self.c_fc.weight.t()
                x = FusedBiasActivation.apply(x, self.c_fc.bias, act)
            x = x @ self.c_proj.weight.t()
        if residual is None:
            return FusedBiasDropout.apply(x, self.c_proj.bias, self.training, self.dropout.p)
        # bias, dropout and the block's residual addition in one pass
        return FusedBiasDropoutResidual.apply(x, self.c_proj.bias, residual, self.training, self.dropout.p)


class GPTNeoBlock(nn.Module):
    def __init__(self, config, layer_id):
        super().__init__()
        inner = config.intermediate_size if config.intermediate_size is not None else 4 * config.hidden_size
        self.ln_1 = nn.LayerNorm(config.hidden_size, eps=config.layer_norm_epsilon)
        self.attn = GPTNeoAttention(config, layer_id)
        self.ln_2 = nn.LayerNorm(config.hidden_size, eps=config.layer_norm_epsilon)
        self.mlp = GPTNeoMLP(inner, config)

    def forward(self, hidden_states, layer_past=None, attention_mask=None, head_mask=None, use_cache=False):
        a = self.attn(self.ln_1(hidden_states), layer_past=layer_past, attention_mask=attention_mask,
                      head_mask=head_mask, use_cache=use_cache)
        hidden_states = a[0] + hidden_states
        hidden_states = hidden_states + self.mlp(self.ln_2(hidden_states))
        return hidden_states, a[1]


class FusedGPTNeoBlock(GPTNeoBlock):
    """The block with its two residual additions handed to the fused modules,
    which take them into their last projection's launch in a decoding step.
    No counterpart in the reference, which fuses attention and MLP only
    (oslo/models/gpt_neo/configuration_gpt_neo.py:330-342); the arithmetic is
    that of oslo/models/gpt_neo/modeling_gpt_neo.py:333-380."""

    def forward(self, hidden_states, layer_past=None, attention_mask=None, head_mask=None, use_cache=False):
        inner = self.attn.attention
        if not (isinstance(inner, FusedGPTNeoSelfAttention) and isinstance(self.mlp, FusedGPTNeoMLP)):
            return super().forward(hidden_states, layer_past, attention_mask, head_mask, use_cache)
        a = inner(self.ln_1(hidden_states), attention_mask=attention_mask, layer_past=layer_past,
                  head_mask=head_mask, use_cache=use_cache, residual=hidden_states)
        hidden_states = self.mlp(self.ln_2(a[0]), residual=a[0])
        return hidden_states, a[1]


class GPTNeoLayerPolicy(LayerPolicy):
    """oslo/models/gpt_neo/configuration_gpt_neo.py:330-342."""

    @staticmethod
    def fused_modules():
        return {GPTNeoSelfAttention: FusedGPTNeoSelfAttention, GPTNeoMLP: FusedGPTNeoMLP,
                GPTNeoLocalSelfAttention: FusedGPTNeoLocalSelfAttention, GPTNeoBlock: FusedGPTNeoBlock}


class GPTNeoModel(nn.Module):
    def __init__(self, config):
        super().__init__()
        self.wte = nn.Embedding(config.vocab_size, config.hidden_size)
        self.wpe = nn.Embedding(config.max_position_embeddings, config.hidden_size)
        self.drop = nn.Dropout(config.embed_dropout)
        self.h = nn.ModuleList([GPTNeoBlock(config, layer_id=i) for i in range(config.num_layers)])
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


class GPTNeoForCausalLM(PreTrainedModel):
    is_fusable = True

    def __init__(self, config):
        super().__init__(config)
        self.transformer = GPTNeoModel(config)
        self.lm_head = nn.Linear(config.hidden_size, config.vocab_size, bias=False)
        self.init_weights()
        self.lm_head.weight = self.transformer.wte.weight  # tied

    def get_layer_policies(self):
        return [GPTNeoLayerPolicy]

    def forward(self, input_ids, attention_mask=None, past_key_values=None, use_cache=False, labels=None):
        h, presents = self.transformer(input_ids, attention_mask, past_key_values, use_cache)
        fused_head = getattr(self, "fused_lm_head", False) and not self.training
        logits = FusedLinearRows.project(self.lm_head, h) if fused_head else self.lm_head(h)
        loss = causal_lm_loss(logits, labels) if labels is not None else None
        return {"loss": loss, "logits": logits, "past_key_values": presents}
