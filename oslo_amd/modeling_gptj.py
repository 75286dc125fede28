"""GPT-J blocks with the reference's kernel-fusion hooks.

``GPTJAttention`` / ``GPTJMLP`` compute what the reference's unfused modules
compute (oslo/models/gptj/modeling_gptj.py:49-257): rotary position embedding
on the first ``rotary_dim`` features, scores and softmax in fp32, attention and
MLP fed from the same LayerNorm. ``FusedGPTJAttention`` / ``FusedGPTJMLP`` are
the classes ``fuse()`` swaps in (oslo/models/gptj/modeling_gptj.py:936-1065).

One deliberate difference: the reference's fused attention passes
``scale=self.scale_attn`` (= sqrt(head_dim)) to a kernel that multiplies by the
scale (oslo/models/gptj/modeling_gptj.py:941-946), while its unfused attention
divides by it (:175). The fused class here passes ``1/scale_attn``, so fused
and unfused agree."""

from dataclasses import dataclass
from typing import Optional

import torch
from torch import nn

from .fused_kernels_utils import (FusedBiasActivation, FusedBiasDropout, FusedBiasDropoutResidual,
                                 FusedDecodeAttention, FusedLinearBiasActivation, FusedLinearRows, FusedPrefillAttention,
                                 FusedMergeHeads,
                                 FusedRotaryPositionEmbedding,
                                 FusedScaleMaskSoftmax, FusedScaleMaskSoftmaxDropout)
from .modeling_utils import (ACT2FN, LayerPolicy, PreTrainedModel, StaticKV, additive_attention_mask, append_kv,
                             causal_lm_loss, static_cache_mask)


@dataclass
class GPTJConfig:
    vocab_size: int = 50400
    n_positions: int = 2048
    n_embd: int = 4096
    n_layer: int = 28
    n_head: int = 16
    rotary_dim: Optional[int] = 64
    n_inner: Optional[int] = None
    activation_function: str = "gelu_new"
    resid_pdrop: float = 0.0
    embd_pdrop: float = 0.0
    attn_pdrop: float = 0.0
    layer_norm_epsilon: float = 1e-5

    @property
    def hidden_size(self):
        return self.n_embd

    @property
    def num_attention_heads(self):
        return self.n_head

    @property
    def max_position_embeddings(self):
        return self.n_positions


_rotary_table_cache = {}


def rotary_tables(dim, seq_len, device):
    """sin and cos of position * 10000^(-2i/dim), each [seq_len, dim/2], fp32.
    Every layer asks for the same tables, so the last few are kept."""
    key = (int(dim), int(seq_len), str(device))
    hit = _rotary_table_cache.get(key)
    if hit is not None:
        return hit
    inv_freq = 1.0 / (10000 ** (torch.arange(0, dim, 2, device=device, dtype=torch.float32) / dim))
    angles = torch.arange(seq_len, device=device, dtype=torch.float32)[:, None] * inv_freq[None, :]
    tables = (torch.sin(angles), torch.cos(angles))
    if len(_rotary_table_cache) >= 8:
        _rotary_table_cache.pop(next(iter(_rotary_table_cache)))
    _rotary_table_cache[key] = tables
    return tables


def rotary_for_step(layer_past, dim, seq_len, device):
    """(sin, cos, offset) for ``seq_len`` new tokens after the cached ones. With
    a static cache the position lives on the device: the one table row of the
    step is gathered there and the offset into it is 0."""
    if isinstance(layer_past, StaticKV):
        state = layer_past.state
        row = state.step_values.get(("rotary", dim))
        if row is None:  # the first layer of a step gathers the row, the others reuse it
            sin, cos = rotary_tables(dim, state.capacity, device)
            row = state.step_values[("rotary", dim)] = (sin.index_select(0, state.pos), cos.index_select(0, state.pos))
        return row[0], row[1], 0
    offset = 0 if layer_past is None else layer_past[0].shape[-2]
    sin, cos = rotary_tables(dim, seq_len + offset, device)
    return sin, cos, offset


def apply_rotary(x, sin, cos, offset=0):
    """x [B, S, H, D]: rotates consecutive feature pairs (2i, 2i+1) by the angle
    of position offset+s."""
    s = x.shape[1]
    sin = sin[offset:offset + s].repeat_interleave(2, dim=-1)[None, :, None, :]
    cos = cos[offset:offset + s].repeat_interleave(2, dim=-1)[None, :, None, :]
    rotated = torch.stack((-x[..., 1::2], x[..., ::2]), dim=-1).flatten(-2)
    return x * cos + rotated * sin


class GPTJAttention(nn.Module):
    def __init__(self, config):
        super().__init__()
        n_pos = config.max_position_embeddings
        self.register_buffer(
            "bias", torch.tril(torch.ones((n_pos, n_pos), dtype=torch.uint8)).view(1, 1, n_pos, n_pos))
        self.register_buffer("masked_bias", torch.tensor(-1e9))
        self.attn_dropout = nn.Dropout(config.attn_pdrop)
        self.resid_dropout = nn.Dropout(config.resid_pdrop)
        self.embed_dim = config.hidden_size
        self.num_attention_heads = config.num_attention_heads
        self.head_dim = self.embed_dim // self.num_attention_heads
        if self.head_dim * self.num_attention_heads != self.embed_dim:
            raise ValueError("embed_dim must be divisible by num_attention_heads")
        self.scale_attn = float(self.head_dim) ** 0.5
        self.k_proj = nn.Linear(self.embed_dim, self.embed_dim, bias=False)
        self.v_proj = nn.Linear(self.embed_dim, self.embed_dim, bias=False)
        self.q_proj = nn.Linear(self.embed_dim, self.embed_dim, bias=False)
        self.out_proj = nn.Linear(self.embed_dim, self.embed_dim, bias=False)
        self.rotary_dim = config.rotary_dim

    def _merge_heads(self, t):
        t = t.permute(0, 2, 1, 3).contiguous()
        return t.view(t.size()[:-2] + (self.num_attention_heads * self.head_dim,))

    def _attn(self, query, key, value, attention_mask=None, head_mask=None, causal=True):
        """The unfused path: fp32 scores, where(causal, w, -1e9), / sqrt(d), + mask, softmax."""
        w = torch.matmul(query.to(torch.float32), key.to(torch.float32).transpose(-1, -2))
        if causal:
            sq, sk = query.size(-2), key.size(-2)
            w = torch.where(self.bias[:, :, sk - sq:sk, :sk].bool(), w, self.masked_bias.to(w.dtype))
        w = w / self.scale_attn
        if attention_mask is not None:
            w = w + attention_mask
        w = nn.functional.softmax(w, dim=-1).to(value.dtype)
        w = self.attn_dropout(w)
        if head_mask is not None:
            w = w * head_mask
        return torch.matmul(w, value), w

    def _project_qkv(self, hidden_states, layer_past, use_cache):
        b, s, _ = hidden_states.shape
        shape = (b, s, self.num_attention_heads, self.head_dim)
        query = self.q_proj(hidden_states).view(shape)
        key = self.k_proj(hidden_states).view(shape)
        value = self.v_proj(hidden_states).view(shape).permute(0, 2, 1, 3)
        rot = self.rotary_dim if self.rotary_dim is not None else self.head_dim
        sin, cos, offset = rotary_for_step(layer_past, rot, s, hidden_states.device)
        if rot < self.head_dim:
            key = torch.cat([apply_rotary(key[..., :rot], sin, cos, offset), key[..., rot:]], dim=-1)
            query = torch.cat([apply_rotary(query[..., :rot], sin, cos, offset), query[..., rot:]], dim=-1)
        else:
            key = apply_rotary(key, sin, cos, offset)
            query = apply_rotary(query, sin, cos, offset)
        key = key.to(value.dtype).permute(0, 2, 1, 3)
        query = query.to(value.dtype).permute(0, 2, 1, 3)
        key, value, present = append_kv(layer_past, key, value, use_cache)
        return query, key, value, present

    def forward(self, hidden_states, attention_mask=None, layer_past=None, head_mask=None,
                use_cache=False, output_attentions=False):
        query, key, value, present = self._project_qkv(hidden_states, layer_past, use_cache)
        static = isinstance(layer_past, StaticKV)
        if static:
            attention_mask = static_cache_mask(layer_past, attention_mask, fused=False)
        out, w = self._attn(query, key, value, attention_mask, head_mask, causal=not static)
        out = self.resid_dropout(self.out_proj(self._merge_heads(out)))
        return (out, present, w) if output_attentions else (out, present)


class FusedGPTJAttention(GPTJAttention):
    """oslo/models/gptj/modeling_gptj.py:936-1038. Beyond the reference's fused
    class, the rotary embedding of q and k and the split-heads permute of
    q, k and v run as one kernel (the reference keeps the torch operators)."""

    def _project_qkv(self, hidden_states, layer_past, use_cache):
        rot = self.rotary_dim if self.rotary_dim is not None else self.head_dim
        if not (hidden_states.is_cuda and
                FusedRotaryPositionEmbedding.is_available(hidden_states.dtype, self.head_dim, rot)):
            return super()._project_qkv(hidden_states, layer_past, use_cache)
        b, s, _ = hidden_states.shape
        shape = (b, s, self.num_attention_heads, self.head_dim)
        sin, cos, offset = rotary_for_step(layer_past, rot, s, hidden_states.device)
        # (a decoding step streams the three weights in one launch)
        query, key, value = FusedLinearRows.project_many((self.q_proj, self.k_proj, self.v_proj), hidden_states)
        query, key, value = FusedRotaryPositionEmbedding.apply(
            query.view(shape), key.view(shape), value.view(shape), (sin, cos), rot, offset)
        key, value, present = append_kv(layer_past, key, value, use_cache, defer=True)
        return query, key, value, present

    def _fused_attn(self, query, key, value, attention_mask=None, head_mask=None, causal=True):
        w = torch.matmul(query, key.transpose(-1, -2))
        # softmax and attn_dropout in one kernel (the reference runs nn.Dropout
        # as a second pass over the probabilities)
        w = FusedScaleMaskSoftmaxDropout.apply(w, attention_mask, 1.0 / self.scale_attn, causal,
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
        # a single query over a key/value cache (a decoding step) sees every key:
        # the causal mask is empty and the key-mask kernel applies
        causal = sq > 1
        static = isinstance(layer_past, StaticKV)
        fused = FusedScaleMaskSoftmax.is_available(query.dtype, bsz, np_, sq, sk, use_triang_mask=causal)
        one_pass = (sq == 1 and attention_mask is None and head_mask is None and not output_attentions
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
                                             1.0 / self.scale_attn, None, *fresh)
            w = None
        elif prompt:
            # a whole prompt: one kernel, the scores stay on chip (in training too: it has a backward
            # and drops attention probabilities itself)
            out, w = FusedPrefillAttention.apply(query, key, value, attention_mask, 1.0 / self.scale_attn, None,
                                                 self.attn_dropout.p if self.training else 0.0), None
        elif fused:
            out, w = self._fused_attn(query, key, value, attention_mask, head_mask, causal)
        else:
            out, w = self._attn(query, key, value, attention_mask, head_mask, causal=not static)
        # out_proj has no bias: the epilogue kernel runs with the bias term
        # dropped (in training; it is skipped when there is nothing to drop)
        vec_ok = FusedRotaryPositionEmbedding.is_available(out.dtype, self.head_dim, 0)
        out = FusedMergeHeads.apply(out) if out.is_cuda and vec_ok else self._merge_heads(out)
        if residual is not None and FusedLinearRows.is_available(out, self.out_proj.weight) and not (
                self.training and self.resid_dropout.p > 0.0):
            out = FusedLinearRows.apply(out, self.out_proj.weight, residual=residual)  # a decoding step
        else:
            out = FusedLinearRows.project(self.out_proj, out)
            if residual is None:
                out = FusedBiasDropout.apply(out, None, self.training, self.resid_dropout.p)
            else:  # dropout and the block's residual addition in one pass
                out = FusedBiasDropoutResidual.apply(out, None, residual, self.training, self.resid_dropout.p)
        return (out, present, w) if output_attentions else (out, present)


class GPTJMLP(nn.Module):
    def __init__(self, intermediate_size, config):
        super().__init__()
        self.fc_in = nn.Linear(config.n_embd, intermediate_size)
        self.fc_out = nn.Linear(intermediate_size, config.n_embd)
        self.act = ACT2FN[config.activation_function]
        self.dropout = nn.Dropout(config.resid_pdrop)

    def forward(self, hidden_states):
        return self.dropout(self.fc_out(self.act(self.fc_in(hidden_states))))


class FusedGPTJMLP(GPTJMLP):
    """oslo/models/gptj/modeling_gptj.py:1041-1065."""

    def forward(self, x, residual=None, residual2=None):
        """``residual``, ``residual2``: added to the output (the residual
        connection of the block and, for the block's three-term sum, the
        attention output)."""
        if FusedLinearRows.is_available(x, self.fc_in.weight, self.fc_in.bias) and \
                FusedLinearRows.is_available(None, self.fc_out.weight, self.fc_out.bias, rows_of=x):
            # a decoding step: each projection is one pass over its weight with
            # the bias (and the activation, and the residual) applied to the fp32 sums
            x = FusedLinearRows.apply(x, self.fc_in.weight, self.fc_in.bias, self.config.activation_function)
            if residual2 is None and not (self.training and self.dropout.p > 0.0):
                return FusedLinearRows.apply(x, self.fc_out.weight, self.fc_out.bias, residual=residual)
            x = FusedLinearRows.apply(x, self.fc_out.weight)
        else:
            act = self.config.activation_function
            if FusedLinearBiasActivation.is_available(x, self.fc_in.weight, self.fc_in.bias, act):
                # bias and GeLU on the product's fp32 sums, in its own launch
                x = FusedLinearBiasActivation.apply(x, self.fc_in.weight, self.fc_in.bias, act)
            else:
                x = x @ self.fc_in.weight.t()
                x = FusedBiasActivation.apply(x, self.fc_in.bias, act)
            x = x @ self.fc_out.weight.t()
        if residual is None and residual2 is None:
            return FusedBiasDropout.apply(x, self.fc_out.bias, self.training, self.dropout.p)
        # bias, dropout and the block's residual addition(s) in one pass
        return FusedBiasDropoutResidual.apply(x, self.fc_out.bias, residual, self.training, self.dropout.p,
                                              residual2)


class GPTJBlock(nn.Module):
    def __init__(self, config):
        super().__init__()
        inner = config.n_inner if config.n_inner is not None else 4 * config.n_embd
        self.ln_1 = nn.LayerNorm(config.n_embd, eps=config.layer_norm_epsilon)
        self.attn = GPTJAttention(config)
        self.mlp = GPTJMLP(inner, config)

    def forward(self, hidden_states, layer_past=None, attention_mask=None, head_mask=None, use_cache=False):
        residual = hidden_states
        hidden_states = self.ln_1(hidden_states)
        a = self.attn(hidden_states, layer_past=layer_past, attention_mask=attention_mask,
                      head_mask=head_mask, use_cache=use_cache)
        hidden_states = a[0] + self.mlp(hidden_states) + residual
        return hidden_states, a[1]


class FusedGPTJBlock(GPTJBlock):
    """The block with its residual additions handed to the fused modules. The
    unfused block adds attention output, feed-forward output and residual
    stream with two torch additions (oslo/models/gptj/modeling_gptj.py:306-327).
    Over a prompt (and in training) the feed-forward's epilogue kernel takes
    all three: bias + dropout of its own term, then the attention output and
    the residual stream, summed in fp32 and rounded once -- one rounding at the
    magnitude of the residual stream per layer, as in the unfused block (adding
    the attention output into the stream first and the feed-forward output in a
    second pass rounds there twice, and 28 layers of it showed in the logits).
    In a decoding step the two modules take the additions into the launches of
    their last projections instead (attention output + residual first, the
    feed-forward output on top). No counterpart in the reference, which fuses
    attention and MLP only (oslo/models/gptj/configuration_gptj.py:155-167)."""

    def forward(self, hidden_states, layer_past=None, attention_mask=None, head_mask=None, use_cache=False):
        if not (isinstance(self.attn, FusedGPTJAttention) and isinstance(self.mlp, FusedGPTJMLP)):
            return super().forward(hidden_states, layer_past, attention_mask, head_mask, use_cache)
        normed = self.ln_1(hidden_states)
        if hidden_states.shape[-2] > 1 and hidden_states.is_cuda:
            a = self.attn(normed, layer_past=layer_past, attention_mask=attention_mask, head_mask=head_mask,
                          use_cache=use_cache)
            return self.mlp(normed, residual=hidden_states, residual2=a[0]), a[1]
        a = self.attn(normed, layer_past=layer_past, attention_mask=attention_mask, head_mask=head_mask,
                      use_cache=use_cache, residual=hidden_states)
        return self.mlp(normed, residual=a[0]), a[1]


class GPTJLayerPolicy(LayerPolicy):
    """oslo/models/gptj/configuration_gptj.py:155-167."""

    @staticmethod
    def fused_modules():
        return {GPTJAttention: FusedGPTJAttention, GPTJMLP: FusedGPTJMLP, GPTJBlock: FusedGPTJBlock}


class GPTJModel(nn.Module):
    def __init__(self, config):
        super().__init__()
        self.wte = nn.Embedding(config.vocab_size, config.n_embd)
        self.drop = nn.Dropout(config.embd_pdrop)
        self.h = nn.ModuleList([GPTJBlock(config) for _ in range(config.n_layer)])
        self.ln_f = nn.LayerNorm(config.n_embd, eps=config.layer_norm_epsilon)

    def forward(self, input_ids, attention_mask=None, past_key_values=None, use_cache=False):
        h = self.drop(self.wte(input_ids))
        mask = additive_attention_mask(attention_mask, h.dtype)
        presents = []
        for i, block in enumerate(self.h):
            h, present = block(h, layer_past=None if past_key_values is None else past_key_values[i],
                               attention_mask=mask, use_cache=use_cache)
            presents.append(present)
        return self.ln_f(h), (tuple(presents) if use_cache else None)


class GPTJForCausalLM(PreTrainedModel):
    is_fusable = True

    def __init__(self, config):
        super().__init__(config)
        self.transformer = GPTJModel(config)
        self.lm_head = nn.Linear(config.n_embd, config.vocab_size)
        self.init_weights()

    def get_layer_policies(self):
        return [GPTJLayerPolicy]

    def forward(self, input_ids, attention_mask=None, past_key_values=None, use_cache=False, labels=None):
        h, presents = self.transformer(input_ids, attention_mask, past_key_values, use_cache)
        fused_head = getattr(self, "fused_lm_head", False) and not self.training
        logits = FusedLinearRows.project(self.lm_head, h) if fused_head else self.lm_head(h)
        loss = causal_lm_loss(logits, labels) if labels is not None else None
        return {"loss": loss, "logits": logits, "past_key_values": presents}
