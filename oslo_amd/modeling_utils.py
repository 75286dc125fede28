"""What the three model files share: the GPT-2 style ``Conv1D`` projection, the
activation table, the layer-policy hook ``fuse()`` reads, and a small base class
that gives a model random initialisation and the ``fuse()`` method.

The reference builds its models on HuggingFace's PreTrainedModel
(oslo/modeling_utils.py:107-111); the models here are self-contained torch
modules with the same sub-module names and call signatures on the fusion path,
so that ``FusedKernelMixin.fuse`` and the fused module classes read like the
reference's (oslo/fused_kernels_utils.py:524-566)."""

import math

import torch
from torch import nn

from .fused_kernels_utils import FusedKernelMixin
from .generation_utils import GenerationMixin


class Conv1D(nn.Module):
    """y = x @ weight + bias with weight stored [in, out] (the GPT-2 layout)."""

    def __init__(self, nf, nx):
        super().__init__()
        self.nf = nf
        self.weight = nn.Parameter(torch.empty(nx, nf))
        self.bias = nn.Parameter(torch.zeros(nf))
        nn.init.normal_(self.weight, std=0.02)

    def forward(self, x):
        size_out = x.size()[:-1] + (self.nf,)
        x = torch.addmm(self.bias, x.view(-1, x.size(-1)), self.weight)
        return x.view(size_out)


class NewGELU(nn.Module):
    """The "gelu_new" of the GPT family: 0.5x(1 + tanh(sqrt(2/pi)(x + 0.044715 x^3)))."""

    def forward(self, x):
        return 0.5 * x * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * torch.pow(x, 3.0))))


class _ActTable(dict):
    def __missing__(self, key):
        from transformers.activations import ACT2FN as hf_table  # anything not listed below

        return hf_table[key]


ACT2FN = _ActTable(
    gelu_new=NewGELU(),
    gelu=nn.GELU(),
    gelu_pytorch_tanh=nn.GELU(approximate="tanh"),
    relu=nn.ReLU(),
    silu=nn.SiLU(),
    swish=nn.SiLU(),
    tanh=nn.Tanh(),
)


class LayerPolicy(object):
    """The part of the reference's LayerPolicy (oslo/parallelism/mpu.py:964-1043)
    that kernel fusion uses: the map from module class to fused subclass."""

    @staticmethod
    def fused_modules():
        raise NotImplementedError


class PreTrainedModel(nn.Module, FusedKernelMixin, GenerationMixin):
    """Random-initialised model with ``fuse()`` and ``generate()``. Sub-classes
    set ``is_fusable`` and ``get_layer_policies()`` as the reference's model
    classes do (oslo/models/gpt2/modeling_gpt2.py:496, :521-523)."""

    is_fusable = False

    def __init__(self, config):
        super().__init__()
        self.config = config

    def get_layer_policies(self):
        return []

    def init_weights(self, std=0.02):
        for m in self.modules():
            if isinstance(m, (nn.Linear, Conv1D)):
                nn.init.normal_(m.weight, mean=0.0, std=std)
                if m.bias is not None:
                    nn.init.zeros_(m.bias)
            elif isinstance(m, nn.Embedding):
                nn.init.normal_(m.weight, mean=0.0, std=std)
            elif isinstance(m, nn.LayerNorm):
                nn.init.ones_(m.weight)
                nn.init.zeros_(m.bias)


class DecodeState(object):
    """What the layers' static caches share while one token is decoded at a
    time: ``pos``, the index of the token being fed (a device tensor, so that
    a step can be replayed as a HIP graph while it advances), and the key masks
    that hide the slots past it."""

    def __init__(self, capacity, device, dtype):
        self.capacity = int(capacity)
        self.dtype = dtype
        self.pos = torch.zeros(1, dtype=torch.long, device=device)
        self.slots = torch.arange(self.capacity, device=device)
        self._hidden = {}  # window (None: all earlier keys) -> bool [1,1,1,capacity], True = hidden
        self.step_values = {}  # what layers share within one step (the rotary table row of ``pos``)

    def begin_step(self):
        """Recomputes the masks from ``pos``; called once per step, before the
        model's forward (inside the graph when the step is captured)."""
        self.step_values.clear()
        for window, mask in self._hidden.items():
            mask.copy_(self._compute(window))

    def _compute(self, window):
        hidden = self.slots > self.pos
        if window is not None:
            hidden = hidden | (self.slots <= self.pos - window)
        return hidden.view(1, 1, 1, -1)

    def hidden_keys(self, window=None):
        """bool [1,1,1,capacity]: True where the query at ``pos`` must not look
        (slots not written yet; for a sliding window also keys too far back)."""
        mask = self._hidden.get(window)
        if mask is None:
            mask = self._hidden[window] = self._compute(window).clone()
        return mask


class StaticKV(object):
    """One layer's key/value cache as two preallocated [rows, heads, capacity,
    head_dim] buffers. Passed where the models take ``layer_past``: the new key
    and value are written at ``state.pos`` and attention runs over the whole
    buffers under ``state.hidden_keys()``. Shapes never change from step to
    step, which is what capturing a step as a graph needs."""

    def __init__(self, state, k, v):
        if k.shape != v.shape or k.dim() != 4 or k.size(2) != state.capacity:
            raise ValueError("StaticKV: buffers must be two [rows, heads, capacity, head_dim] tensors")
        self.state, self.k, self.v = state, k, v
        self.pending = None  # (key, value) of the step, handed over but not yet in the buffers

    @classmethod
    def allocate(cls, state, layers, rows, heads, head_dim, dtype, device):
        """The caches of ``layers`` layers as views of one [layers, 2, rows,
        heads, capacity, head_dim] tensor, which is returned with them: beam
        search reorders all of them with one gather along its rows."""
        store = torch.zeros((layers, 2, rows, heads, state.capacity, head_dim), dtype=dtype, device=device)
        return store, tuple(cls(state, store[i, 0], store[i, 1]) for i in range(layers))

    def fill(self, key, value):
        """Takes over the keys/values of a prompt ([rows, heads, n, head_dim])."""
        n = key.size(-2)
        self.k[:, :, :n].copy_(key)
        self.v[:, :, :n].copy_(value)

    def update(self, key, value, defer=False):
        """The step's key and value join the buffers at ``state.pos``. With
        ``defer`` they are only kept: the caller then either passes them to the
        one-pass attention kernel, which writes them into their slot itself
        (``take_pending``), or has them written before it reads the buffers
        (``flush``)."""
        if key.size(-2) != 1:
            raise RuntimeError("StaticKV: a static cache takes one token per step")
        self.pending = (key, value)
        if not defer:
            self.flush()
        return self.k, self.v

    def pending_is_dense(self):
        """A key/value pair is waiting and the kernel can read it as it lies:
        the heads of a sequence side by side (sequences may be strided, as the
        slices of a packed projection are)."""
        if self.pending is None:
            return False
        key, value = self.pending
        b, h, _, d = key.shape

        def ok(t):
            return t.stride(3) == 1 and (h == 1 or t.stride(1) == d) and (b == 1 or t.stride(0) >= h * d)
        return ok(key) and ok(value) and (b == 1 or key.stride(0) == value.stride(0))

    def take_pending(self):
        pending, self.pending = self.pending, None
        return pending

    def flush(self):
        if self.pending is not None:
            key, value = self.take_pending()
            self.k.index_copy_(2, self.state.pos, key)
            self.v.index_copy_(2, self.state.pos, value)


def append_kv(layer_past, key, value, use_cache, defer=False):
    """key/value of this call joined to the cache -> (key, value, present).
    ``defer``: see StaticKV.update (no effect on other caches)."""
    if isinstance(layer_past, StaticKV):
        key, value = layer_past.update(key, value, defer)
        return key, value, layer_past
    if layer_past is not None:
        key = torch.cat((layer_past[0], key), dim=-2)
        value = torch.cat((layer_past[1], value), dim=-2)
    return key, value, ((key, value) if use_cache else None)


def static_cache_mask(layer_past, attention_mask, fused, window=None):
    """With a static cache the mask of a step comes from the decode state: a
    bool key mask for the fused key-mask kernel, an additive one (0 / -10000,
    the convention of ``additive_attention_mask``) for the unfused attention."""
    if attention_mask is not None:
        raise RuntimeError("a static key/value cache does not combine with an attention_mask")
    hidden = layer_past.state.hidden_keys(window)
    if fused:
        return hidden
    return hidden.to(layer_past.state.dtype) * -10000.0


def additive_attention_mask(attention_mask, dtype):
    """[B, S] mask of ones (keep) and zeros (padding) -> additive [B,1,1,S] of
    0 / -10000, as the reference's model forward builds it
    (oslo/models/gpt2/modeling_gpt2.py:669-687)."""
    if attention_mask is None:
        return None
    m = attention_mask[:, None, None, :].to(dtype)
    return (1.0 - m) * -10000.0


def causal_lm_loss(logits, labels):
    shift_logits = logits[..., :-1, :].contiguous()
    shift_labels = labels[..., 1:].contiguous()
    return nn.functional.cross_entropy(shift_logits.view(-1, shift_logits.size(-1)).float(),
                                       shift_labels.view(-1))
