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


class PreTrainedModel(nn.Module, FusedKernelMixin):
    """Random-initialised model with ``fuse()``. Sub-classes set ``is_fusable``
    and ``get_layer_policies()`` as the reference's model classes do
    (oslo/models/gpt2/modeling_gpt2.py:496, :521-523)."""

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
