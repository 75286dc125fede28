"""The reference's unfused attention-softmax / MLP-epilogue arithmetic written
with the same torch operators the reference calls, for CPU tensors.

THIS IS TEST INFRASTRUCTURE, like oslo_oracle.py: it is the "reference CPU path"
that the benchmark times on the host cores (cpu_baseline) and that model-level
tests compare against. Nothing the library ships imports it.

Follows, operator for operator:
* attention_probs: oslo/models/gpt2/modeling_gpt2.py:194-218 (matmul result ->
  scale -> torch.where(causal, w, masked_bias) -> + attention_mask -> softmax);
  masked_bias is -1e4 there and -1e9 in oslo/models/gptj/modeling_gptj.py:95;
* bias_gelu: Conv1D bias add + ACT2FN["gelu_new"], oslo/models/gpt2/
  modeling_gpt2.py:394-399;
* bias_dropout_add: nn.Dropout(c_proj(x)) + residual, oslo/models/gpt2/
  modeling_gpt2.py:397-399 and :444.
"""

import math

import torch


def attention_probs(scores, scale, causal=True, attention_mask=None, masked_bias=-1e4):
    """scores [B,H,Sq,Sk] (the Q K^T product); returns softmax probabilities."""
    w = scores * scale
    if causal:
        sq, sk = scores.shape[-2:]
        keep = torch.tril(torch.ones((sk, sk), dtype=torch.bool))[sk - sq:sk, :sk]
        w = torch.where(keep, w, torch.tensor(masked_bias, dtype=w.dtype))
    if attention_mask is not None:
        w = w + attention_mask
    return torch.nn.functional.softmax(w, dim=-1)


def gelu_new(x):
    return 0.5 * x * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * torch.pow(x, 3.0))))


def bias_gelu(y, bias):
    return gelu_new(y + bias)


def bias_dropout_add(x, bias, residual, p, training):
    out = torch.nn.functional.dropout(x + bias, p=p, training=training)
    return out if residual is None else out + residual
