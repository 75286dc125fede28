"""Fused operator API: the classes of oslo/fused_kernels_utils.py:259-479 and
:524-566 of the reference, with the same names and ``apply`` / ``is_available``
signatures, running on the gfx950 kernels of ``liboslo_amd.so``.

Differences from the reference, all widening:

* fp16, bf16 and fp32 scores up to 8192 keys are fused (the reference gates on
  fp16 and 2048, oslo/fused_kernels_utils.py:462), with no divisibility rules;
* the additive padding mask of the causal path is applied inside the kernel,
  after scaling and in fp32 (the order of the unfused attention,
  oslo/models/gpt2/modeling_gpt2.py:197-216), instead of being added into a
  copy of the scores beforehand (oslo/fused_kernels_utils.py:444-449);
* the key mask of the non-causal path is read through strides instead of being
  repeated to [B,1,Sq,Sk] (oslo/fused_kernels_utils.py:456-458), and is
  *added* as -10000 like the unfused attention does, where the reference's
  kernel *replaces* the score (oslo/fused_kernels/includes/fused_softmax.h
  :171-175); the two differ only on rows with every key masked;
* bias-GeLU and bias-dropout(-residual) are single hand-written kernels rather
  than TorchScript (oslo/fused_kernels_utils.py:259-308); their backward also
  returns the reduced bias gradient.
"""

import inspect
import threading
import weakref

import torch
from torch.autograd.function import once_differentiable

from . import _lib, kernels

_custom_kernels = None


def _needs_grad(*tensors):
    """False when autograd would record nothing: the operators then call the
    kernels directly and skip the autograd.Function machinery (a decoding step
    is bound by such per-call overheads, not by its kernels)."""
    return torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors)


def get_custom_kernels():
    """The native module (oslo/fused_kernels_utils.py:219-232). Nothing is
    compiled here: the library is built ahead of time and only loaded.
    Raises EnvironmentError if it is missing, like the reference does when its
    build fails (:226-230)."""
    global _custom_kernels
    if _custom_kernels is None:
        _lib.load()
        _custom_kernels = kernels
    return _custom_kernels


def get_datasets_builder():
    """The native index builders of the data pipeline
    (oslo/fused_kernels_utils.py:235-256). The reference returns None when its
    C++ module does not compile and falls back to Python loops; here the
    library either loads or EnvironmentError is raised."""
    from . import datasets_builder

    _lib.load()
    return datasets_builder


# ---------------------------------------------------------------------------
# softmax
# ---------------------------------------------------------------------------

class ScaledUpperTriangMaskedSoftmaxFunction(torch.autograd.Function):
    """oslo/fused_kernels_utils.py:311-331. inputs: [attn_batches, S, S]."""

    @staticmethod
    def forward(ctx, inputs, scale):
        scale_t = torch.tensor([scale])
        softmax_results = get_custom_kernels().scaled_upper_triang_masked_softmax_forward(
            inputs, scale_t[0]
        )
        ctx.save_for_backward(softmax_results, scale_t)
        return softmax_results

    @staticmethod
    @once_differentiable
    def backward(ctx, output_grads):
        softmax_results, scale_t = ctx.saved_tensors
        input_grads = get_custom_kernels().scaled_upper_triang_masked_softmax_backward(
            output_grads, softmax_results, scale_t[0]
        )
        return input_grads, None


class ScaledMaskedSoftmaxFunction(torch.autograd.Function):
    """oslo/fused_kernels_utils.py:334-352. inputs [B,H,Sq,Sk], mask bytes
    [B or 1, 1, Sq, Sk]; a set byte replaces the score by -10000."""

    @staticmethod
    def forward(ctx, inputs, mask, scale):
        scale_t = torch.tensor([scale])
        softmax_results = get_custom_kernels().scaled_masked_softmax_forward(
            inputs, mask, scale_t[0]
        )
        ctx.save_for_backward(softmax_results, scale_t)
        return softmax_results

    @staticmethod
    @once_differentiable
    def backward(ctx, output_grads):
        softmax_results, scale_t = ctx.saved_tensors
        input_grads = get_custom_kernels().scaled_masked_softmax_backward(
            output_grads, softmax_results, scale_t[0]
        )
        return input_grads, None, None


class _CausalSoftmaxWithPad(torch.autograd.Function):
    """Causal softmax of [B,H,S,S] scores with an fp32 additive key mask [B,S]
    applied inside the kernel."""

    @staticmethod
    def forward(ctx, inputs, pad_add, scale):
        y = get_custom_kernels().causal_softmax_forward(inputs, pad_add, scale)
        ctx.save_for_backward(y)
        ctx.scale = float(scale)
        return y

    @staticmethod
    @once_differentiable
    def backward(ctx, output_grads):
        (y,) = ctx.saved_tensors
        b, h, s, _ = y.shape
        dx = get_custom_kernels().scaled_upper_triang_masked_softmax_backward(
            output_grads.reshape(b * h, s, s), y.view(b * h, s, s), ctx.scale
        )
        return dx.view(b, h, s, s), None, None


class _KeyMaskedSoftmax(torch.autograd.Function):
    """Softmax of [B,H,Sq,Sk] scores with a broadcastable byte mask that adds
    -10000 to masked keys."""

    @staticmethod
    def forward(ctx, inputs, mask, scale):
        y = get_custom_kernels().masked_softmax_forward(inputs, mask, scale, kernels.MASK_ADD)
        ctx.save_for_backward(y)
        ctx.scale = float(scale)
        return y

    @staticmethod
    @once_differentiable
    def backward(ctx, output_grads):
        (y,) = ctx.saved_tensors
        dx = get_custom_kernels().scaled_masked_softmax_backward(output_grads, y, ctx.scale)
        return dx, None, None


class _CausalWindowSoftmax(torch.autograd.Function):
    """Sliding-window causal softmax of [B,H,S,S] scores, optional fp32 additive
    key mask [B,S] applied inside the kernel."""

    @staticmethod
    def forward(ctx, inputs, pad_add, scale, window):
        y = get_custom_kernels().causal_window_softmax_forward(inputs, pad_add, scale, window)
        ctx.save_for_backward(y)
        ctx.args = (float(scale), int(window))
        return y

    @staticmethod
    @once_differentiable
    def backward(ctx, output_grads):
        (y,) = ctx.saved_tensors
        scale, window = ctx.args
        dx = get_custom_kernels().causal_window_softmax_backward(output_grads, y, scale, window)
        return dx, None, None, None


class _CausalSoftmaxDropout(torch.autograd.Function):
    """Causal softmax of [B,H,S,S] scores followed by dropout of the
    probabilities, one kernel each way. Only the dropped probabilities are
    written; the backward regenerates the keep mask from the generator state
    taken in the forward and recomputes the probabilities from the scores and
    two numbers per row, so the scores (not the probabilities) are what stays
    alive between the two."""

    @staticmethod
    def forward(ctx, inputs, pad_add, scale, p):
        seed, offset = _next_philox(inputs.device)
        yd, stats = get_custom_kernels().causal_softmax_dropout_forward(inputs, pad_add, scale, p, seed, offset)
        ctx.save_for_backward(inputs, stats)
        ctx.pad_add = pad_add
        ctx.args = (float(scale), float(p), seed, offset)
        return yd

    @staticmethod
    @once_differentiable
    def backward(ctx, output_grads):
        inputs, stats = ctx.saved_tensors
        scale, p, seed, offset = ctx.args
        dx = get_custom_kernels().causal_softmax_dropout_backward(
            output_grads, inputs, stats, ctx.pad_add, scale, p, seed, offset)
        return dx, None, None, None


def _key_mask_bytes(pad_mask):
    """Any mask form -> bool, True = masked. Float masks follow the reference's
    ``.bool()`` (oslo/fused_kernels_utils.py:453-457): non-zero means masked."""
    return pad_mask if pad_mask.dtype == torch.bool else pad_mask != 0


_pad_cache = threading.local()  # .entry = (weakref to the mask, its version, the fp32 [B, Sk] form)


def _pad_additive_f32(pad_mask, bsz, sk):
    """[B or 1, 1, 1, Sk] mask (bool/uint8: True = padded -> -10000; float:
    additive as given) -> fp32 [B, Sk]. Every layer of a model passes the same
    mask tensor, so the calling thread's last conversion is kept and reused
    while that tensor is alive and unmodified. A tensor created under
    ``torch.inference_mode()`` has no version counter, so an in-place change
    of it could not be noticed: such masks are converted on every call."""
    if pad_mask.dim() != 4 or pad_mask.shape[1] != 1 or pad_mask.shape[2] != 1 \
            or pad_mask.shape[3] != sk or pad_mask.shape[0] not in (1, bsz):
        raise RuntimeError(
            "FusedScaleMaskSoftmax: with use_triang_mask the pad_mask must be "
            f"[batch or 1, 1, 1, {sk}], got {tuple(pad_mask.shape)}"
        )
    cacheable = not pad_mask.is_inference()
    if cacheable:
        entry = getattr(_pad_cache, "entry", None)
        if entry is not None:
            ref, version, converted = entry
            if ref() is pad_mask and pad_mask._version == version and tuple(converted.shape) == (bsz, sk):
                return converted
    m = pad_mask.reshape(pad_mask.shape[0], sk)
    if m.dtype in (torch.bool, torch.uint8):
        m = m.to(torch.float32) * -10000.0
    else:
        m = m.to(torch.float32)
    m = m.expand(bsz, sk).contiguous()
    if cacheable:
        _pad_cache.entry = (weakref.ref(pad_mask), pad_mask._version, m)
    return m


class FusedScaleMaskSoftmax(object):
    """
    Kernel fusion function: Scale + Mask + Softmax
    (oslo/fused_kernels_utils.py:431-479)

    Before fusion: Matmul (Q * K^T) -> Scale -> Mask -> Softmax -> Matmul (Score * V) -> ...
    After fusion: Matmul (Q * K^T) -> (Scale + Mask + Softmax) -> Matmul (Score * V) -> ...
    """

    @staticmethod
    def apply(input, pad_mask, scale, use_triang_mask):
        bsz, np, sq, sk = input.size()
        scale = scale if scale is not None else 1.0
        grad = _needs_grad(input)

        if use_triang_mask:
            pad_add = None if pad_mask is None else _pad_additive_f32(pad_mask, bsz, sk)
            if not grad:
                return get_custom_kernels().causal_softmax_forward(input, pad_add, scale)
            if pad_add is None:
                return ScaledUpperTriangMaskedSoftmaxFunction.apply(
                    input.view(-1, sq, sk), scale
                ).view(bsz, np, sq, sk)
            return _CausalSoftmaxWithPad.apply(input, pad_add, scale)

        mask = None if pad_mask is None else _key_mask_bytes(pad_mask)
        if not grad:
            return get_custom_kernels().masked_softmax_forward(input, mask, scale, kernels.MASK_ADD)
        return _KeyMaskedSoftmax.apply(input, mask, scale)

    @staticmethod
    def is_available(dtype, bsz, np, sq, sk, use_triang_mask):
        """Integer gate of oslo/fused_kernels_utils.py:461-479, widened: true
        wherever the reference's is true."""
        get_custom_kernels()  # raises if the library is missing, as the reference's gate does
        if dtype not in (torch.half, torch.bfloat16, torch.float32):
            return False
        if sk <= 0 or sk > _max_cols():
            return False
        if bsz <= 0 or np <= 0 or sq <= 0:
            return False
        if bsz * np * sq > _MAX_ROWS:  # the entry points' limit is on rows; elements are indexed with 64 bits
            return False
        # the reference also tests divisibility by get_batch_per_block here; no
        # kernel of this library needs it
        if use_triang_mask:
            return sq == sk
        return True


_softmax_max_cols = None
_MAX_ROWS = 2 ** 31 - 1


def _max_cols():
    global _softmax_max_cols
    if _softmax_max_cols is None:
        _softmax_max_cols = _lib.load().oslo_softmax_max_cols()
    return _softmax_max_cols


class FusedScaleMaskWindowSoftmax(object):
    """
    Kernel fusion function: Scale + sliding-window causal Mask + Softmax

    Not in the reference, which leaves GPT-Neo's local attention layers on the
    unfused path (oslo/models/gpt_neo/modeling_gpt_neo.py:268-272). ``apply``
    is FusedScaleMaskSoftmax.apply with use_triang_mask=True and one more
    argument: row r attends the keys max(0, r-window+1) .. r, the band
    ``tril(ones) xor tril(ones, -window)`` of :153-163.
    """

    @staticmethod
    def apply(input, pad_mask, scale, window):
        bsz, np, sq, sk = input.size()
        scale = scale if scale is not None else 1.0
        pad_add = None if pad_mask is None else _pad_additive_f32(pad_mask, bsz, sk)
        if not _needs_grad(input):
            return get_custom_kernels().causal_window_softmax_forward(input, pad_add, scale, window)
        return _CausalWindowSoftmax.apply(input, pad_add, scale, window)

    @staticmethod
    def is_available(dtype, bsz, np, sq, sk, window):
        return window >= 1 and FusedScaleMaskSoftmax.is_available(dtype, bsz, np, sq, sk, True)


class FusedScaleMaskSoftmaxDropout(object):
    """
    Kernel fusion function: Scale + Mask + Softmax + attention Dropout

    Before fusion: ... -> (Scale + Mask + Softmax) -> Dropout -> Matmul (Score * V) -> ...
    After fusion: ... -> (Scale + Mask + Softmax + Dropout) -> Matmul (Score * V) -> ...

    Not in the reference, whose fused attention runs nn.Dropout as a separate
    pass over the [B,H,S,S] probabilities (oslo/models/gptj/modeling_gptj.py
    :947-948). ``apply`` has FusedScaleMaskSoftmax.apply's arguments plus the
    dropout module's ``p`` and ``training``; causal scores in training with
    0 < p < 1 take the fused kernel, everything else is the softmax operator
    followed by torch's dropout.
    """

    @staticmethod
    def apply(input, pad_mask, scale, use_triang_mask, drop_prop, training):
        p = float(drop_prop) if training else 0.0
        if not (use_triang_mask and 0.0 < p < 1.0):
            y = FusedScaleMaskSoftmax.apply(input, pad_mask, scale, use_triang_mask)
            return y if p == 0.0 else torch.nn.functional.dropout(y, p=p, training=training)
        bsz, np, sq, sk = input.size()
        scale = scale if scale is not None else 1.0
        pad_add = None if pad_mask is None else _pad_additive_f32(pad_mask, bsz, sk)
        return _CausalSoftmaxDropout.apply(input, pad_add, scale, p)


# ---------------------------------------------------------------------------
# rotary position embedding + split heads
# ---------------------------------------------------------------------------

class _RotaryQKV(torch.autograd.Function):
    @staticmethod
    def forward(ctx, query, key, value, sin, cos, rotary_dim, offset):
        ctx.save_for_backward(sin, cos)
        ctx.args = (int(rotary_dim), int(offset))
        return get_custom_kernels().rotary_qkv_forward(query, key, value, sin, cos, rotary_dim, offset)

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_query, grad_key, grad_value):
        sin, cos = ctx.saved_tensors
        rotary_dim, offset = ctx.args
        gq, gk, gv = get_custom_kernels().rotary_qkv_backward(
            grad_query, grad_key, grad_value, sin, cos, rotary_dim, offset)
        return gq, gk, gv, None, None, None, None


class FusedRotaryPositionEmbedding(object):
    """
    Kernel fusion function: rotary position embedding + split heads

    Before fusion: view -> slice -> (x * cos) + (rotate_every_two(x) * sin) -> cat -> permute -> copy
    After fusion: view -> (Rotary + Permute)

    Not in the reference, whose fused GPT-J attention keeps the torch
    operators of oslo/models/gptj/modeling_gptj.py:49-80, :205-233. ``apply``
    takes the query / key / value projections viewed as [B, S, H, D] and the
    fp32 (sin, cos) tables of ``fixed_pos_embedding``, and returns the three
    tensors as contiguous [B, H, S, D], query and key rotated in their first
    ``rotary_dim`` features by the angle of position ``offset + s``, in fp32
    and rounded once to the input dtype.
    """

    @staticmethod
    def apply(query, key, value, sincos, rotary_dim, offset=0):
        sin, cos = sincos
        if rotary_dim == 0 and query.size(1) == 1 and all(t.is_contiguous() for t in (query, key, value)):
            # one position and nothing to rotate: [B,1,H,D] and [B,H,1,D] are the same memory
            b, _, h, d = query.shape
            return query.view(b, h, 1, d), key.view(b, h, 1, d), value.view(b, h, 1, d)
        if not _needs_grad(query, key, value):
            return get_custom_kernels().rotary_qkv_forward(query, key, value, sin, cos, rotary_dim, offset)
        return _RotaryQKV.apply(query, key, value, sin, cos, rotary_dim, offset)

    @staticmethod
    def is_available(dtype, head_dim, rotary_dim):
        if dtype not in (torch.half, torch.bfloat16, torch.float32):
            return False
        vec = 4 if dtype == torch.float32 else 8
        return head_dim % vec == 0 and rotary_dim % 2 == 0 and 0 <= rotary_dim <= head_dim


class _MergeHeads(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x):
        return get_custom_kernels().rotary_qkv_backward(None, None, x, None, None, 0)[2]

    @staticmethod
    @once_differentiable
    def backward(ctx, grad):
        return get_custom_kernels().rotary_qkv_forward(None, None, grad, None, None, 0)[2]


class FusedMergeHeads(object):
    """[B, H, S, D] -> contiguous [B, S, H*D]: the ``permute(0, 2, 1, 3)
    .contiguous().view(...)`` of ``_merge_heads``
    (oslo/models/gptj/modeling_gptj.py:129-140) as one pass of the
    transposition kernel, forward and backward."""

    @staticmethod
    def apply(x):
        b, h, s, d = x.shape
        if s == 1 and x.is_contiguous():  # one position: the permute moves nothing
            return x.view(b, 1, h * d)
        if x.stride() == (s * h * d, d, h * d, 1):  # [B, S, H, D] memory already (FusedPrefillAttention)
            return x.permute(0, 2, 1, 3).view(b, s, h * d)
        if not _needs_grad(x):
            return get_custom_kernels().rotary_qkv_backward(None, None, x, None, None, 0)[2].view(b, s, h * d)
        return _MergeHeads.apply(x).view(b, s, h * d)


class _SplitHeadsPacked(torch.autograd.Function):
    @staticmethod
    def forward(ctx, qkv, heads):
        return get_custom_kernels().split_heads_packed_forward(qkv, heads)

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_query, grad_key, grad_value):
        return get_custom_kernels().split_heads_packed_backward(grad_query, grad_key, grad_value), None


class FusedSplitHeads(object):
    """[B, S, 3*H*D] packed q|k|v projection -> query, key, value as contiguous
    [B, H, S, D]: GPT-2's ``split(split_size, dim=2)`` and three
    ``_split_heads`` permutes (oslo/models/gpt2/modeling_gpt2.py:300-306,
    :176-183) in one pass of the transposition kernel, forward and backward."""

    @staticmethod
    def apply(qkv, heads):
        if qkv.dim() == 3 and qkv.size(1) == 1 and qkv.size(2) % (3 * heads) == 0:
            # one position: the three head-major tensors are strided views of the packed row
            b, e = qkv.size(0), qkv.size(2) // 3
            return tuple(qkv[:, :, i * e:(i + 1) * e].reshape(b, heads, 1, e // heads) for i in range(3))
        if not _needs_grad(qkv):
            return get_custom_kernels().split_heads_packed_forward(qkv, heads)
        return _SplitHeadsPacked.apply(qkv, heads)

    @staticmethod
    def is_available(dtype, head_dim):
        return FusedRotaryPositionEmbedding.is_available(dtype, head_dim, 0)


# ---------------------------------------------------------------------------
# bias + GeLU
# ---------------------------------------------------------------------------

class FusedBiasGeLU(torch.autograd.Function):
    """
    Kernel fusion function: Bias + GeLU (oslo/fused_kernels_utils.py:366-380)
    """

    @staticmethod
    def forward(ctx, input, bias):
        ctx.save_for_backward(input, bias)
        return get_custom_kernels().bias_gelu_forward(input, bias)

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_output):
        input, bias = ctx.saved_tensors
        want_dbias = ctx.needs_input_grad[1]
        dy, dbias = get_custom_kernels().bias_gelu_backward(grad_output, input, bias, want_dbias)
        return dy, dbias


def _act2fn(act):
    # Only reached for activations without "gelu" in the name, as in the
    # reference (oslo/fused_kernels_utils.py:396).
    from transformers.activations import ACT2FN

    return ACT2FN[act]


class FusedBiasActivation(object):
    """
    Kernel fusion function: Bias + Activation (oslo/fused_kernels_utils.py:383-396)

    Before fusion: MLP FFN1 -> (Bias Addition -> Activation) -> MLP FFN2 -> ...
    After fusion: MLP FFN1 -> Fused Bias Activation -> MLP FFN2 -> ...
    """

    @staticmethod
    def apply(x, bias, act):
        if "gelu" in act:
            if not _needs_grad(x, bias):
                return get_custom_kernels().bias_gelu_forward(x, bias)
            return FusedBiasGeLU.apply(x, bias)
        else:
            return _act2fn(act)(x + bias)


class FusedLinearBiasActivation(object):
    """
    Kernel fusion function: Linear + Bias + GeLU in the matrix product's own launch

    Before: MLP FFN1 -> Fused Bias Activation -> MLP FFN2 -> ...
    After:  (MLP FFN1 + Bias + Activation) -> MLP FFN2 -> ...

    No counterpart in the reference, whose fused MLP runs the projection
    without its bias and then the bias-GeLU operator
    (oslo/models/gptj/modeling_gptj.py:1046-1055). The library's GEMM can add a
    bias vector and apply the tanh form of GeLU (the form the reference takes
    for every activation with "gelu" in its name, oslo/fused_kernels_utils.py:393)
    to its fp32 sums before it stores them: the product is rounded once instead
    of twice and one pass over the ``[tokens, d_ff]`` tensor is gone (GPT-J shape,
    bf16: 1.46 ms against 1.63 ms for product + kernel). Taken where autograd
    records nothing; a training step keeps the bias-GeLU kernel, whose backward
    reads the product before the bias.
    """

    @staticmethod
    def is_available(x, weight, bias, act):
        return (
            x.is_cuda and x.dim() >= 2 and bias is not None and "gelu" in act
            and x.dtype in (torch.float16, torch.bfloat16, torch.float32)
            and weight.dtype == x.dtype and bias.dtype == x.dtype
            and not _needs_grad(x, weight, bias)
        )

    @staticmethod
    def apply(x, weight, bias, act, conv1d=False):
        """``weight``: ``[out, in]`` of an ``nn.Linear``, or ``[in, out]`` of a
        ``Conv1D`` with ``conv1d=True``."""
        assert "gelu" in act
        kn = weight if conv1d else weight.t()
        out = torch._addmm_activation(bias, x.reshape(-1, x.shape[-1]), kn, use_gelu=True)
        return out.view(*x.shape[:-1], out.shape[-1])


class FusedDecodeAttention(object):
    """
    Kernel fusion function: the attention of a decoding step

    Before fusion: Matmul (q * K^T) -> (Scale + Mask + Softmax) -> Matmul (Score * V)
    After fusion: one pass over the visible keys and values

    Not in the reference, whose fused attention keeps both matmuls
    (oslo/models/gptj/modeling_gptj.py:936-951) and, its gate wanting
    ``sq == sk``, runs decoding steps unfused altogether. ``apply`` takes the
    one query per head [B, H, 1, D], the key and value caches [B, H, L, D], the
    index of the last visible key (an int, or an int64 device tensor that the
    kernel reads, for steps replayed as a graph) and an optional sliding
    window. Inference only.
    """

    @staticmethod
    def is_available(query, key, training=False, dropout_p=0.0):
        if not (query.is_cuda and query.dim() == 4 and key.dim() == 4 and query.size(2) == 1):
            return False
        if query.dtype not in (torch.half, torch.bfloat16, torch.float32) or key.dtype != query.dtype:
            return False
        if training and dropout_p > 0.0:
            return False
        head_bytes = query.size(3) * query.element_size()
        if head_bytes not in (128, 256, 512, 1024) or key.size(2) * head_bytes >= 2 ** 31:
            return False
        if key.size(2) > 2048 * (32 if head_bytes == 1024 else 64):  # the merge kernel takes 2048 splits of 32 / 64 keys
            return False
        return not _needs_grad(query, key)

    @staticmethod
    def apply(query, key, value, pos, scale, window=None, new_key=None, new_value=None):
        """``new_key``, ``new_value``: the key and value of position ``pos``
        when they are not in the caches yet; the kernel then also writes them
        into slot ``pos`` of ``key`` and ``value``."""
        scale = 1.0 if scale is None else scale
        return get_custom_kernels().attention_decode_forward(query, key, value, pos, scale, window or 0,
                                                             new_key, new_value)


class _PrefillAttention(torch.autograd.Function):
    """The prompt attention with its backward: the forward keeps q, k, v, its
    output and one fp32 number per row (the log-sum-exp); the backward
    recomputes the probabilities (and the dropout mask, from the same Philox
    seed and offset) tile by tile on the matrix cores. The backward is a raw
    kernel call: it cannot be differentiated again (a second-order request
    raises), and it always computes all three gradients, whichever of them the
    caller asked for."""

    @staticmethod
    def forward(ctx, query, key, value, pad, scale, window, p):
        seed, offset = _next_philox(query.device) if p > 0.0 else (0, 0)
        out, lse = get_custom_kernels().attention_prefill_forward(query, key, value, scale, pad, window,
                                                                  want_lse=True, p=p, seed=seed, offset=offset)
        ctx.save_for_backward(query, key, value, out, lse)
        ctx.pad = pad
        ctx.args = (float(scale), int(window), float(p), seed, offset)
        return out

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_out):
        query, key, value, out, lse = ctx.saved_tensors
        scale, window, p, seed, offset = ctx.args
        dq, dk, dv = get_custom_kernels().attention_prefill_backward(
            grad_out, query, key, value, out, lse, scale, ctx.pad, window, p, seed, offset)
        return dq, dk, dv, None, None, None, None


class FusedPrefillAttention(object):
    """
    Kernel fusion function: causal attention over a whole prompt

    Before fusion: Matmul (Q * K^T) -> (Scale + Mask + Softmax) -> Dropout -> Matmul (Score * V)
    After fusion: one kernel on the matrix cores; the [S, S] scores stay on chip

    Not in the reference, whose fused attention keeps both matmuls around the
    softmax kernel (oslo/models/gptj/modeling_gptj.py:936-951). ``apply`` takes
    query, key and value as [B, H, S, D] (views with any strides), the model's
    additive padding mask [B, 1, 1, S] or None, and the scale; it returns the
    attention output shaped [B, H, S, D] over [B, S, H, D] memory, which
    ``FusedMergeHeads`` turns into [B, S, H*D] without a copy. fp16 and bf16,
    heads of 64, 128 or 256 features; no probabilities to return. With
    gradients recorded the forward also keeps the log-sum-exp of every row and
    the backward recomputes the probabilities from it, so a training step
    keeps no [B, H, S, S] tensor between forward and backward either (heads of
    256 features: the backward's passes hand the 16-bit probabilities of the
    tiles below the diagonal to one another through a workspace of the call,
    ``kernels.PREFILL_BWD_STORE_LIMIT`` bytes at most). ``dropout_p`` > 0 (training) drops
    attention probabilities inside the kernel, with the keep mask the softmax
    kernel with fused dropout would draw from the device generator (S must be
    a multiple of 8 then).
    """

    MIN_LENGTH = 2  # one query is a decoding step (FusedDecodeAttention); from two on, one launch beats three

    @staticmethod
    def is_available(query, key, attention_mask=None, training=False, dropout_p=0.0):
        if not (query.is_cuda and query.dim() == 4 and key.dim() == 4 and key.shape == query.shape):
            return False
        if query.dtype not in (torch.half, torch.bfloat16) or key.dtype != query.dtype:
            return False
        b, _, s, d = query.shape
        if training and dropout_p > 0.0 and (s % 8 != 0 or not dropout_p < 1.0):
            return False
        if d not in (64, 128, 256) or s < FusedPrefillAttention.MIN_LENGTH or s * d * query.element_size() >= 2 ** 30:
            return False
        if attention_mask is not None and not (
                s % 4 == 0 and attention_mask.is_floating_point() and attention_mask.numel() == b * s
                and tuple(attention_mask.shape) in ((b, 1, 1, s), (b, s))):
            return False
        return True

    @staticmethod
    def apply(query, key, value, attention_mask=None, scale=None, window=None, dropout_p=0.0):
        """``window``: GPT-Neo's local attention (query i sees keys i - window < s <= i).
        ``dropout_p``: attention dropout, 0 outside training."""
        b, _, s, _ = query.shape
        pad = None if attention_mask is None else attention_mask.reshape(b, s).float()
        scale = 1.0 if scale is None else scale
        if dropout_p > 0.0 or _needs_grad(query, key, value):
            return _PrefillAttention.apply(query, key, value, pad, scale, window or 0, float(dropout_p))
        return get_custom_kernels().attention_prefill_forward(query, key, value, scale, pad, window or 0)


class FusedLinearRows(object):
    """
    Kernel fusion function: Linear + Bias + Activation for a decoding step

    Before fusion: matmul(x, weight.t()) -> (Bias Addition -> Activation)
    After fusion: one pass over the weight, bias and activation on the fp32 sums

    Not in the reference, whose fused modules keep ``torch.matmul`` and fuse
    only what follows it (oslo/models/gptj/modeling_gptj.py:1049-1065). With
    one token per sequence the matmul of a projection is a stream over the
    weight matrix for a handful of input rows, which the GEMM library runs at
    a quarter to a half of the memory bandwidth; ``apply`` runs it as such a
    stream. Inference only (``is_available`` is False when autograd would
    record the call), at most ``kernels.LINEAR_ROWS_MAX`` rows. Weights in the
    [out_features, in_features] layout of ``nn.Linear``, or with ``conv1d``
    in the [in_features, out_features] layout of GPT-2's ``Conv1D``.
    """

    @staticmethod
    def is_available(x, weight, bias=None, conv1d=False, rows_of=None):
        """``rows_of``: a tensor whose leading dimensions give the rows when ``x``
        itself does not exist yet (the second projection of a feed-forward
        module is asked about before the first has run); ``x`` may then be None."""
        ref = x if x is not None else rows_of
        if not (isinstance(ref, torch.Tensor) and ref.is_cuda and weight.is_cuda) or ref.dim() < 1 or weight.dim() != 2:
            return False
        n, k = (weight.shape[1], weight.shape[0]) if conv1d else weight.shape
        if k == 0 or ref.dtype != weight.dtype or (x is not None and x.shape[-1] != k):
            return False
        if ref.dtype not in (torch.half, torch.bfloat16, torch.float32) or not weight.is_contiguous():
            return False
        rows = ref.numel() // ref.shape[-1] if ref.shape[-1] else 0
        es = ref.element_size()
        if not 0 < rows <= kernels.LINEAR_ROWS_MAX or (k * es) % 16 or n * k * es >= 2 ** 31:
            return False
        if conv1d and (n * es) % 16:
            return False
        if x is None:
            return not _needs_grad(rows_of, weight, bias)
        return not _needs_grad(x, weight, bias)

    @staticmethod
    def apply(x, weight, bias=None, act=None, conv1d=False, residual=None):
        """``residual``: a tensor of the output's shape added last (the residual
        connection around the module), inside the same launch."""
        gelu = act is not None and "gelu" in act
        forward = get_custom_kernels().linear_rows_kn_forward if conv1d else get_custom_kernels().linear_rows_forward
        if act is not None and not gelu:
            out = _act2fn(act)(forward(x, weight, bias, False))
            return out if residual is None else out + residual
        return forward(x, weight, bias, gelu, residual)

    @staticmethod
    def project(module, x):
        """``module(x)`` for an ``nn.Linear``, through the few-row kernel
        where it applies."""
        if FusedLinearRows.is_available(x, module.weight, module.bias):
            return FusedLinearRows.apply(x, module.weight, module.bias)
        return module(x)

    @staticmethod
    def project_conv1d(module, x):
        """``module(x)`` for a GPT-2 ``Conv1D``, through the few-row kernel
        where it applies."""
        if FusedLinearRows.is_available(x, module.weight, module.bias, conv1d=True):
            return FusedLinearRows.apply(x, module.weight, module.bias, conv1d=True)
        return module(x)

    @staticmethod
    def project_many(modules, x):
        """``[m(x) for m in modules]`` for up to three ``nn.Linear`` of one
        shape (the query, key and value projections), in one launch where the
        few-row kernel applies."""
        first = modules[0]
        if (len(modules) <= 3 and all(m.weight.shape == first.weight.shape for m in modules)
                and all(FusedLinearRows.is_available(x, m.weight, m.bias) for m in modules)):
            return get_custom_kernels().linear_rows_forward_multi(
                x, [m.weight for m in modules], [m.bias for m in modules])
        return [m(x) for m in modules]


# ---------------------------------------------------------------------------
# bias + dropout (+ residual)
# ---------------------------------------------------------------------------

PHILOX_WORDS_PER_CALL = 4  # generator offset one dropout call consumes


def _next_philox(device):
    """Takes (seed, offset) from the device's default generator and advances it,
    the way a torch random op does."""
    gen = torch.cuda.default_generators[device.index if device.index is not None
                                        else torch.cuda.current_device()]
    seed = gen.initial_seed()
    offset = gen.get_offset()
    gen.set_offset(offset + PHILOX_WORDS_PER_CALL)
    return seed, offset


class _BiasDropoutAdd(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, bias, residual, p, residual2=None):
        if p > 0.0:
            seed, offset = _next_philox(x.device)
        else:
            seed, offset = 0, 0
        ctx.p, ctx.seed, ctx.offset = p, seed, offset
        return get_custom_kernels().bias_dropout_add_forward(x, bias, residual, p, seed, offset, residual2)

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_output):
        want_dbias = ctx.needs_input_grad[1]
        dx = dbias = None
        if ctx.needs_input_grad[0] or want_dbias:
            dx, dbias = get_custom_kernels().bias_dropout_add_backward(
                grad_output, ctx.p, ctx.seed, ctx.offset, want_dbias
            )
        dres = grad_output if ctx.needs_input_grad[2] else None
        dres2 = grad_output if ctx.needs_input_grad[4] else None
        return dx, dbias, dres, None, dres2


def _bias_dropout_add(x, bias, residual, training, drop_prop, residual2=None):
    p = float(drop_prop) if training else 0.0
    if not x.is_cuda:
        raise RuntimeError(f"expected a tensor on a ROCm device, got {x.device} (this library has no CPU path)")
    if p < 0.0 or p > 1.0:
        raise ValueError(f"dropout probability has to be between 0 and 1, but got {p}")
    if residual is None and residual2 is not None:
        residual, residual2 = residual2, None
    if p == 1.0:  # everything dropped: F.dropout returns zeros
        out = torch.zeros_like(x)
        out = out if residual is None else out + residual
        return out if residual2 is None else out + residual2
    if p == 0.0 and bias is None and residual is None:
        return x  # nothing to add and nothing to drop
    if not _needs_grad(x, bias, residual, residual2):
        seed, offset = _next_philox(x.device) if p > 0.0 else (0, 0)
        return get_custom_kernels().bias_dropout_add_forward(x, bias, residual, p, seed, offset, residual2)
    return _BiasDropoutAdd.apply(x, bias, residual, p, residual2)


class FusedBiasDropout(object):
    """
    Kernel fusion function: Bias + Dropout (oslo/fused_kernels_utils.py:399-412)

    Before fusion: MLP FFN2 -> (Bias Addition -> Dropout) -> Residual Addition ->. ..
    After fusion: MLP FFN2 -> Fused Bias Dropout -> Residual Addition -> ...
    """

    @staticmethod
    def apply(x, bias, training, drop_prop):
        return _bias_dropout_add(x, bias, None, training, drop_prop)


class FusedBiasDropoutResidual(object):
    """
    Kernel fusion function: Bias + Dropout + Residual
    (oslo/fused_kernels_utils.py:415-428)

    Before fusion: MLP FFN2 -> (Bias Addition -> Dropout -> Residual Addition) -> LayerNorm -> ...
    After fusion: MLP FFN2 -> Fused Bias Dropout Residual -> LayerNorm -> ...

    ``residual2`` (not in the reference's signature, optional): a second tensor
    added in the same pass, for blocks whose output is a sum of three terms
    (GPT-J: attention output + feed-forward output + residual stream). The sum
    is formed in fp32 and rounded once.
    """

    @staticmethod
    def apply(x, bias, residual, training, drop_prop, residual2=None):
        return _bias_dropout_add(x, bias, residual, training, drop_prop, residual2)


# ---------------------------------------------------------------------------
# repeated n-gram blocking for generation
# ---------------------------------------------------------------------------

class NGramRepeatBlockFunction(torch.autograd.Function):
    """oslo/fused_kernels_utils.py:355-363."""

    @staticmethod
    def forward(ctx, tokens, lprobs, bsz, step, beam_size, no_repeat_ngram_size):
        return get_custom_kernels().ngram_repeat_block_forward(
            tokens, lprobs, bsz, step, beam_size, no_repeat_ngram_size
        )

    def backward(*args):
        raise NotImplementedError


def _banned_tokens_on_host(ngram_size, input_ids):
    """Per hypothesis, the tokens that would complete an n-gram already in it:
    those that followed an earlier occurrence of its last ngram_size - 1 tokens
    (what ``_calc_banned_ngram_tokens`` gives the reference's host branch,
    oslo/fused_kernels_utils.py:506-512)."""
    cur_len = input_ids.shape[-1]
    if cur_len + 1 < ngram_size:
        return [[] for _ in range(input_ids.shape[0])]
    banned = []
    for row in input_ids.tolist():
        last = row[cur_len + 1 - ngram_size:]
        banned.append([row[i + ngram_size - 1] for i in range(cur_len - ngram_size + 1)
                       if row[i:i + ngram_size - 1] == last])
    return banned


class FusedNoRepeatNGramLogitsProcessor(object):
    """Logits processor that bans every token that would repeat an n-gram
    (oslo/fused_kernels_utils.py:482-521). Callable as
    ``processor(input_ids, scores)`` like a HuggingFace LogitsProcessor.
    Device tensors go to the kernel and nowhere else (a missing library raises).
    Host tensors are the reference's other branch (:505-517), which is host
    code there too: the bans are worked out in Python and written into
    ``scores`` in place."""

    def __init__(self, ngram_size: int, batch_size: int, beam_size: int):
        if not isinstance(ngram_size, int) or ngram_size <= 0:
            raise ValueError(
                f"`ngram_size` has to be a strictly positive integer, but is {ngram_size}"
            )
        self.ngram_size = ngram_size
        self.batch_size = batch_size
        self.beam_size = beam_size

    def __call__(self, input_ids, scores):
        if input_ids.is_cuda != scores.is_cuda:
            raise RuntimeError(
                "FusedNoRepeatNGramLogitsProcessor: input_ids and scores must both be on the "
                f"device or both on the host, got {input_ids.device} and {scores.device}"
            )
        if not input_ids.is_cuda:
            for i, tokens in enumerate(_banned_tokens_on_host(self.ngram_size, input_ids)):
                scores[i, tokens] = -float("inf")
            return scores
        cur_len = input_ids.shape[-1]
        return NGramRepeatBlockFunction.apply(
            input_ids.contiguous(),
            scores.float().contiguous(),
            self.batch_size,
            cur_len - 1,
            self.beam_size,
            self.ngram_size,
        )


class FusedKernelMixin(object):
    """oslo/fused_kernels_utils.py:524-566: swaps the class of every fusable
    sub-module for its fused subclass; parameters and buffers are untouched."""

    def fuse(self, modules=None):
        user_modules = modules

        assert user_modules is None or isinstance(
            user_modules, list
        ), "Param `modules` must be type of List[Class]."

        if not getattr(self, "is_fusable", False):
            raise RuntimeError(
                "This model doesn't support kernel fusion. please check the document."
            )

        for policy in self.get_layer_policies():
            fused_modules = policy.fused_modules()

            if user_modules is not None:
                for user_module in user_modules:
                    assert user_module in fused_modules, (
                        f"Module {user_module} can't be fused! "
                        f"{self.__class__.__qualname__} only supports {list(fused_modules.keys())}"
                    )
                    assert inspect.isclass(user_module), (
                        f"The element in the ``modules`` must be Class type. "
                        f"but you input {type(user_module)}"
                    )

            for model_module in self.modules():
                cls = model_module.__class__
                if cls not in fused_modules:
                    continue
                if user_modules is not None and cls not in user_modules:
                    continue  # not in the list the user asked for
                model_module.__class__ = fused_modules[cls]
                setattr(model_module, "config", self.config)

        # beyond the reference: with everything fused, a decoding step also
        # streams the output head's weight through the few-row kernel
        self.fused_lm_head = user_modules is None
        return self
