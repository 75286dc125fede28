"""Tensor-level front of ``liboslo_amd.so``: the functions of the reference's
native module ``oslo_kernels`` (oslo/fused_kernels/bindings/pybind_kernels.cpp
:159-177) with the same names, argument order and error behaviour, plus the
wider entry points the fused operators of this package use.

Every function takes device tensors, allocates its output with torch, and
enqueues one kernel on torch's current stream of that device. There is no CPU
implementation: a CPU tensor is rejected with ``RuntimeError``.
"""

import ctypes

import torch

from . import _lib

_DTYPE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}
MASK_ADD = 0
MASK_REPLACE = 1
EPILOGUE_NONE = 0
EPILOGUE_GELU_TANH = 1
LINEAR_ROWS_MAX = 8  # oslo_linear_rows_max()


def _require(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def _dtype_code(t, what):
    _require(t.dtype in _DTYPE, f"{what}: only fp16, bf16 and fp32 are supported, got {t.dtype}")
    return _DTYPE[t.dtype]


def _device_tensor(t, what, like=None):
    _require(isinstance(t, torch.Tensor), f"{what}: expected a tensor")
    _require(t.is_cuda, f"{what}: expected a tensor on a ROCm device, got {t.device} "
                        "(this library has no CPU path)")
    if like is not None:
        _require(t.device == like.device, f"{what} is on {t.device}, the input on {like.device}")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(t):
    """torch's current stream on t's device, as the library's stream argument."""
    if _raw_stream is not None:
        return ctypes.c_void_p(_raw_stream(t.device.index))
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


class _NoSwitch(object):
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_SWITCH = _NoSwitch()


def _on_device(t):
    """Context that makes t's device current for the launch; nothing to do (and
    nothing to pay) when it already is."""
    if t.device.index == torch.cuda.current_device():
        return _NO_SWITCH
    return torch.cuda.device(t.device)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


# ---------------------------------------------------------------------------
# the reference's five softmax symbols
# ---------------------------------------------------------------------------

def get_batch_per_block(query_seq_len, key_seq_len, batches, attn_heads):
    """oslo/fused_kernels/bindings/pybind_kernels.cpp:77-83."""
    return _lib.load().oslo_get_batch_per_block(
        int(query_seq_len), int(key_seq_len), int(batches), int(attn_heads))


def scaled_upper_triang_masked_softmax_forward(input, scale_factor):
    """oslo/fused_kernels/bindings/pybind_kernels.cpp:98-105: input [attn_batches, S, S]."""
    _require(input.dim() == 3, "expected 3D tensor")
    return causal_softmax_forward(input.unsqueeze(0), None, scale_factor).squeeze(0)


def scaled_upper_triang_masked_softmax_backward(output_grads, softmax_results, scale_factor):
    """oslo/fused_kernels/bindings/pybind_kernels.cpp:107-123. Writes the input
    gradient over ``output_grads`` (when it is contiguous) and returns it, as
    the reference does (oslo/fused_kernels/fused_triang_softmax.cu:84-95)."""
    _require(output_grads.dim() == 3, "expected 3D tensor")
    _require(softmax_results.dim() == 3, "expected 3D tensor")
    _device_tensor(output_grads, "output_grads")
    _device_tensor(softmax_results, "softmax_results", output_grads)
    code = _dtype_code(output_grads, "output_grads")
    _require(softmax_results.dtype == output_grads.dtype, "output_grads and softmax_results differ in dtype")
    _require(softmax_results.shape == output_grads.shape, "output_grads and softmax_results differ in shape")
    bh, sq, sk = output_grads.shape
    _require(sq == sk, "causal softmax needs square score matrices")
    g = output_grads.contiguous()
    y = softmax_results.contiguous()
    with _on_device(g):
        _lib.check(_lib.load().oslo_softmax_causal_bwd(
            _ptr(g), _ptr(g), _ptr(y), float(scale_factor), bh, sk, code, _stream(g)))
    return g


def scaled_masked_softmax_forward(input, mask, scale_factor):
    """oslo/fused_kernels/bindings/pybind_kernels.cpp:46-57: input [B,H,Sq,Sk],
    mask [B or 1, 1, Sq, Sk] bytes; a set byte replaces the score by -10000
    (oslo/fused_kernels/includes/fused_softmax.h:171-175)."""
    _require(input.dim() == 4, "expected 4D tensor")
    _require(mask.dim() == 4, "expected 4D tensor")
    return masked_softmax_forward(input, mask, scale_factor, MASK_REPLACE)


def scaled_masked_softmax_backward(output_grads, softmax_results, scale_factor):
    """oslo/fused_kernels/bindings/pybind_kernels.cpp:59-75; in place over
    ``output_grads`` (oslo/fused_kernels/fused_softmax.cu:103-114)."""
    _require(output_grads.dim() == 4, "expected 4D tensor")
    _require(softmax_results.dim() == 4, "expected 4D tensor")
    _device_tensor(output_grads, "output_grads")
    _device_tensor(softmax_results, "softmax_results", output_grads)
    code = _dtype_code(output_grads, "output_grads")
    _require(softmax_results.dtype == output_grads.dtype, "output_grads and softmax_results differ in dtype")
    _require(softmax_results.shape == output_grads.shape, "output_grads and softmax_results differ in shape")
    g = output_grads.contiguous()
    y = softmax_results.contiguous()
    sk = g.shape[-1]
    rows = g.numel() // sk if sk else 0
    with _on_device(g):
        _lib.check(_lib.load().oslo_softmax_masked_bwd(
            _ptr(g), _ptr(g), _ptr(y), float(scale_factor), rows, sk, code, _stream(g)))
    return g


def ngram_repeat_block_forward(tokens, lprobs, bsz, step, beam_size, no_repeat_ngram_size):
    """oslo/fused_kernels/bindings/pybind_kernels.cpp:143-157: tokens int64
    [bsz*beam_size, len], lprobs fp32 [bsz*beam_size, vocab]; bans in place and
    returns lprobs."""
    _device_tensor(tokens, "tokens")
    _device_tensor(lprobs, "lprobs", tokens)
    _require(tokens.is_contiguous(), "tokens must be contiguous")
    _require(lprobs.is_contiguous(), "lprobs must be contiguous")
    _require(tokens.dtype == torch.int64, "tokens must be int64")
    _require(lprobs.dtype == torch.float32, "lprobs must be float32")
    _require(tokens.dim() == 2 and lprobs.dim() == 2, "expected 2D tensors")
    assert bsz > 0 and step >= 0 and beam_size > 0 and no_repeat_ngram_size > 0
    rows = bsz * beam_size
    _require(tokens.shape[0] == rows and lprobs.shape[0] == rows,
             "tokens and lprobs must have bsz * beam_size rows")
    with _on_device(lprobs):
        _lib.check(_lib.load().oslo_ngram_repeat_block(
            _ptr(lprobs), _ptr(tokens), rows, tokens.shape[1], int(step), lprobs.shape[1],
            int(no_repeat_ngram_size), _stream(lprobs)))
    return lprobs


# ---------------------------------------------------------------------------
# wider entry points
# ---------------------------------------------------------------------------

def causal_softmax_forward(input, pad_add, scale_factor):
    """input [B,H,S,S]; pad_add None or fp32 [B,S] added after scaling."""
    _device_tensor(input, "input")
    _require(input.dim() == 4, "expected 4D tensor")
    code = _dtype_code(input, "input")
    b, h, sq, sk = input.shape
    _require(sq == sk, "causal softmax needs square score matrices")
    x = input.contiguous()
    if pad_add is not None:
        _device_tensor(pad_add, "pad_add", input)
        _require(pad_add.dtype == torch.float32 and tuple(pad_add.shape) == (b, sk),
                 "pad_add must be fp32 [batch, S]")
        pad_add = pad_add.contiguous()
    y = torch.empty_like(x, requires_grad=False)
    with _on_device(x):
        _lib.check(_lib.load().oslo_softmax_causal_fwd(
            _ptr(y), _ptr(x), _ptr(pad_add), float(scale_factor), b, h, sk, code, _stream(x)))
    return y


def causal_window_softmax_forward(input, pad_add, scale_factor, window):
    """input [B,H,S,S]; row r attends the keys max(0, r-window+1) .. r."""
    _device_tensor(input, "input")
    _require(input.dim() == 4, "expected 4D tensor")
    code = _dtype_code(input, "input")
    b, h, sq, sk = input.shape
    _require(sq == sk, "causal softmax needs square score matrices")
    x = input.contiguous()
    pad_add = _pad_add_arg(pad_add, b, sk, input)
    y = torch.empty_like(x, requires_grad=False)
    with _on_device(x):
        _lib.check(_lib.load().oslo_softmax_causal_window_fwd(
            _ptr(y), _ptr(x), _ptr(pad_add), float(scale_factor), int(window), b, h, sk, code, _stream(x)))
    return y


def causal_window_softmax_backward(output_grads, softmax_results, scale_factor, window):
    """[B,H,S,S] gradients; written over ``output_grads`` when it is contiguous."""
    _device_tensor(output_grads, "output_grads")
    _device_tensor(softmax_results, "softmax_results", output_grads)
    code = _dtype_code(output_grads, "output_grads")
    _require(softmax_results.dtype == output_grads.dtype and softmax_results.shape == output_grads.shape,
             "output_grads and softmax_results differ in dtype or shape")
    _require(output_grads.dim() == 4 and output_grads.shape[-1] == output_grads.shape[-2], "expected [B,H,S,S]")
    b, h, s, _ = output_grads.shape
    g = output_grads.contiguous()
    y = softmax_results.contiguous()
    with _on_device(g):
        _lib.check(_lib.load().oslo_softmax_causal_window_bwd(
            _ptr(g), _ptr(g), _ptr(y), float(scale_factor), int(window), b * h, s, code, _stream(g)))
    return g


def _pad_add_arg(pad_add, b, sk, like):
    if pad_add is None:
        return None
    _device_tensor(pad_add, "pad_add", like)
    _require(pad_add.dtype == torch.float32 and tuple(pad_add.shape) == (b, sk),
             "pad_add must be fp32 [batch, S]")
    return pad_add.contiguous()


def causal_softmax_dropout_forward(input, pad_add, scale_factor, p, seed, offset):
    """Causal softmax + attention dropout in one pass. Returns (probs_after_
    dropout, row_stats): the probabilities themselves are not stored; the
    backward recomputes them from ``input`` and the fp32 [B,H,S,2] row_stats
    (row maximum and reciprocal row sum)."""
    _device_tensor(input, "input")
    _require(input.dim() == 4, "expected 4D tensor")
    code = _dtype_code(input, "input")
    b, h, sq, sk = input.shape
    _require(sq == sk, "causal softmax needs square score matrices")
    x = input.contiguous()
    pad_add = _pad_add_arg(pad_add, b, sk, input)
    yd = torch.empty_like(x, requires_grad=False)
    stats = torch.empty((b, h, sq, 2), dtype=torch.float32, device=x.device)
    with _on_device(x):
        _lib.check(_lib.load().oslo_softmax_causal_dropout_fwd(
            _ptr(yd), _ptr(stats), _ptr(x), _ptr(pad_add), float(scale_factor), float(p),
            int(seed), int(offset), b, h, sk, code, _stream(x)))
    return yd, stats


def causal_softmax_dropout_backward(output_grads, input, row_stats, pad_add, scale_factor, p, seed, offset):
    """output_grads: gradient of the probabilities after dropout, [B,H,S,S];
    overwritten with the input gradient when contiguous, like the plain
    backward. input, row_stats, pad_add: the forward's."""
    _device_tensor(output_grads, "output_grads")
    _device_tensor(input, "input", output_grads)
    _device_tensor(row_stats, "row_stats", output_grads)
    code = _dtype_code(output_grads, "output_grads")
    _require(input.dtype == output_grads.dtype and input.shape == output_grads.shape,
             "output_grads and input differ in dtype or shape")
    _require(output_grads.dim() == 4 and output_grads.shape[-1] == output_grads.shape[-2],
             "expected [B,H,S,S]")
    b, h, s, _ = output_grads.shape
    _require(row_stats.dtype == torch.float32 and tuple(row_stats.shape) == (b, h, s, 2)
             and row_stats.is_contiguous(), "row_stats must be contiguous fp32 [B,H,S,2]")
    g = output_grads.contiguous()
    x = input.contiguous()
    pad_add = _pad_add_arg(pad_add, b, s, output_grads)
    with _on_device(g):
        _lib.check(_lib.load().oslo_softmax_causal_dropout_bwd(
            _ptr(g), _ptr(g), _ptr(x), _ptr(row_stats), _ptr(pad_add), float(scale_factor), float(p),
            int(seed), int(offset), b, h, s, code, _stream(g)))
    return g


def masked_softmax_forward(input, mask, scale_factor, mask_mode=MASK_ADD):
    """input [B,H,Sq,Sk]; mask None or bool/uint8 [B or 1, 1, Sq or 1, Sk]
    (size-1 dimensions are broadcast by stride, not copied)."""
    _device_tensor(input, "input")
    _require(input.dim() == 4, "expected 4D tensor")
    code = _dtype_code(input, "input")
    b, h, sq, sk = input.shape
    x = input.contiguous()
    msb = msq = 0
    if mask is not None:
        _device_tensor(mask, "mask", input)
        _require(mask.dim() == 4, "expected 4D tensor")
        _require(mask.dtype in (torch.bool, torch.uint8), "mask must be bool or uint8")
        mb, mh, mq, mk = mask.shape
        _require(mb in (1, b), "mask batch must be 1 or the input's batch")
        _require(mh == 1, "mask must have one head")
        _require(mq in (1, sq), "mask rows must be 1 or the input's query length")
        _require(mk == sk, "mask and input differ in key length")
        mask = mask.contiguous()
        if mask.dtype == torch.bool:
            mask = mask.view(torch.uint8)
        msb = mq * mk if mb == b and b > 1 else 0
        msq = mk if mq == sq and sq > 1 else 0
    y = torch.empty_like(x, requires_grad=False)
    with _on_device(x):
        _lib.check(_lib.load().oslo_softmax_masked_fwd(
            _ptr(y), _ptr(x), _ptr(mask), msb, msq, int(mask_mode), float(scale_factor),
            b, h, sq, sk, code, _stream(x)))
    return y


def _as_rows_cols(t, bias, what):
    _device_tensor(t, what)
    code = _dtype_code(t, what)
    _require(t.dim() >= 1, f"{what}: expected at least 1 dimension")
    cols = t.shape[-1]
    if bias is not None:
        _device_tensor(bias, "bias", t)
        _require(bias.dim() == 1 and bias.shape[0] == cols, "bias must be [last dimension of the input]")
        _require(bias.dtype == t.dtype, "bias and input differ in dtype")
    rows = t.numel() // cols if cols else 0
    return rows, cols, code


def _workspace(rows, cols, device):
    nbytes = _lib.load().oslo_colsum_workspace_bytes(rows, cols)
    return torch.empty(max(nbytes // 4, 1), dtype=torch.float32, device=device)


def bias_gelu_forward(y, bias):
    rows, cols, code = _as_rows_cols(y, bias, "input")
    y = y.contiguous()
    bias = bias.contiguous()
    out = torch.empty_like(y, requires_grad=False)
    with _on_device(y):
        _lib.check(_lib.load().oslo_bias_gelu_fwd(
            _ptr(out), _ptr(y), _ptr(bias), rows, cols, code, _stream(y)))
    return out


def bias_gelu_backward(grad, y, bias, want_dbias=True):
    """Returns (d_input, d_bias or None); d_input is a new tensor."""
    rows, cols, code = _as_rows_cols(y, bias, "input")
    _device_tensor(grad, "grad", y)
    _require(grad.shape == y.shape and grad.dtype == y.dtype, "grad and input differ in shape or dtype")
    grad = grad.contiguous()
    y = y.contiguous()
    bias = bias.contiguous()
    dy = torch.empty_like(y, requires_grad=False)
    dbias = torch.empty_like(bias, requires_grad=False) if want_dbias else None
    ws = _workspace(rows, cols, y.device) if want_dbias else None
    with _on_device(y):
        _lib.check(_lib.load().oslo_bias_gelu_bwd(
            _ptr(dy), _ptr(dbias), _ptr(ws), _ptr(grad), _ptr(y), _ptr(bias),
            rows, cols, code, _stream(y)))
    return dy, dbias


def bias_dropout_add_forward(x, bias, residual, p, seed, offset, residual2=None):
    """dropout(x + bias, p) + residual (+ residual2): every term but x may be
    None; a second residual needs a first. The sum is formed in fp32 and
    rounded once."""
    rows, cols, code = _as_rows_cols(x, bias, "input")
    x = x.contiguous()
    if bias is not None:
        bias = bias.contiguous()
    _require(residual2 is None or residual is not None, "a second residual without a first")
    res = []
    for what, r in (("residual", residual), ("residual2", residual2)):
        if r is not None:
            _device_tensor(r, what, x)
            _require(r.shape == x.shape and r.dtype == x.dtype, f"{what} and input differ in shape or dtype")
            r = r.contiguous()
        res.append(r)
    out = torch.empty_like(x, requires_grad=False)
    with _on_device(x):
        if res[1] is None:
            _lib.check(_lib.load().oslo_bias_dropout_add_fwd(
                _ptr(out), _ptr(x), _ptr(bias), _ptr(res[0]), float(p), int(seed), int(offset),
                rows, cols, code, _stream(x)))
        else:
            _lib.check(_lib.load().oslo_bias_dropout_add2_fwd(
                _ptr(out), _ptr(x), _ptr(bias), _ptr(res[0]), _ptr(res[1]), float(p), int(seed), int(offset),
                rows, cols, code, _stream(x)))
    return out


def bias_dropout_add_backward(grad, p, seed, offset, want_dbias=True):
    """Returns (d_input, d_bias or None). The residual's gradient is ``grad``."""
    rows, cols, code = _as_rows_cols(grad, None, "grad")
    grad = grad.contiguous()
    dx = torch.empty_like(grad, requires_grad=False)
    dbias = torch.empty(cols, dtype=grad.dtype, device=grad.device) if want_dbias else None
    ws = _workspace(rows, cols, grad.device) if want_dbias else None
    with _on_device(grad):
        _lib.check(_lib.load().oslo_bias_dropout_add_bwd(
            _ptr(dx), _ptr(dbias), _ptr(ws), _ptr(grad), float(p), int(seed), int(offset),
            rows, cols, code, _stream(grad)))
    return dx, dbias


# ---------------------------------------------------------------------------
# rotary position embedding + split-heads transposition
# ---------------------------------------------------------------------------

def _rotary_call(tensors, sin, cos, rotary_dim, offset, inverse):
    first = next((t for t in tensors if t is not None), None)
    _require(first is not None, "rotary: at least one of query, key and value is needed")
    _device_tensor(first, "rotary input")
    code = _dtype_code(first, "rotary input")
    _require(first.dim() == 4, "expected 4D tensors")
    if inverse:
        b, h, s, d = first.shape
        out_shape = (b, s, h, d)
    else:
        b, s, h, d = first.shape
        out_shape = (b, h, s, d)
    ins, outs = [], []
    for t in tensors:
        if t is None:
            ins.append(None)
            outs.append(None)
            continue
        _device_tensor(t, "rotary input", first)
        _require(t.shape == first.shape and t.dtype == first.dtype, "q, k and v differ in shape or dtype")
        ins.append(t.contiguous())
        outs.append(torch.empty(out_shape, dtype=t.dtype, device=t.device))
    positions = 0
    if rotary_dim > 0:
        _device_tensor(sin, "sin", first)
        _device_tensor(cos, "cos", first)
        _require(sin.dtype == torch.float32 and cos.dtype == torch.float32 and sin.dim() == 2
                 and sin.shape == cos.shape and sin.shape[1] == rotary_dim // 2,
                 "sin and cos must be fp32 [positions, rotary_dim/2]")
        sin, cos = sin.contiguous(), cos.contiguous()
        positions = sin.shape[0]
    else:
        sin = cos = None
    with _on_device(first):
        _lib.check(_lib.load().oslo_rotary_qkv(
            _ptr(outs[0]), _ptr(outs[1]), _ptr(outs[2]), _ptr(ins[0]), _ptr(ins[1]), _ptr(ins[2]),
            _ptr(sin), _ptr(cos), positions, b, s, h, d, 0, int(rotary_dim), int(offset),
            1 if inverse else 0, code, _stream(first)))
    return tuple(outs)


def linear_rows_forward(x, weight, bias=None, gelu=False, residual=None):
    """x [..., K] with at most LINEAR_ROWS_MAX rows in all, weight [N, K] (the
    layout of nn.Linear), bias None or [N] -> act(x @ weight.t() + bias) as
    [..., N], act = tanh-form GeLU if ``gelu``; ``residual`` [..., N] is added
    last. One pass over the weight; sums and the epilogue in fp32
    (oslo/models/gptj/modeling_gptj.py:1049-1065 for a decoding step)."""
    return linear_rows_forward_multi(x, (weight,), (bias,), gelu, residual)[0]


def _residual_like(residual, shape, x):
    if residual is None:
        return None
    _device_tensor(residual, "residual", x)
    _require(tuple(residual.shape) == tuple(shape) and residual.dtype == x.dtype,
             "residual must have the output's shape and dtype")
    return residual.contiguous()


def linear_rows_kn_forward(x, weight, bias=None, gelu=False, residual=None):
    """The same with the weight stored [K, N], the layout of GPT-2's Conv1D:
    act(x @ weight + bias) + residual (oslo/models/gpt2/modeling_gpt2.py
    :1553-1567 for a decoding step)."""
    _device_tensor(x, "x")
    _device_tensor(weight, "weight", x)
    code = _dtype_code(x, "x")
    _require(weight.dim() == 2, "weight must be [in_features, out_features]")
    _require(weight.dtype == x.dtype, "weight and x differ in dtype")
    k, n = weight.shape
    _require(x.dim() >= 1 and x.shape[-1] == k, "x must be [..., in_features]")
    m = x.numel() // k if k else 0
    if bias is not None:
        _device_tensor(bias, "bias", x)
        _require(bias.dim() == 1 and bias.shape[0] == n and bias.dtype == x.dtype,
                 "bias must be [out_features] of the input's dtype")
        bias = bias.contiguous()
    x2, w = x.contiguous(), weight.contiguous()
    out = torch.empty(x.shape[:-1] + (n,), dtype=x.dtype, device=x.device)
    residual = _residual_like(residual, out.shape, x)
    with _on_device(x):
        _lib.check(_lib.load().oslo_linear_rows_kn_fwd(
            _ptr(out), _ptr(x2), _ptr(w), _ptr(bias), _ptr(residual), m, n, k,
            EPILOGUE_GELU_TANH if gelu else EPILOGUE_NONE, code, _stream(x)))
    return out


def linear_rows_forward_multi(x, weights, biases=None, gelu=False, residual=None):
    """One to three layers of the same shape applied to the same x in one
    launch (the query, key and value projections): a list of outputs.
    ``residual`` goes with a single layer only."""
    count = len(weights)
    _require(residual is None or count == 1, "a residual goes with one layer")
    _require(1 <= count <= 3, "one to three layers per launch")
    biases = (None,) * count if biases is None else tuple(biases)
    _require(len(biases) == count, "one bias (or None) per weight")
    _device_tensor(x, "x")
    code = _dtype_code(x, "x")
    n, k = weights[0].shape if weights[0].dim() == 2 else (0, 0)
    _require(x.dim() >= 1 and x.shape[-1] == k, "x must be [..., in_features]")
    m = x.numel() // k if k else 0
    ws, bs = [], []
    for w, b in zip(weights, biases):
        _device_tensor(w, "weight", x)
        _require(w.dim() == 2 and tuple(w.shape) == (n, k), "weights must be [out_features, in_features], all alike")
        _require(w.dtype == x.dtype, "weight and x differ in dtype")
        ws.append(w.contiguous())
        if b is not None:
            _device_tensor(b, "bias", x)
            _require(b.dim() == 1 and b.shape[0] == n and b.dtype == x.dtype,
                     "bias must be [out_features] of the input's dtype")
            b = b.contiguous()
        bs.append(b)
    x2 = x.contiguous()
    outs = [torch.empty(x.shape[:-1] + (n,), dtype=x.dtype, device=x.device) for _ in range(count)]
    epilogue = EPILOGUE_GELU_TANH if gelu else EPILOGUE_NONE
    residual = _residual_like(residual, outs[0].shape, x)
    with _on_device(x):
        if count == 1:
            _lib.check(_lib.load().oslo_linear_rows_fwd(
                _ptr(outs[0]), _ptr(x2), _ptr(ws[0]), _ptr(bs[0]), _ptr(residual), m, n, k, epilogue, code,
                _stream(x)))
        else:
            table = ctypes.c_void_p * count
            _lib.check(_lib.load().oslo_linear_rows_fwd_multi(
                table(*(o.data_ptr() for o in outs)), _ptr(x2), table(*(w.data_ptr() for w in ws)),
                table(*(None if b is None else b.data_ptr() for b in bs)), count, m, n, k, epilogue, code,
                _stream(x)))
    return outs


def _heads_side_by_side(t):
    """[B, H, 1, D] whose heads of one sequence are consecutive runs of D elements."""
    b, h, _, d = t.shape
    return t.stride(3) == 1 and (h == 1 or t.stride(1) == d) and (b == 1 or t.stride(0) >= h * d)


def attention_decode_forward(query, key, value, pos, scale, window=0, new_key=None, new_value=None):
    """query [B, H, 1, D]; key, value [B, H, L, D] caches; attends keys
    first..last, last = ``pos`` (an int, or an int64 device tensor of one
    element that the kernel reads), first = last - window + 1 for window > 0,
    else 0. Returns softmax(scale * q k^T) v as [B, H, 1, D]
    (oslo/models/gptj/modeling_gptj.py:936-951 for a query length of 1).
    ``new_key``, ``new_value`` [B, H, 1, D]: the key and value of position
    ``pos``, not yet in the caches; the kernel uses them and writes them into
    slot ``pos`` of ``key`` and ``value``, which must then be contiguous. They
    may be strided between sequences (views of a packed projection) as long as
    a sequence's heads lie side by side."""
    _device_tensor(query, "query")
    _device_tensor(key, "key", query)
    _device_tensor(value, "value", query)
    code = _dtype_code(query, "query")
    _require(query.dim() == 4 and key.dim() == 4 and value.dim() == 4, "expected 4D tensors")
    b, h, sq, d = query.shape
    _require(sq == 1, "one query per sequence and head")
    _require(key.shape == value.shape and tuple(key.shape[:2]) == (b, h) and key.shape[3] == d,
             "key and value must be [B, H, L, D] caches of the query's heads")
    _require(key.dtype == query.dtype and value.dtype == query.dtype, "query, key and value differ in dtype")
    cap = key.shape[2]
    q, k, v = query.contiguous(), key.contiguous(), value.contiguous()
    _require((new_key is None) == (new_value is None), "new_key and new_value go together")
    if new_key is not None:
        _require(key.is_contiguous() and value.is_contiguous(), "caches that take a new key must be contiguous")
        for t, what in ((new_key, "new_key"), (new_value, "new_value")):
            _device_tensor(t, what, query)
            _require(t.shape == query.shape and t.dtype == query.dtype, f"{what} must be like the query")
        if not (_heads_side_by_side(new_key) and _heads_side_by_side(new_value)
                and (b == 1 or new_key.stride(0) == new_value.stride(0))):
            new_key, new_value = new_key.contiguous(), new_value.contiguous()
        new_stride = new_key.stride(0) if b > 1 else 0
    pos_dev, pos_host = None, 0
    if isinstance(pos, torch.Tensor):
        _device_tensor(pos, "pos", query)
        _require(pos.dtype == torch.int64 and pos.numel() == 1, "pos must be one int64")
        pos_dev = pos
    else:
        pos_host = int(pos)
    lib = _lib.load()
    nbytes = lib.oslo_attention_decode_workspace_bytes(b * h, cap, d, code)
    _require(nbytes > 0 or b * h == 0, f"attention_decode: heads of {d} x {query.dtype} are not supported")
    ws = torch.empty(nbytes // 4, dtype=torch.float32, device=query.device)
    out = torch.empty_like(q)
    with _on_device(q):
        _lib.check(lib.oslo_attention_decode_fwd(
            _ptr(out), _ptr(q), _ptr(k), _ptr(v), _ptr(new_key), _ptr(new_value), h,
            new_stride if new_key is not None else 0, _ptr(ws), _ptr(pos_dev), pos_host, int(window),
            float(scale), b * h, cap, d, code, _stream(q)))
    return out


PREFILL_HEAD_DIMS = (64, 128, 256)


def _prefill_args(query, key, value, pad):
    _device_tensor(query, "query")
    _device_tensor(key, "key", query)
    _device_tensor(value, "value", query)
    code = _dtype_code(query, "query")
    _require(query.dtype in (torch.float16, torch.bfloat16), "attention_prefill: fp16 or bf16 tensors")
    _require(query.dim() == 4 and key.shape == query.shape and value.shape == query.shape,
             "query, key and value must be [B, H, S, D] alike")
    _require(key.dtype == query.dtype and value.dtype == query.dtype, "query, key and value differ in dtype")
    b, h, s, d = query.shape
    _require(d in PREFILL_HEAD_DIMS, f"attention_prefill: heads of {d} features (64, 128 or 256 are taken)")
    if pad is not None:
        _device_tensor(pad, "pad", query)
        _require(pad.dtype == torch.float32 and tuple(pad.shape) == (b, s), "pad must be fp32 [B, S]")
        _require(s % 4 == 0, "attention_prefill: with a padding mask S must be a multiple of 4")
        pad = pad.contiguous()
    return code, pad


def _prefill_strided(t):
    """t as the prompt attention can read it: features contiguous, strides
    multiples of 8 elements, 32-bit byte offsets inside a head; a copy if not."""
    s, d = t.shape[2], t.shape[3]
    ok = t.stride(3) == 1 and all(st % 8 == 0 for st in t.stride()[:3]) and t.data_ptr() % 16 == 0 \
        and (s == 1 or t.stride(2) >= d) and (s + 128) * t.stride(2) * 2 < 2 ** 31
    return t if ok else t.contiguous()


def _stride_table(tensors):
    strides = (ctypes.c_int64 * (3 * len(tensors)))()
    for i, t in enumerate(tensors):
        strides[3 * i], strides[3 * i + 1], strides[3 * i + 2] = t.stride(0), t.stride(1), t.stride(2)
    return strides


def attention_prefill_forward(query, key, value, scale, pad=None, window=0, want_lse=False, p=0.0, seed=0,
                              offset=0):
    """Causal attention of a whole prompt in one kernel: query, key, value
    [B, H, S, D] fp16/bf16 views (features contiguous, any batch/head/position
    strides that are multiples of 8 elements), ``pad`` an optional additive
    fp32 [B, S] key mask, ``window`` > 0 a sliding window (query i sees keys
    i - window < s <= i). Returns softmax(scale * q k^T + causal + pad) v,
    shaped [B, H, S, D] over [B, S, H, D] memory, so that merging the heads
    afterwards moves nothing (oslo/models/gptj/modeling_gptj.py:936-951 and
    the ``_merge_heads`` that follows it). The [S, S] scores never reach memory.
    With ``want_lse`` also the fp32 [B, H, S] log2-sum-exp of every row, which
    ``attention_prefill_backward`` takes; then ``p`` > 0 applies attention
    dropout inside the kernel (keep mask of Philox ``seed`` / ``offset`` as the
    softmax kernel with fused dropout draws it; S a multiple of 8)."""
    code, pad = _prefill_args(query, key, value, pad)
    b, h, s, d = query.shape
    _require(p == 0.0 or want_lse, "attention dropout belongs to the training forward (want_lse)")
    q, k, v = _prefill_strided(query), _prefill_strided(key), _prefill_strided(value)
    out = torch.empty((b, s, h, d), dtype=query.dtype, device=query.device).permute(0, 2, 1, 3)
    lse = torch.empty((b, h, s), dtype=torch.float32, device=query.device) if want_lse else None
    if out.numel() > 0:
        strides = _stride_table((q, k, v, out))
        with _on_device(q):
            if want_lse:
                _lib.check(_lib.load().oslo_attention_prefill_fwd_lse(
                    _ptr(out), _ptr(lse), _ptr(q), _ptr(k), _ptr(v), _ptr(pad), float(scale), float(p), int(seed),
                    int(offset), b, h, s, d, int(window), strides, code, _stream(q)))
            else:
                _lib.check(_lib.load().oslo_attention_prefill_fwd(
                    _ptr(out), _ptr(q), _ptr(k), _ptr(v), _ptr(pad), float(scale), b, h, s, d, int(window), strides,
                    code, _stream(q)))
    return (out, lse) if want_lse else out


# Bytes of tile store a call of the attention's backward may allocate: the
# store of a call is freed when it returns (the next layer's call reuses the
# block), so this bounds what the backward adds to a training step's peak.
PREFILL_BWD_STORE_LIMIT = 2 << 30


def attention_prefill_backward(grad_out, query, key, value, out, lse, scale, pad=None, window=0, p=0.0, seed=0,
                               offset=0, store=None):
    """Gradients of ``attention_prefill_forward`` with respect to query, key and
    value (each [B, H, S, D], dense), from the gradient of its output, its
    inputs, its output and the log-sum-exp it returned with ``want_lse`` (and
    its ``p``, ``seed``, ``offset`` if it dropped attention probabilities). The
    [S, S] probabilities and their keep mask are recomputed tile by tile.
    ``store``: True = the pass that computes dQ hands the probabilities and their
    gradients to the pass for dK and dV through a workspace (16-bit, the tiles
    on and below the diagonal, for as many heads at a time as
    ``PREFILL_BWD_STORE_LIMIT`` bytes hold; freed on return); False = every pass
    computes the scores it needs and nothing of that size is in memory. Both
    give the same bits. None = whichever is faster: the store for heads of 256
    features (its traffic does not depend on the head size, the matrix products
    it saves do: at 128 features the two are even at best, at 64 the store
    loses by a factor of two), if 8 heads fit the limit."""
    code, pad = _prefill_args(query, key, value, pad)
    _device_tensor(grad_out, "grad_out", query)
    _device_tensor(out, "out", query)
    _device_tensor(lse, "lse", query)
    _require(grad_out.shape == query.shape and out.shape == query.shape, "grad_out and out must be shaped like query")
    _require(grad_out.dtype == query.dtype and out.dtype == query.dtype, "grad_out and out must have query's dtype")
    b, h, s, d = query.shape
    _require(lse.dtype == torch.float32 and tuple(lse.shape) == (b, h, s) and lse.is_contiguous(),
             "lse must be the fp32 [B, H, S] tensor of the forward")
    q, k, v, o, g = (_prefill_strided(t) for t in (query, key, value, out, grad_out))
    dq, dk, dv = (torch.empty((b, h, s, d), dtype=query.dtype, device=query.device) for _ in range(3))
    if dq.numel() == 0:
        return dq, dk, dv
    lib = _lib.load()
    ws = torch.empty(max(lib.oslo_attention_prefill_bwd_workspace_bytes(b, h, s) // 4, 1), dtype=torch.float32,
                     device=query.device)
    strides = _stride_table((q, k, v, o, g, dq, dk, dv))
    least = lib.oslo_attention_prefill_bwd_store_bytes(1, 8, s)
    if store is None:
        store = d == 256 and least <= PREFILL_BWD_STORE_LIMIT
    with _on_device(q):
        if store:
            want = lib.oslo_attention_prefill_bwd_store_bytes(b, h, s)
            size = max(least, min(want, PREFILL_BWD_STORE_LIMIT // least * least))
            tiles = torch.empty(size, dtype=torch.uint8, device=query.device)
            _lib.check(lib.oslo_attention_prefill_bwd_stored(
                _ptr(dq), _ptr(dk), _ptr(dv), _ptr(g), _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(lse), _ptr(ws),
                _ptr(tiles), size, _ptr(pad), float(scale), float(p), int(seed), int(offset), b, h, s, d,
                int(window), strides, code, _stream(q)))
        else:
            _lib.check(lib.oslo_attention_prefill_bwd(
                _ptr(dq), _ptr(dk), _ptr(dv), _ptr(g), _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(lse), _ptr(ws),
                _ptr(pad), float(scale), float(p), int(seed), int(offset), b, h, s, d, int(window), strides, code,
                _stream(q)))
    return dq, dk, dv


def rotary_qkv_forward(query, key, value, sin, cos, rotary_dim, offset=0):
    """query, key, value: [B, S, H, D] (any may be None); sin, cos: fp32
    [positions, rotary_dim/2]. Returns the three tensors as [B, H, S, D], query
    and key with their first rotary_dim features rotated by the angle of
    position offset + s (oslo/models/gptj/modeling_gptj.py:49-80, :205-233)."""
    return _rotary_call((query, key, value), sin, cos, rotary_dim, offset, inverse=False)


def rotary_qkv_backward(grad_query, grad_key, grad_value, sin, cos, rotary_dim, offset=0):
    """Gradients [B, H, S, D] of rotary_qkv_forward's outputs -> gradients
    [B, S, H, D] of its inputs."""
    return _rotary_call((grad_query, grad_key, grad_value), sin, cos, rotary_dim, offset, inverse=True)


def split_heads_packed_forward(qkv, heads):
    """qkv: [B, S, 3*H*D], the packed projection of GPT-2's c_attn
    (oslo/models/gpt2/modeling_gpt2.py:300-306). Returns query, key and value as
    contiguous [B, H, S, D]: the split and the three split-heads permutes in one
    launch, reading the slices in place."""
    _device_tensor(qkv, "qkv")
    code = _dtype_code(qkv, "qkv")
    _require(qkv.dim() == 3 and qkv.shape[2] % (3 * heads) == 0, "expected [B, S, 3*heads*head_dim]")
    qkv = qkv.contiguous()
    b, s, e3 = qkv.shape
    e = e3 // 3
    d = e // heads
    outs = [torch.empty((b, heads, s, d), dtype=qkv.dtype, device=qkv.device) for _ in range(3)]
    step = e * qkv.element_size()
    ins = [ctypes.c_void_p(qkv.data_ptr() + i * step) for i in range(3)]
    with _on_device(qkv):
        _lib.check(_lib.load().oslo_rotary_qkv(
            _ptr(outs[0]), _ptr(outs[1]), _ptr(outs[2]), ins[0], ins[1], ins[2], None, None, 0,
            b, s, heads, d, e3, 0, 0, 0, code, _stream(qkv)))
    return tuple(outs)


def split_heads_packed_backward(grad_query, grad_key, grad_value):
    """Gradients [B, H, S, D] of split_heads_packed_forward's outputs -> the
    gradient [B, S, 3*H*D] of the packed projection."""
    grads = []
    for t in (grad_query, grad_key, grad_value):
        _device_tensor(t, "gradient", grad_query)
        _require(t.shape == grad_query.shape and t.dtype == grad_query.dtype and t.dim() == 4,
                 "gradients differ in shape or dtype")
        grads.append(t.contiguous())
    code = _dtype_code(grad_query, "gradient")
    b, h, s, d = grad_query.shape
    e = h * d
    out = torch.empty((b, s, 3 * e), dtype=grad_query.dtype, device=grad_query.device)
    step = e * out.element_size()
    outs = [ctypes.c_void_p(out.data_ptr() + i * step) for i in range(3)]
    with _on_device(out):
        _lib.check(_lib.load().oslo_rotary_qkv(
            outs[0], outs[1], outs[2], _ptr(grads[0]), _ptr(grads[1]), _ptr(grads[2]), None, None, 0,
            b, s, h, d, 3 * e, 0, 0, 1, code, _stream(out)))
    return out
