"""CPU restatement of the reference's arithmetic for the kernel-fusion path.

THIS IS TEST INFRASTRUCTURE. Only tests, the smoke check and the cpu_baseline
leg of the benchmark may import it; nothing the library ships routes through
it. It is written with numpy only, one explicit step per line, and is pinned in
tests/test_oracle.py against independent evidence: library routines
(torch.softmax, torch.nn.functional.gelu(approximate="tanh"), autograd and
gradcheck), pure-Python float64 loops on tiny inputs, closed-form special cases,
and the published known-answer vectors of Philox4x32-10.

What each function follows in the reference (paths relative to the reference
root):

* softmax_causal / softmax_masked(mode="add"): the unfused attention,
  oslo/models/gpt2/modeling_gpt2.py:194-218 (scale, causal where(), additive
  padding mask, softmax), which oslo/models/gptj/modeling_gptj.py:151-180 and
  oslo/models/gpt_neo/modeling_gpt_neo.py:195-214 repeat;
* softmax_masked(mode="replace"): the fused kernel,
  oslo/fused_kernels/includes/fused_softmax.h:171-222;
* softmax_bwd: oslo/fused_kernels/includes/fused_softmax.h:283-319 and
  oslo/fused_kernels/includes/fused_triang_softmax.h:305-347;
* bias_gelu_fwd / bias_gelu_bwd: oslo/fused_kernels_utils.py:295-308 and the
  sum_to_size autograd applies to FusedBiasGeLU.backward's second output (:380);
* bias_dropout_add_fwd / _bwd: oslo/fused_kernels_utils.py:259-292
  (F.dropout(x + bias, p, training) + residual) given an explicit keep mask;
* get_batch_per_block: oslo/fused_kernels/includes/fused_softmax.h:328-340;
* ngram_banned_tokens: oslo/fused_kernels/fused_ngram_repeat_block.cu:18-49;
* reference_is_available: oslo/fused_kernels_utils.py:461-479;
* philox4x32_10 / dropout_bits / dropout_keep_mask: no counterpart in the
  reference (it uses torch's generator through F.dropout); they restate the
  published Philox algorithm and this library's documented element -> counter
  mapping (pinned by the Random123 known answers and a fixture written from
  torch's own Philox engine, tests/golden/philox_vectors.json);
* rotary_tables / rotary_split_heads: oslo/models/gptj/modeling_gptj.py:49-80
  and :205-233 (pinned by complex multiplication in float64, the adjoint
  identity and the torch operators of the unfused attention);
* linear_rows: the projection of the fused feed-forward and attention modules
  with its bias and activation, oslo/models/gptj/modeling_gptj.py:1049-1065
  (x @ weight.t(), then bias_gelu_fwd or + bias), written as explicit
  multiply-and-sum (pinned by a pure-Python float64 loop, numpy's matmul and
  torch.nn.functional.linear + gelu(approximate="tanh"));
* attention_decode: the attention of one query over cached keys and values,
  oslo/models/gptj/modeling_gptj.py:151-191 with a query length of 1 (scores,
  scale, the keys past the query hidden, softmax, weighted sum of the values),
  in float64 (pinned by softmax_masked of this file composed with numpy
  matmuls, by torch.nn.functional.scaled_dot_product_attention, and by the
  closed form for equal scores: the mean of the visible values);
* attention_prefill: the same attention for a whole prompt,
  oslo/models/gptj/modeling_gptj.py:151-191 (scores, scale, causal where(),
  additive padding mask, softmax, weighted sum of the values), row by row in
  float64 (pinned by softmax_causal of this file composed with numpy matmuls,
  by torch.nn.functional.scaled_dot_product_attention, by the closed form for
  equal scores -- the running mean of the values -- and by attention_decode
  on the last row);
* attention_prefill_bwd: what autograd derives for those operators (pinned by
  torch.autograd through torch.nn.functional.scaled_dot_product_attention in
  float64, by central differences of attention_prefill, and by the identities
  sum_k dS = 0 per row and dV = dO for a single position);
* build_sample_idx / build_blending_indices:
  oslo/fused_kernels/bindings/pybind_datasets.cpp:35-160 (pinned by the closed
  form "sample k starts at token k*seq_length", the share bound of the
  blending, and, where oracle/_ref holds a build of it, the reference's own
  module);
* build_mapping / build_blocks_mapping and the two Mersenne Twisters they draw
  from: oslo/fused_kernels/bindings/pybind_datasets.cpp:163-574 (the
  generators pinned by the C++ standard's 10000th-output values; the cutting
  by a cumulative-sum formulation of "the shortest run of sentences that
  reaches the target" for fixed targets and by the invariants every row must
  satisfy for random ones; the whole, where oracle/_ref holds a build of it, by
  the reference's own module).

Parity unpinned: none of the functions above. The reference itself holds no
golden vectors for this path.
"""

import numpy as np

MASK_VALUE = -10000.0


def _acc(dtype):
    return np.dtype(dtype).type


# ---------------------------------------------------------------------------
# softmax
# ---------------------------------------------------------------------------

def _softmax_lastdim(e):
    """softmax over the last axis of e, entries may be -inf (excluded)."""
    m = np.max(e, axis=-1, keepdims=True)
    p = np.exp(e - m)
    return p / np.sum(p, axis=-1, keepdims=True, dtype=e.dtype)


def softmax_causal(x, scale, pad_add=None, dtype=np.float32, window=None):
    """x [B,H,S,S]; pad_add None or [B,S] additive. Row r attends keys 0..r, or,
    with a window, the keys max(0, r-window+1)..r of GPT-Neo's local attention
    (oslo/models/gpt_neo/modeling_gpt_neo.py:153-163)."""
    t = _acc(dtype)
    x = np.asarray(x, dtype=dtype)
    b, h, s, s2 = x.shape
    assert s == s2
    e = x * t(scale)                                      # scale first ...
    if pad_add is not None:
        e = e + np.asarray(pad_add, dtype=dtype)[:, None, None, :]  # ... then the mask
    keep = np.tril(np.ones((s, s), dtype=bool))
    if window is not None:
        keep &= ~np.tril(np.ones((s, s), dtype=bool), -int(window))
    e = np.where(keep, e, t(-np.inf))
    return _softmax_lastdim(e)


def softmax_masked(x, mask, scale, mode="add", dtype=np.float32):
    """x [B,H,Sq,Sk]; mask None or boolean broadcastable to [B,1,Sq,Sk],
    True = masked. mode "add": e = scale*x + (-10000); "replace": e = -10000."""
    t = _acc(dtype)
    x = np.asarray(x, dtype=dtype)
    e = x * t(scale)
    if mask is not None:
        mask = np.broadcast_to(np.asarray(mask, dtype=bool), (x.shape[0], 1) + x.shape[2:])
        if mode == "add":
            e = np.where(mask, e + t(MASK_VALUE), e)
        elif mode == "replace":
            e = np.where(mask, t(MASK_VALUE), e)
        else:
            raise ValueError(mode)
    return _softmax_lastdim(e)


def softmax_bwd(g, y, scale, causal=False, dtype=np.float32, window=None):
    """dx = scale * (g*y - y * sum_k(g*y)); with causal=True only k <= r (and,
    with a window, k > r - window) takes part and dx is 0 elsewhere.
    g, y: [..., Sq, Sk]."""
    t = _acc(dtype)
    g = np.asarray(g, dtype=dtype)
    y = np.asarray(y, dtype=dtype)
    if causal:
        s = y.shape[-1]
        keep = np.tril(np.ones((s, s), dtype=bool))
        if window is not None:
            keep &= ~np.tril(np.ones((s, s), dtype=bool), -int(window))
        g = np.where(keep, g, t(0))
        y = np.where(keep, y, t(0))
    gy = g * y
    total = np.sum(gy, axis=-1, keepdims=True, dtype=dtype)
    return t(scale) * (gy - y * total)


def get_batch_per_block(sq, sk, batches, heads):
    log2_elements = 0
    while (1 << log2_elements) < sk:
        log2_elements += 1
    n2 = 1 << log2_elements
    warp_size = n2 if n2 < 32 else 32
    rows_per_warp = 2 if n2 <= 128 else 1
    return rows_per_warp * (128 // warp_size)


def reference_is_available(is_half, bsz, np_, sq, sk, use_triang_mask):
    """The reference's gate, with `is_half` standing for dtype == torch.half."""
    if not is_half or sk > 2048 or sk <= 0:
        return False
    bpb = get_batch_per_block(sq, sk, bsz, np_)
    if use_triang_mask:
        return sq == sk and (sk <= 64 or sk % 4 == 0) and (bsz * np_) % bpb == 0
    return sq > 1 and sq % bpb == 0


def ngram_banned_tokens(tokens, n):
    """tokens: list of the generated ids of one hypothesis. Returns the set of
    ids that would complete an n-gram already present: for every i with
    tokens[i:i+n-1] == tokens[-(n-1):] (or every i, for n == 1), tokens[i+n-1].
    Follows oslo/fused_kernels/fused_ngram_repeat_block.cu:18-49 (threads
    0 .. step-n+1 compare their n-1 tokens with the last n-1)."""
    cur_len = len(tokens)
    banned = set()
    if cur_len + 1 < n:
        return banned
    last = tokens[cur_len - (n - 1):] if n > 1 else []
    for i in range(cur_len - n + 1):
        if tokens[i:i + n - 1] == last:
            banned.add(tokens[i + n - 1])
    return banned


# ---------------------------------------------------------------------------
# bias + GeLU
# ---------------------------------------------------------------------------

def bias_gelu_fwd(y, bias, dtype=np.float32):
    t = _acc(dtype)
    x = np.asarray(y, dtype=dtype) + np.asarray(bias, dtype=dtype)
    return x * t(0.5) * (t(1.0) + np.tanh(t(0.79788456) * x * (t(1) + t(0.044715) * x * x)))


def linear_rows(x, weight, bias=None, gelu=False, dtype=np.float64):
    """x [m, k], weight [n, k] -> act(x . weight^T + bias) [m, n]."""
    x = np.asarray(x, dtype=dtype)
    w = np.asarray(weight, dtype=dtype)
    out = (x[:, None, :] * w[None, :, :]).sum(axis=-1)
    b = np.zeros(w.shape[0], dtype=dtype) if bias is None else np.asarray(bias, dtype=dtype)
    return bias_gelu_fwd(out, b, dtype=dtype) if gelu else out + b


def attention_decode(q, k, v, last, scale, window=0, dtype=np.float64):
    """q [n, d]; k, v [n, capacity, d]; keys first..last visible -> [n, d]."""
    q, k, v = (np.asarray(t, dtype=dtype) for t in (q, k, v))
    first = max(0, last - window + 1) if window > 0 else 0
    out = np.zeros_like(q)
    for i in range(q.shape[0]):
        scores = np.array([scale * np.dot(q[i], k[i, s]) for s in range(first, last + 1)], dtype=dtype)
        e = np.exp(scores - scores.max())
        p = e / e.sum()
        for j, s in enumerate(range(first, last + 1)):
            out[i] += p[j] * v[i, s]
    return out


def attention_prefill(q, k, v, scale, pad=None, dtype=np.float64, keep=None, p=0.0):
    """q, k, v [n, S, d]; pad None or additive [S] / [n, S] key mask -> [n, S, d]:
    row i attends keys 0..i. keep (bool [n, S, S]) and p: attention dropout, the
    probabilities are multiplied by keep / (1 - p) before they meet the values
    (self.attn_dropout, oslo/models/gptj/modeling_gptj.py:947-948)."""
    q, k, v = (np.asarray(t, dtype=dtype) for t in (q, k, v))
    n, S, _ = q.shape
    if pad is not None:
        pad = np.broadcast_to(np.asarray(pad, dtype=dtype), (n, S))
    out = np.zeros_like(q)
    for b in range(n):
        for i in range(S):
            scores = scale * (k[b, :i + 1] @ q[b, i])
            if pad is not None:
                scores = scores + pad[b, :i + 1]
            e = np.exp(scores - scores.max())
            probs = e / e.sum()
            if keep is not None:
                probs = np.where(keep[b, i, :i + 1], probs / (1.0 - p), 0.0)
            out[b, i] = probs @ v[b, :i + 1]
    return out


def attention_prefill_bwd(q, k, v, dout, scale, pad=None, window=None, dtype=np.float64, keep=None, p=0.0):
    """Gradients of attention_prefill (with GPT-Neo's sliding window if given:
    row i attends keys i - window < s <= i) for the upstream gradient dout:
    q, k, v, dout [n, S, d] -> (dq, dk, dv). With P the probabilities,
    dV = P^T dO, dP = dO V^T, dS = P o (dP - rowsum(dP o P)), dQ = scale dS K,
    dK = scale dS^T Q: what autograd derives for the matmul, softmax, matmul
    of oslo/models/gptj/modeling_gptj.py:151-191. With attention dropout (keep
    bool [n, S, S], p) the values met m o P, m = keep / (1 - p): dV = (m o P)^T
    dO and dP = m o (dO V^T)."""
    q, k, v, dout = (np.asarray(t, dtype=dtype) for t in (q, k, v, dout))
    n, S, _ = q.shape
    if pad is not None:
        pad = np.broadcast_to(np.asarray(pad, dtype=dtype), (n, S))
    i = np.arange(S)
    visible = i[None, :] <= i[:, None]
    if window is not None and window > 0:
        visible &= i[None, :] > i[:, None] - int(window)
    dq, dk, dv = np.zeros_like(q), np.zeros_like(k), np.zeros_like(v)
    for b in range(n):
        scores = scale * (q[b] @ k[b].T)
        if pad is not None:
            scores = scores + pad[b][None, :]
        scores = np.where(visible, scores, -np.inf)
        e = np.exp(scores - scores.max(axis=1, keepdims=True))
        prob = e / e.sum(axis=1, keepdims=True)
        m = np.ones_like(prob) if keep is None else np.where(keep[b], 1.0 / (1.0 - p), 0.0)
        dv[b] = (m * prob).T @ dout[b]
        dp = m * (dout[b] @ v[b].T)
        ds = prob * (dp - (dp * prob).sum(axis=1, keepdims=True))
        dq[b] = scale * (ds @ k[b])
        dk[b] = scale * (ds.T @ q[b])
    return dq, dk, dv


def bias_gelu_bwd(g, y, bias, dtype=np.float32):
    """Returns (dy, dbias); dbias sums dy over every axis but the last."""
    t = _acc(dtype)
    g = np.asarray(g, dtype=dtype)
    x = np.asarray(y, dtype=dtype) + np.asarray(bias, dtype=dtype)
    tanh_out = np.tanh(t(0.79788456) * x * (t(1) + t(0.044715) * x * x))
    ff = t(0.5) * x * ((t(1) - tanh_out * tanh_out) * (t(0.79788456) + t(0.1070322243) * x * x)) \
        + t(0.5) * (t(1) + tanh_out)
    dy = ff * g
    dbias = dy.reshape(-1, dy.shape[-1]).sum(axis=0, dtype=np.float64).astype(dtype)
    return dy, dbias


# ---------------------------------------------------------------------------
# Philox4x32-10 and the dropout mask
# ---------------------------------------------------------------------------

_M0, _M1 = np.uint64(0xD2511F53), np.uint64(0xCD9E8D57)
_W0, _W1 = np.uint32(0x9E3779B9), np.uint32(0xBB67AE85)
_LO = np.uint64(0xFFFFFFFF)
_S32 = np.uint64(32)


def philox4x32_10(key, counter):
    """key: 2 uint32 scalars; counter: 4 arrays of uint32 (same shape).
    Returns 4 arrays of uint32: ten rounds of the Philox-4x32 bijection
    (Salmon, Moraes, Dror, Shaw, SC'11), key bumped by the Weyl constants
    between rounds."""
    k0, k1 = np.uint32(key[0]), np.uint32(key[1])
    c0, c1, c2, c3 = [np.asarray(c, dtype=np.uint32) for c in counter]
    with np.errstate(over="ignore"):
        for _ in range(10):
            p0 = _M0 * c0.astype(np.uint64)
            p1 = _M1 * c2.astype(np.uint64)
            hi0, lo0 = (p0 >> _S32).astype(np.uint32), (p0 & _LO).astype(np.uint32)
            hi1, lo1 = (p1 >> _S32).astype(np.uint32), (p1 & _LO).astype(np.uint32)
            c0, c1, c2, c3 = hi1 ^ c1 ^ k0, lo1, hi0 ^ c3 ^ k1, lo0
            k0 = np.uint32((int(k0) + int(_W0)) & 0xFFFFFFFF)
            k1 = np.uint32((int(k1) + int(_W1)) & 0xFFFFFFFF)
    return c0, c1, c2, c3


def dropout_threshold(p):
    """floor(p * 2^16), at most 0xFFFF: an element is dropped with probability
    threshold / 2^16."""
    t = float(np.float32(p)) * 65536.0
    return 0xFFFF if t >= 65535.0 else int(t)


def dropout_bits(seed, offset, n, start=0):
    """The 16 random bits of elements start..start+n-1 (start a multiple of 8):
    element i owns the low (i even) or high (i odd) half of word (i mod 8) // 2
    of Philox4x32-10 with key = seed and counter = (offset // 4 as 64 bits,
    i // 8 as 64 bits)."""
    assert start % 8 == 0
    groups = (n + 7) // 8
    g = np.arange(groups, dtype=np.uint64) + np.uint64(start // 8)
    block = np.uint64(offset // 4)
    c0 = np.full(groups, block & _LO, dtype=np.uint64).astype(np.uint32)
    c1 = np.full(groups, block >> _S32, dtype=np.uint64).astype(np.uint32)
    c2 = (g & _LO).astype(np.uint32)
    c3 = (g >> _S32).astype(np.uint32)
    key = (seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF)
    words = np.stack(philox4x32_10(key, (c0, c1, c2, c3)), axis=1)          # [groups, 4]
    halves = np.stack((words & np.uint32(0xFFFF), words >> np.uint32(16)), axis=2)  # [groups, 4, 2]
    return halves.reshape(-1)[:n]


def dropout_keep_mask(seed, offset, n, p, start=0):
    """keep[i], i in [start, start + n): the element's 16 bits >= floor(p * 2^16)."""
    return dropout_bits(seed, offset, n, start) >= np.uint32(dropout_threshold(p))


def bias_dropout_add_fwd(x, bias, residual, p, keep, dtype=np.float32, residual2=None):
    """F.dropout(x + bias, p) + residual (+ residual2, the third term of GPT-J's
    block sum, oslo/models/gptj/modeling_gptj.py:319-320) with the keep mask
    given. keep: bool array of x's shape (ignored when p == 0)."""
    t = _acc(dtype)
    out = np.asarray(x, dtype=dtype)
    if bias is not None:
        out = out + np.asarray(bias, dtype=dtype)
    if p > 0:
        scale = t(1.0 / (1.0 - float(np.float32(p))))
        out = np.where(keep, out * scale, t(0))
    if residual is not None:
        out = out + np.asarray(residual, dtype=dtype)
    if residual2 is not None:
        out = out + np.asarray(residual2, dtype=dtype)
    return out


def bias_dropout_add_bwd(g, p, keep, dtype=np.float32):
    """Returns (dx, dbias, dresidual)."""
    t = _acc(dtype)
    g = np.asarray(g, dtype=dtype)
    dx = g
    if p > 0:
        scale = t(1.0 / (1.0 - float(np.float32(p))))
        dx = np.where(keep, g * scale, t(0))
    dbias = dx.reshape(-1, dx.shape[-1]).sum(axis=0, dtype=np.float64).astype(dtype)
    return dx, dbias, g


# ---------------------------------------------------------------------------
# rotary position embedding (GPT-J)
# ---------------------------------------------------------------------------

def rotary_tables(rotary_dim, positions):
    """fixed_pos_embedding (oslo/models/gptj/modeling_gptj.py:49-60): fp32 sin
    and cos of position * 10000^(-2i/rotary_dim), each [positions, rotary_dim/2];
    exponent, power, reciprocal and product each rounded to fp32."""
    expo = (np.arange(0, rotary_dim, 2, dtype=np.float32) / np.float32(rotary_dim)).astype(np.float32)
    inv_freq = (np.float32(1.0) / np.power(np.float32(10000.0), expo, dtype=np.float32)).astype(np.float32)
    angle = (np.arange(positions, dtype=np.float32)[:, None] * inv_freq[None, :]).astype(np.float32)
    return np.sin(angle, dtype=np.float32), np.cos(angle, dtype=np.float32)


def rotary_split_heads(x, sin, cos, rotary_dim, offset=0, rotate=True, inverse=False):
    """apply_rotary_pos_emb + cat + permute (modeling_gptj.py:63-80, :205-233)
    for one projection. Forward: x [B,S,H,D] -> [B,H,S,D] with
    out[2i] = x[2i]*cos_i + (-x[2i+1])*sin_i, out[2i+1] = x[2i+1]*cos_i + x[2i]*sin_i
    on the first rotary_dim features, every product and sum rounded to fp32.
    inverse: the transposed map, x [B,H,S,D] -> [B,S,H,D] with sin negated."""
    x = np.asarray(x, dtype=np.float32)
    if inverse:
        x = x.transpose(0, 2, 1, 3)          # work in [B,S,H,D]
    out = x.copy()
    if rotate and rotary_dim > 0:
        s_len = x.shape[1]
        sn = sin[offset:offset + s_len][None, :, None, :].astype(np.float32)
        cs = cos[offset:offset + s_len][None, :, None, :].astype(np.float32)
        if inverse:
            sn = -sn
        x0 = x[..., 0:rotary_dim:2]
        x1 = x[..., 1:rotary_dim:2]
        out[..., 0:rotary_dim:2] = (x0 * cs).astype(np.float32) + ((-x1) * sn).astype(np.float32)
        out[..., 1:rotary_dim:2] = (x1 * cs).astype(np.float32) + (x0 * sn).astype(np.float32)
    if inverse:
        return np.ascontiguousarray(out)
    return np.ascontiguousarray(out.transpose(0, 2, 1, 3))


# ---------------------------------------------------------------------------
# dataset index builders
# ---------------------------------------------------------------------------

def build_sample_idx(sizes, doc_idx, seq_length, num_epochs, tokens_per_epoch):
    """oslo/fused_kernels/bindings/pybind_datasets.cpp:85-160 (and its Python
    twin, oslo/data/datasets/dataset_causal_lm.py:323-358), one step per line.
    Returns int32 [num_samples + 1, 2]."""
    num_samples = (num_epochs * tokens_per_epoch - 1) // seq_length
    out = np.zeros((num_samples + 1, 2), dtype=np.int32)
    at, offset = 0, 0
    for k in range(1, num_samples + 1):
        remaining = seq_length + 1
        while remaining != 0:
            left_in_doc = int(sizes[doc_idx[at]]) - offset
            remaining -= left_in_doc
            if remaining <= 0:
                offset += remaining + left_in_doc - 1
                remaining = 0
            else:
                at += 1
                offset = 0
        out[k] = (at, offset)
    return out


def build_blending_indices(weights, num_datasets, size):
    """oslo/fused_kernels/bindings/pybind_datasets.cpp:35-82. Returns
    (dataset_index int32 [size], dataset_sample_index int64 [size])."""
    dataset_index = np.zeros(size, dtype=np.int32)
    dataset_sample_index = np.zeros(size, dtype=np.int64)
    drawn = [0] * num_datasets
    for i in range(size):
        at = max(float(i), 1.0)
        best, best_error = 0, float(weights[0]) * at - drawn[0]
        for d in range(1, num_datasets):
            error = float(weights[d]) * at - drawn[d]
            if error > best_error:
                best, best_error = d, error
        dataset_index[i] = best
        dataset_sample_index[i] = drawn[best]
        drawn[best] += 1
    return dataset_index, dataset_sample_index


class MersenneTwister:
    """std::mt19937 (w=32) and std::mt19937_64 (w=64) as the C++ standard
    defines them ([rand.predef]: the 10000th output of a default-constructed
    engine, seed 5489, is 4123659995 and 9981545732273789042 respectively);
    the reference draws sample lengths from the first and shuffles with the
    second (oslo/fused_kernels/bindings/pybind_datasets.cpp:218, :346)."""

    PARAMS = {
        32: dict(n=624, m=397, r=31, a=0x9908B0DF, u=11, d=0xFFFFFFFF, s=7, b=0x9D2C5680, t=15, c=0xEFC60000, l=18,
                 f=1812433253),
        64: dict(n=312, m=156, r=31, a=0xB5026F5AA96619E9, u=29, d=0x5555555555555555, s=17, b=0x71D67FFFEDA60000,
                 t=37, c=0xFFF7EEE000000000, l=43, f=6364136223846793005),
    }

    def __init__(self, seed, w=32):
        self.w, self.p = w, self.PARAMS[w]
        self.full = (1 << w) - 1
        state = [seed & self.full]
        for i in range(1, self.p["n"]):
            prev = state[-1]
            state.append((self.p["f"] * (prev ^ (prev >> (w - 2))) + i) & self.full)
        self.state, self.at = state, self.p["n"]

    def _twist(self):
        p, x = self.p, self.state
        upper = (self.full >> p["r"]) << p["r"]
        lower = self.full ^ upper
        for i in range(p["n"]):
            y = (x[i] & upper) | (x[(i + 1) % p["n"]] & lower)
            x[i] = x[(i + p["m"]) % p["n"]] ^ (y >> 1) ^ (p["a"] if y & 1 else 0)
        self.at = 0

    def __call__(self):
        p = self.p
        if self.at == p["n"]:
            self._twist()
        y = self.state[self.at]
        self.at += 1
        y ^= (y >> p["u"]) & p["d"]
        y ^= (y << p["s"]) & p["b"]
        y ^= (y << p["t"]) & p["c"]
        y ^= y >> p["l"]
        return y & self.full


LONG_SENTENCE_LEN = 512  # oslo/fused_kernels/bindings/pybind_datasets.cpp:32


def _shuffle_rows(rows, seed):
    """oslo/fused_kernels/bindings/pybind_datasets.cpp:346-355 (and :543-553)."""
    gen = MersenneTwister(seed + 1, 64)
    for i in range(len(rows) - 1, 0, -1):
        j = gen() % (i + 1)
        rows[i], rows[j] = rows[j], rows[i]
    return rows


def build_mapping(docs, sizes, num_epochs, max_num_samples, max_seq_length, short_seq_prob, seed, min_num_sent):
    """oslo/fused_kernels/bindings/pybind_datasets.cpp:163-372, the second of
    its two passes (the first only counts). Returns uint32 [num_samples, 3]
    (uint64 beyond 2^32 sentences, :384-412)."""
    # C's round(): halves away from zero (:205-208)
    ratio = int(np.floor(1.0 / short_seq_prob + 0.5)) if short_seq_prob > 0 else 0
    gen = MersenneTwister(seed, 32)

    def target_len():                                       # :163-176
        if ratio == 0:
            return max_seq_length
        draw = gen()
        if draw % ratio == 0:
            return 2 + draw % (max_seq_length - 1)
        return max_seq_length

    rows = []
    for _ in range(num_epochs):
        if len(rows) >= max_num_samples:
            break
        for doc in range(len(docs) - 1):
            first, last = int(docs[doc]), int(docs[doc + 1])
            start, remain = first, last - first
            long_sentence = remain > 1 and any(int(sizes[s]) > LONG_SENTENCE_LEN for s in range(first, last))
            if remain >= min_num_sent and not long_sentence:
                seq_len, num_sent, target = 0, 0, target_len()
                for s in range(first, last):
                    seq_len += int(sizes[s])
                    num_sent += 1
                    remain -= 1
                    if (seq_len >= target and remain > 1 and num_sent >= min_num_sent) or remain == 0:
                        rows.append((start, s + 1, target))
                        start = s + 1
                        target = target_len()
                        seq_len, num_sent = 0, 0
    dtype = np.uint64 if len(sizes) > np.iinfo(np.uint32).max else np.uint32
    return np.array(_shuffle_rows(rows, seed), dtype=dtype).reshape(-1, 3)


def build_blocks_mapping(docs, sizes, titles_sizes, num_epochs, max_num_samples, max_seq_length, seed,
                         use_one_sent_blocks):
    """oslo/fused_kernels/bindings/pybind_datasets.cpp:374-574. Returns uint32
    [num_blocks, 4]: first sentence, one past the last, document, block id."""
    min_num_sent = 1 if use_one_sent_blocks else 2
    rows = []
    for _ in range(num_epochs):
        block_id = 0
        if len(rows) >= max_num_samples:
            break
        for doc in range(len(docs) - 1):
            first, last = int(docs[doc]), int(docs[doc + 1])
            target = max_seq_length - int(titles_sizes[doc])
            start, remain = first, last - first
            long_sentence = remain >= min_num_sent and any(
                int(sizes[s]) > LONG_SENTENCE_LEN for s in range(first, last))
            if remain >= min_num_sent and not long_sentence:
                seq_len, num_sent = 0, 0
                for s in range(first, last):
                    seq_len += int(sizes[s])
                    num_sent += 1
                    remain -= 1
                    if (seq_len >= target and remain >= min_num_sent and num_sent >= min_num_sent) or remain == 0:
                        rows.append((start, s + 1, doc, block_id))
                        block_id += 1
                        start = s + 1
                        seq_len, num_sent = 0, 0
    dtype = np.uint64 if len(sizes) > np.iinfo(np.uint32).max else np.uint32
    return np.array(_shuffle_rows(rows, seed), dtype=dtype).reshape(-1, 4)
