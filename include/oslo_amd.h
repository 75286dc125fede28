/*
 * oslo_amd.h -- C ABI of the MI355X (gfx950) kernel-fusion library.
 *
 * One shared library, liboslo_amd.so, replaces the native module `oslo_kernels`
 * of tunib-ai/oslo (oslo/fused_kernels/bindings/pybind_kernels.cpp:159-177) and
 * the TorchScript-fused elementwise epilogues of
 * oslo/fused_kernels_utils.py:259-308.
 *
 * Conventions shared by every entry point:
 *   - plain device pointers and sizes; no torch or ATen type appears here;
 *   - tensors are dense row-major ("contiguous"), last dimension fastest;
 *   - `dtype` selects the storage type of every `void*` tensor argument of a
 *     call (enum oslo_dtype); arithmetic is always done in fp32;
 *   - work is enqueued on `stream` (a hipStream_t; NULL = the null stream) and
 *     the call returns without synchronising;
 *   - no entry point allocates or frees device memory;
 *   - the return value is OSLO_OK (0) or a negative oslo_status; nothing throws.
 *     oslo_last_error() gives the text of the calling thread's last failure.
 */
#ifndef OSLO_AMD_H_
#define OSLO_AMD_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *oslo_stream_t; /* a hipStream_t */

enum oslo_dtype { OSLO_F32 = 0, OSLO_F16 = 1, OSLO_BF16 = 2 };

enum oslo_status {
  OSLO_OK = 0,
  OSLO_E_BAD_ARG = -1,     /* null pointer, negative size, unknown enum value   */
  OSLO_E_UNSUPPORTED = -2, /* shape outside the supported range (see limits)   */
  OSLO_E_LAUNCH = -3       /* the HIP runtime refused the launch               */
};

/* How a set mask byte changes a score (oslo_softmax_masked_fwd). */
enum oslo_mask_mode {
  /* e = scale*x + (-10000): what the unfused attention computes
   * (oslo/models/gpt2/modeling_gpt2.py:214-216). */
  OSLO_MASK_ADD = 0,
  /* e = -10000: what the reference's fused kernel computes
   * (oslo/fused_kernels/includes/fused_softmax.h:171-175). The two differ only
   * on rows whose every key is masked. */
  OSLO_MASK_REPLACE = 1
};

/* Library identity and limits ------------------------------------------- */

/* ABI version of this header; bumped on any incompatible change. */
int oslo_abi_version(void);
/* Longest softmax row (key length) any softmax entry point accepts. The
 * reference stops at 2048 (oslo/fused_kernels/fused_softmax.cu:48,
 * oslo/fused_kernels/fused_triang_softmax.cu:39). */
int oslo_softmax_max_cols(void);
/* Text for a status code; never NULL. */
const char *oslo_status_string(int status);
/* Text of the calling thread's most recent failure ("" if none). */
const char *oslo_last_error(void);

/* Scale + causal mask + softmax ------------------------------------------ */

/*
 * Size limits of every softmax entry point (causal, windowed, key-mask, with
 * or without dropout): a row of at most oslo_softmax_max_cols() keys, and at
 * most 2^31 - 1 rows per call (batch * heads * S, or B * H * Sq); beyond either
 * the call returns OSLO_E_UNSUPPORTED and launches nothing. Elements are
 * indexed with 64 bits: tensors of 2^31 elements and more are single calls
 * (the reference launches any number of attention batches,
 * oslo/fused_kernels/fused_triang_softmax.cu:44-60).
 */

/*
 * y[b,h,r,k] = softmax over k<=r of ( scale*x[b,h,r,k] + pad_add[b,k] ),
 * y[b,h,r,k] = 0 for k>r. x, y: [batch, heads, S, S]; y may alias x.
 * pad_add: NULL or fp32 [batch, S], added after scaling (the order of the
 * unfused path, oslo/models/gpt2/modeling_gpt2.py:197-216).
 * Replaces scaled_upper_triang_masked_softmax::fwd
 * (oslo/fused_kernels/bindings/pybind_kernels.cpp:98-105,
 *  oslo/fused_kernels/fused_triang_softmax.cu:32-62,
 *  kernel oslo/fused_kernels/includes/fused_triang_softmax.h:134-251), which
 * has no pad argument: its caller adds the mask into a copy of x first
 * (oslo/fused_kernels_utils.py:444-449).
 */
int oslo_softmax_causal_fwd(void *y, const void *x, const float *pad_add,
                            float scale, int64_t batch, int64_t heads,
                            int64_t S, int dtype, oslo_stream_t stream);

/*
 * dx[n,r,k] = scale * y[n,r,k] * ( g[n,r,k] - sum_{j<=r} g[n,r,j]*y[n,r,j] )
 * for k<=r, 0 for k>r. g, y, dx: [bh, S, S]; dx may alias g (the reference
 * always writes over g). Entries of g and y above the diagonal are not read.
 * Replaces scaled_upper_triang_masked_softmax::bwd
 * (oslo/fused_kernels/bindings/pybind_kernels.cpp:107-123,
 *  oslo/fused_kernels/fused_triang_softmax.cu:64-96,
 *  kernel oslo/fused_kernels/includes/fused_triang_softmax.h:253-351).
 */
int oslo_softmax_causal_bwd(void *dx, const void *g, const void *y, float scale,
                            int64_t bh, int64_t S, int dtype,
                            oslo_stream_t stream);

/*
 * Causal softmax with attention-probability dropout in the same pass:
 * yd[b,h,r,k] = keep * y[b,h,r,k] / (1-p) with y as oslo_softmax_causal_fwd
 * (what is multiplied with V). keep for the flat element index i of the
 * [batch, heads, S, S] tensor is drawn like in oslo_bias_dropout_add_fwd
 * (Philox4x32-10, counter (offset/4, i/8), 16 bits per element); one call
 * consumes 4 units of generator offset.
 * p in [0,1). y itself is not stored. Instead row_stats (fp32,
 * [batch*heads*S, 2], 8-byte aligned) receives per row the maximum of the
 * exponent e and 1/sum_k exp(e_k - max), where e = scale*x*log2(e) in base-2
 * units when pad_add is NULL and e = scale*x + pad_add in natural units
 * otherwise; the backward recomputes y from x and these two numbers, so the
 * caller keeps x (not y) for the backward. yd may alias x only if x is not
 * needed afterwards.
 * Replaces the softmax kernel followed by the separate nn.Dropout of the
 * reference's fused GPT-Neo / GPT-J attention
 * (oslo/models/gptj/modeling_gptj.py:941-948,
 *  oslo/models/gpt_neo/modeling_gpt_neo.py:997-1005).
 */
int oslo_softmax_causal_dropout_fwd(void *yd, float *row_stats, const void *x,
                                    const float *pad_add, float scale, float p,
                                    uint64_t philox_seed, uint64_t philox_offset,
                                    int64_t batch, int64_t heads, int64_t S,
                                    int dtype, oslo_stream_t stream);

/*
 * Backward of the above: g is the gradient of yd; x, row_stats, pad_add,
 * scale, p, seed and offset are the forward's. With g' = keep * g / (1-p)
 * (mask regenerated) and y recomputed from x and row_stats,
 * dx = scale * y * ( g' - sum_{j<=r} g'_j * y_j ) for k<=r, 0 for k>r.
 * dx may alias g or x.
 */
int oslo_softmax_causal_dropout_bwd(void *dx, const void *g, const void *x,
                                    const float *row_stats, const float *pad_add,
                                    float scale, float p, uint64_t philox_seed,
                                    uint64_t philox_offset, int64_t batch,
                                    int64_t heads, int64_t S, int dtype,
                                    oslo_stream_t stream);

/*
 * Sliding-window causal softmax: as oslo_softmax_causal_fwd, but row r sees only
 * the keys max(0, r-window+1) .. r (window >= 1; window >= S is the plain causal
 * softmax). y is zero outside the window.
 * This is the mask of GPT-Neo's local attention layers, bias = tril(ones) xor
 * tril(ones, -window) (oslo/models/gpt_neo/modeling_gpt_neo.py:153-163), which
 * the reference computes on its unfused path only (:268-272).
 */
int oslo_softmax_causal_window_fwd(void *y, const void *x, const float *pad_add,
                                   float scale, int64_t window, int64_t batch,
                                   int64_t heads, int64_t S, int dtype,
                                   oslo_stream_t stream);

/*
 * Backward of the above: dx = scale * y * (g - sum_j g_j*y_j) over the keys of
 * the window, 0 outside it. dx may alias g.
 */
int oslo_softmax_causal_window_bwd(void *dx, const void *g, const void *y,
                                   float scale, int64_t window, int64_t bh,
                                   int64_t S, int dtype, oslo_stream_t stream);

/* Scale + key/padding mask + softmax -------------------------------------- */

/*
 * y[b,h,q,k] = softmax over k of e, e per `mask_mode` where
 * mask[b*mask_stride_b + q*mask_stride_q + k] != 0, else scale*x[b,h,q,k].
 * x, y: [B, H, Sq, Sk]; y may alias x. mask: NULL (nothing masked) or bytes;
 * a stride of 0 broadcasts that dimension, so a [B,1,1,Sk] key mask is passed
 * as (mask_stride_b=Sk, mask_stride_q=0) and the reference's materialised
 * [B|1,1,Sq,Sk] mask as (Sq*Sk|0, Sk).
 * Replaces scaled_masked_softmax::fwd
 * (oslo/fused_kernels/bindings/pybind_kernels.cpp:46-57,
 *  oslo/fused_kernels/fused_softmax.cu:37-80,
 *  kernel oslo/fused_kernels/includes/fused_softmax.h:111-229).
 */
int oslo_softmax_masked_fwd(void *y, const void *x, const uint8_t *mask,
                            int64_t mask_stride_b, int64_t mask_stride_q,
                            int mask_mode, float scale, int64_t B, int64_t H,
                            int64_t Sq, int64_t Sk, int dtype,
                            oslo_stream_t stream);

/*
 * dx[n,k] = scale * y[n,k] * ( g[n,k] - sum_j g[n,j]*y[n,j] ).
 * g, y, dx: [rows, Sk]; dx may alias g.
 * Replaces scaled_masked_softmax::bwd
 * (oslo/fused_kernels/bindings/pybind_kernels.cpp:59-75,
 *  oslo/fused_kernels/fused_softmax.cu:82-115,
 *  kernel oslo/fused_kernels/includes/fused_softmax.h:231-325).
 */
int oslo_softmax_masked_bwd(void *dx, const void *g, const void *y, float scale,
                            int64_t rows, int64_t Sk, int dtype,
                            oslo_stream_t stream);

/*
 * Rows of attention scores one 128-thread block of the reference's kernels
 * handles: an implementation detail the reference exports so that its
 * availability gate can test divisibility
 * (oslo/fused_kernels/includes/fused_softmax.h:328-340,
 *  oslo/fused_kernels/bindings/pybind_kernels.cpp:77-83,
 *  used at oslo/fused_kernels_utils.py:465). Pure integer arithmetic with the
 * reference's 32-lane constants, so callers see the reference's numbers. The
 * kernels of this library have no divisibility requirement.
 */
int oslo_get_batch_per_block(int sq, int sk, int batches, int heads);

/* Bias + GeLU (tanh form) -------------------------------------------------- */

/*
 * out[r,c] = gelu_tanh( y[r,c] + bias[c] ),
 * gelu_tanh(x) = 0.5*x*(1 + tanh(0.79788456*x*(1 + 0.044715*x*x))).
 * y, out: [rows, cols]; bias: [cols]; out may alias y.
 * Replaces bias_gelu_fwb (oslo/fused_kernels_utils.py:295-298).
 */
int oslo_bias_gelu_fwd(void *out, const void *y, const void *bias, int64_t rows,
                       int64_t cols, int dtype, oslo_stream_t stream);

/*
 * Bytes of fp32 workspace the two backward entry points below need to produce
 * dbias for a [rows, cols] problem (0 if rows or cols is 0).
 */
size_t oslo_colsum_workspace_bytes(int64_t rows, int64_t cols);

/*
 * dy[r,c] = g[r,c] * gelu_tanh'( y[r,c] + bias[c] ) and, if dbias != NULL,
 * dbias[c] = sum_r dy[r,c] (fp32 sum of the unrounded products, stored in
 * `dtype`). workspace: oslo_colsum_workspace_bytes(rows, cols) bytes of device
 * memory, required only when dbias != NULL. dy may alias g.
 * Replaces bias_gelu_bwd (oslo/fused_kernels_utils.py:301-308) and the
 * separate reduction autograd runs on the full-shape bias gradient that
 * FusedBiasGeLU.backward returns (oslo/fused_kernels_utils.py:376-380).
 */
int oslo_bias_gelu_bwd(void *dy, void *dbias, float *workspace, const void *g,
                       const void *y, const void *bias, int64_t rows,
                       int64_t cols, int dtype, oslo_stream_t stream);

/*
 * oslo_bias_gelu_bwd without the workspace argument: the fp32 partial rows of
 * dbias go to a buffer of OSLO_STATIC_WORKSPACE_BYTES that is part of the
 * library's device image (one copy per GPU, held until the process ends), so
 * the caller needs no device allocation of its own for the call. Results are
 * bit-identical to oslo_bias_gelu_bwd's. It has no counterpart in the
 * reference; it is for callers that cannot allocate: code under HIP graph
 * capture, serving loops and harnesses that forbid hipMalloc.
 * Fails with OSLO_E_UNSUPPORTED when dbias != NULL and
 * oslo_colsum_workspace_bytes(rows, cols) exceeds the buffer ([16384, 16384]
 * is the largest square problem that fits). The first call on a device looks
 * the buffer's address up (that loads the library's device image if nothing
 * has yet): make one call, of any size, before a graph capture begins. All
 * calls on a GPU share the one buffer: calls that may overlap there (different
 * streams, different threads) race; order them or use oslo_bias_gelu_bwd.
 * The buffer used is the one of the calling thread's current device, which
 * must be the device that holds the tensors (and owns the stream): a call whose
 * tensors are on another device fails with OSLO_E_BAD_ARG.
 */
#define OSLO_STATIC_WORKSPACE_BYTES (32u << 20)
int oslo_bias_gelu_bwd_static(void *dy, void *dbias, const void *g,
                              const void *y, const void *bias, int64_t rows,
                              int64_t cols, int dtype, oslo_stream_t stream);

/* Bias + dropout (+ residual) ----------------------------------------------- */

/*
 * out[r,c] = keep[r,c] * (x[r,c] + bias[c]) / (1-p) + residual[r,c].
 * bias and residual may each be NULL (term dropped). p in [0,1); p == 0 keeps
 * everything and draws no random numbers. keep[i] for the flat element index
 * i = r*cols + c comes from Philox4x32-10 with key = philox_seed and
 * counter = (philox_offset/4 as 64 bits, i/8 as 64 bits): element i owns 16 of
 * the 128 bits, the low half of word (i mod 8)/2 when i is even, the high half
 * when odd, and keep = bits >= floor(p * 2^16) (p is quantised to a multiple
 * of 2^-16). One call consumes 4 units of generator offset. out may alias x.
 * Replaces bias_dropout / bias_dropout_residual
 * (oslo/fused_kernels_utils.py:259-292).
 */
int oslo_bias_dropout_add_fwd(void *out, const void *x, const void *bias,
                              const void *residual, float p,
                              uint64_t philox_seed, uint64_t philox_offset,
                              int64_t rows, int64_t cols, int dtype,
                              oslo_stream_t stream);

/*
 * The same with a second residual:
 * out = keep * (x + bias) / (1-p) + residual + residual2, the sum formed in
 * fp32 in that order and rounded once. residual2 may be NULL (then exactly
 * oslo_bias_dropout_add_fwd); with residual2 given, residual must be too.
 * For GPT-J's block, whose output is attention output + feed-forward output +
 * residual stream (oslo/models/gptj/modeling_gptj.py:319-320; the reference
 * adds the three with two torch additions, each rounding to the storage
 * type). The backward is oslo_bias_dropout_add_bwd: both residuals receive g.
 */
int oslo_bias_dropout_add2_fwd(void *out, const void *x, const void *bias,
                               const void *residual, const void *residual2,
                               float p, uint64_t philox_seed,
                               uint64_t philox_offset, int64_t rows,
                               int64_t cols, int dtype, oslo_stream_t stream);

/*
 * dx[r,c] = keep[r,c] * g[r,c] / (1-p) with the mask regenerated from the same
 * (seed, offset); if dbias != NULL, dbias[c] = sum_r dx[r,c] (workspace as for
 * oslo_bias_gelu_bwd). The gradient of the residual is g itself. dx may alias
 * g. The reference leaves this to TorchScript autodiff of
 * oslo/fused_kernels_utils.py:259-292.
 */
int oslo_bias_dropout_add_bwd(void *dx, void *dbias, float *workspace,
                              const void *g, float p, uint64_t philox_seed,
                              uint64_t philox_offset, int64_t rows,
                              int64_t cols, int dtype, oslo_stream_t stream);

/* Rotary position embedding + split-heads transposition ----------------------- */

/*
 * q_in, k_in, v_in: [batch, seq, heads, head_dim] (the projections viewed by
 * head); q_out, k_out, v_out: [batch, heads, seq, head_dim]. For q and k the
 * first rotary_dim features are rotated pairwise by the angle of position
 * offset + s, in fp32 and in the reference's order of operations:
 *   out[2i]   = x[2i]  *cos[pos,i] + (-x[2i+1])*sin[pos,i]
 *   out[2i+1] = x[2i+1]*cos[pos,i] +   x[2i]   *sin[pos,i]
 * the remaining features and all of v are only moved. sin_table, cos_table:
 * fp32 [table_positions, rotary_dim/2]. Any of the three tensor pairs may be
 * NULL (both pointers). inverse != 0 runs the transposed map, the backward:
 * *_in are then [batch, heads, seq, head_dim] gradients, *_out
 * [batch, seq, heads, head_dim], rotation by the opposite angle. head_dim must
 * be a multiple of 16 bytes, rotary_dim even; no output may alias an input.
 * row_stride is the distance, in elements, between consecutive positions of
 * the [batch, seq, heads, head_dim] side (its batch stride is seq*row_stride):
 * 0 or heads*head_dim for a dense tensor, 3*heads*head_dim when q, k and v are
 * the three slices of one packed [batch, seq, 3*hidden] projection, as in
 * GPT-2's c_attn (oslo/models/gpt2/modeling_gpt2.py:176-183, :300-306). The
 * [batch, heads, seq, head_dim] side is always dense.
 * Replaces fixed_pos_embedding / rotate_every_two / apply_rotary_pos_emb, the
 * torch.cat of rotated and passed-through features and the permute of
 * GPTJAttention.forward (oslo/models/gptj/modeling_gptj.py:49-80, :205-233).
 */
int oslo_rotary_qkv(void *q_out, void *k_out, void *v_out, const void *q_in,
                    const void *k_in, const void *v_in, const float *sin_table,
                    const float *cos_table, int64_t table_positions,
                    int64_t batch, int64_t seq, int64_t heads, int64_t head_dim,
                    int64_t row_stride, int64_t rotary_dim, int64_t offset,
                    int inverse, int dtype, oslo_stream_t stream);

/* Linear layer of a decoding step -------------------------------------------- */

enum oslo_epilogue {
  OSLO_EPILOGUE_NONE = 0,     /* out = x.w + bias                                 */
  OSLO_EPILOGUE_GELU_TANH = 1 /* out = gelu_tanh(x.w + bias), oslo_bias_gelu_fwd's */
};

/* Most input rows oslo_linear_rows_fwd accepts. */
int oslo_linear_rows_max(void);

/*
 * out[i, j] = epilogue( sum_c x[i, c] * weight[j, c] + bias[j] ) + residual[i, j] for a few
 * input rows: x [m, k], weight [n, k] (the layout of torch.nn.Linear.weight),
 * bias NULL or [n], out [m, n]; 0 <= m <= oslo_linear_rows_max(). residual:
 * NULL or [m, n], added after the epilogue (the residual connection around the
 * attention or the feed-forward module, oslo/models/gpt2/modeling_gpt2.py:444,
 * :474); out may alias it. Sums and the epilogue are fp32, rounded once to the
 * storage type. The kernel streams the
 * weight once (it is bound by HBM, like a GEMV); for more rows a GEMM library
 * is the right tool and the call returns OSLO_E_UNSUPPORTED. k*sizeof(dtype)
 * must be a multiple of 16, x and weight 16-byte aligned, the weight smaller
 * than 2 GiB; out must not alias x or weight.
 * Replaces, for the one-token-per-sequence steps of generation, the pair
 *   x = torch.matmul(x, self.fc_in.weight.t())
 *   x = FusedBiasActivation.apply(x, self.fc_in.bias, act)
 * of the fused feed-forward module (oslo/models/gptj/modeling_gptj.py:1049-1054,
 * oslo/models/gpt_neo/modeling_gpt_neo.py:1086-1091) with epilogue GELU_TANH,
 * its second projection and bias (modeling_gptj.py:1057-1065) and the bias-free
 * projections of the attention (q_proj, k_proj, v_proj, out_proj,
 * modeling_gptj.py:968-970, :1031) with epilogue NONE.
 */
int oslo_linear_rows_fwd(void *out, const void *x, const void *weight,
                         const void *bias, const void *residual, int64_t m,
                         int64_t n, int64_t k, int epilogue, int dtype,
                         oslo_stream_t stream);

/*
 * The same for `count` (1 to 3) layers of one shape applied to the same x in
 * one launch: out[j] = epilogue(x . weight[j]^T + bias[j]). out, weight and
 * bias are host arrays of `count` device pointers; bias may be NULL (no layer
 * has a bias) or hold NULL entries (that layer has none). The query, key and
 * value projections of a decoding step
 * (oslo/models/gptj/modeling_gptj.py:968-970) are such a triple.
 */
int oslo_linear_rows_fwd_multi(void *const *out, const void *x,
                               const void *const *weight,
                               const void *const *bias, int count, int64_t m,
                               int64_t n, int64_t k, int epilogue, int dtype,
                               oslo_stream_t stream);

/*
 * The same layer with the weight stored [k, n] (input features major), the
 * layout of GPT-2's Conv1D (transformers' pytorch_utils.Conv1D, y = x @ w + b):
 * out[i, j] = epilogue( sum_c x[i, c] * weight[c, j] + bias[j] ) + residual[i, j].
 * Both k and n
 * times sizeof(dtype) must be multiples of 16. Replaces, for a decoding step,
 * self.c_attn(hidden_states), `attn_output @= self.c_proj.weight` + bias and the
 * two projections of the fused feed-forward module with FusedBiasActivation
 * (oslo/models/gpt2/modeling_gpt2.py:1485, :1523-1536, :1553-1567).
 */
int oslo_linear_rows_kn_fwd(void *out, const void *x, const void *weight,
                            const void *bias, const void *residual, int64_t m,
                            int64_t n, int64_t k, int epilogue, int dtype,
                            oslo_stream_t stream);

/* Attention of a decoding step ----------------------------------------------- */

/*
 * One query per (sequence, head) over a key/value cache:
 *   out[i, :] = sum_s softmax_s( scale * q[i, :] . k[i, s, :] ) * v[i, s, :]
 * over the visible keys s: first <= s <= last, where last is *pos_dev (if
 * pos_dev is not NULL: an int64 in device memory, read by the kernel, so that a
 * captured launch follows a position that advances) or else pos, and first is
 * last - window + 1 for window > 0 (a sliding window, as in GPT-Neo's local
 * layers), else 0. q, out: [rows_heads, head_dim]; k, v: [rows_heads, capacity,
 * head_dim] (a [batch, heads, capacity, head_dim] cache); 0 <= last < capacity.
 * Keys outside the visible range are not read. k_new, v_new: both NULL, or
 * the key and value of position `last` as [rows_heads / heads, heads, head_dim]
 * with new_seq_stride elements between sequences (0: dense; 3*heads*head_dim
 * for the slices of GPT-2's packed c_attn output), which are then used from
 * there and written into slot `last` of k and v by the kernel (the append to
 * the cache and the attention in one launch); the other slots of k and v are
 * only read. heads is used only with k_new. workspace: fp32, at least
 * oslo_attention_decode_workspace_bytes(...) bytes, contents irrelevant before
 * and after. head_dim * sizeof(dtype) must be 128, 256, 512 or 1024 bytes.
 * Arithmetic in fp32 throughout (scores, softmax, weighted sum), one rounding
 * at the end.
 * Replaces, for a query length of 1, the sequence matmul(q, k^T) ->
 * FusedScaleMaskSoftmax.apply -> matmul(probs, v) of the fused attention
 * (oslo/models/gptj/modeling_gptj.py:936-951,
 *  oslo/models/gpt_neo/modeling_gpt_neo.py:993-1008,
 *  oslo/models/gpt2/modeling_gpt2.py:1435-1459).
 */
size_t oslo_attention_decode_workspace_bytes(int64_t rows_heads,
                                             int64_t capacity, int64_t head_dim,
                                             int dtype);
int oslo_attention_decode_fwd(void *out, const void *q, void *k, void *v,
                              const void *k_new, const void *v_new,
                              int64_t heads, int64_t new_seq_stride,
                              float *workspace,
                              const int64_t *pos_dev, int64_t pos,
                              int64_t window, float scale, int64_t rows_heads,
                              int64_t capacity, int64_t head_dim, int dtype,
                              oslo_stream_t stream);

/*
 * Causal attention over a whole prompt without the [S, S] matrix in memory:
 *   out[b, h, i, :] = sum_{s <= i} softmax_s( scale * q[b,h,i,:] . k[b,h,s,:]
 *                                             + pad[b, s] ) * v[b,h,s,:]
 * q, k, v, out: 16-bit (OSLO_F16 or OSLO_BF16), S positions of head_dim (64,
 * 128 or 256) contiguous features per (batch, head); strides[12] gives, in
 * elements, the batch, head and position strides of q, k, v and out in that
 * order, so that split heads ([B, H, S, D]), merged heads ([B, S, H, D]) and
 * slices of a packed qkv projection are all taken where they lie (multiples
 * of 8 elements, pointers 16-byte aligned, a (batch, head) slice under 2 GiB).
 * window > 0 restricts the sum to the last `window` keys, i - window < s <= i
 * (GPT-Neo's local attention, oslo/models/gpt_neo/modeling_gpt_neo.py:153-163).
 * pad: NULL, or an additive fp32 [batch, S] key mask (then S % 4 == 0).
 * scale > 0. Products of the 16-bit inputs are accumulated in fp32, the softmax is fp32
 * under a running maximum, the probabilities are rounded to the storage type
 * before they multiply v (as the unfused path casts them), the sum over keys
 * is fp32 and is normalised and rounded once at the end. No workspace.
 * Replaces, for inference, matmul(q, k^T) -> FusedScaleMaskSoftmax.apply ->
 * matmul(probs, v) of the fused attention
 * (oslo/models/gptj/modeling_gptj.py:936-951,
 *  oslo/models/gpt_neo/modeling_gpt_neo.py:993-1008,
 *  oslo/models/gpt2/modeling_gpt2.py:1435-1459).
 */
int oslo_attention_prefill_fwd(void *out, const void *q, const void *k,
                               const void *v, const float *pad, float scale,
                               int64_t batch, int64_t heads, int64_t S,
                               int64_t head_dim, int64_t window,
                               const int64_t *strides, int dtype,
                               oslo_stream_t stream);

/*
 * oslo_attention_prefill_fwd for a training step. It also stores what the
 * backward needs: lse[b*heads + h, i] (fp32, [batch*heads, S], 16-byte
 * aligned) = log2 of sum_s 2^(log2(e) * (scale*q.k + pad)) over the visible
 * keys of query i. And it can apply attention dropout, p in [0, 1): the
 * probability of (query i, key s) of head (b, h) is multiplied by keep/(1-p)
 * before it meets v, with keep drawn exactly as
 * oslo_softmax_causal_dropout_fwd draws it for element (b, h, i, s) of a
 * [batch, heads, S, S] tensor (Philox4x32-10, counter (offset/4, flat
 * index/8), 16 bits per element; one call consumes 4 units of generator
 * offset); then S must be a multiple of 8. lse is that of the probabilities
 * before dropout. p == 0 draws nothing.
 * Replaces matmul(q, k^T) -> FusedScaleMaskSoftmax.apply -> attn_dropout ->
 * matmul(probs, v) with gradients recorded
 * (oslo/models/gptj/modeling_gptj.py:936-951).
 */
int oslo_attention_prefill_fwd_lse(void *out, float *lse, const void *q,
                                   const void *k, const void *v,
                                   const float *pad, float scale, float p,
                                   uint64_t philox_seed, uint64_t philox_offset,
                                   int64_t batch, int64_t heads, int64_t S,
                                   int64_t head_dim, int64_t window,
                                   const int64_t *strides, int dtype,
                                   oslo_stream_t stream);

/* Bytes of fp32 workspace oslo_attention_prefill_bwd needs. */
size_t oslo_attention_prefill_bwd_workspace_bytes(int64_t batch, int64_t heads,
                                                  int64_t S);

/*
 * Backward of the causal prompt attention: from the gradient dout of the
 * output, the inputs q, k, v, the forward's out and lse
 * (oslo_attention_prefill_fwd_lse) and its p, seed and offset, with
 * P[i,s] = 2^(log2(e)*(scale*q_i.k_s + pad[s]) - lse[i]) over the visible keys
 * and m[i,s] = keep[i,s]/(1-p) (the forward's mask, regenerated; 1 if p == 0),
 *   dv[s] = sum_i m[i,s] P[i,s] dout[i]
 *   dS[i,s] = scale * P[i,s] * (m[i,s] * dout[i].v[s] - sum_d dout[i,d]*out[i,d])
 *   dq[i] = sum_s dS[i,s] k[s],   dk[s] = sum_i dS[i,s] q[i].
 * strides[24]: batch, head and position strides, in elements, of q, k, v, out,
 * dout, dq, dk, dv in that order (the limits of oslo_attention_prefill_fwd).
 * P and dS are rounded to the storage type before the products that sum over
 * them, every sum is fp32, each gradient is rounded once. No [S, S] tensor is
 * read or written; nothing is accumulated with atomics, so the result is the
 * same from run to run. workspace: oslo_attention_prefill_bwd_workspace_bytes
 * bytes (16-byte aligned), contents irrelevant before and after. No output may
 * alias an input.
 * Replaces what autograd records for matmul(q, k^T) ->
 * FusedScaleMaskSoftmax.apply -> attn_dropout -> matmul(probs, v) of the fused
 * attention in a training step (oslo/models/gptj/modeling_gptj.py:936-951,
 *  oslo/models/gpt_neo/modeling_gpt_neo.py:993-1008,
 *  oslo/models/gpt2/modeling_gpt2.py:1435-1459): two matmul backwards around
 * the softmax kernel's backward, all on [B, H, S, S] tensors.
 */
int oslo_attention_prefill_bwd(void *dq, void *dk, void *dv, const void *dout,
                               const void *q, const void *k, const void *v,
                               const void *out, const float *lse,
                               float *workspace, const float *pad, float scale,
                               float p, uint64_t philox_seed,
                               uint64_t philox_offset, int64_t batch,
                               int64_t heads, int64_t S, int64_t head_dim,
                               int64_t window, const int64_t *strides,
                               int dtype, oslo_stream_t stream);

/*
 * The same gradients with the probabilities handed from pass to pass through
 * memory: the pass that computes dq also writes, for every tile of 32 queries
 * x 32 keys on or below the diagonal, P (after dropout) and dS / scale in the
 * storage type (4 KiB a tile) into `store`, and one more pass accumulates dk
 * and dv from them: 5 matrix products per tile, where the entry point above
 * computes the scores once per pass (7 or 8); worth its memory traffic at
 * head_dim 256, not at 64 or 128. The results obey the same
 * formulas and the same rounding (P and dS are rounded to the storage type
 * before the products either way), sums run in the same order, and they are
 * as reproducible.
 * store: store_bytes bytes, 16-byte aligned, contents irrelevant before and
 * after. oslo_attention_prefill_bwd_store_bytes(batch, heads, S) holds every
 * head at once; with less the heads are processed in groups of 8 x k, as many
 * as fit, and oslo_attention_prefill_bwd_store_bytes(1, 8, S) is the least
 * (less: OSLO_E_BAD_ARG). Everything else as above, workspace included.
 * Replaces the same reference code as oslo_attention_prefill_bwd; autograd
 * there keeps P and dS as whole [B, H, S, S] tensors between forward and
 * backward, here they exist for the heads of one launch during the call.
 */
size_t oslo_attention_prefill_bwd_store_bytes(int64_t batch, int64_t heads,
                                              int64_t S);
int oslo_attention_prefill_bwd_stored(void *dq, void *dk, void *dv,
                                      const void *dout, const void *q,
                                      const void *k, const void *v,
                                      const void *out, const float *lse,
                                      float *workspace, void *store,
                                      size_t store_bytes, const float *pad,
                                      float scale, float p,
                                      uint64_t philox_seed,
                                      uint64_t philox_offset, int64_t batch,
                                      int64_t heads, int64_t S,
                                      int64_t head_dim, int64_t window,
                                      const int64_t *strides, int dtype,
                                      oslo_stream_t stream);

/* Repeated n-gram blocking (beam search) ------------------------------------ */

/*
 * For every row and every i in [0, step-n+1]: if tokens[row, i .. i+n-2] equals
 * the last n-1 tokens tokens[row, step-n+2 .. step], then
 * lprobs[row, tokens[row, i+n-1]] = -inf. tokens: int64 [rows, max_len] holding
 * step+1 generated tokens per row; lprobs: fp32 [rows, vocab], updated in
 * place. Nothing happens while step+1 < n. Token ids outside [0, vocab) are
 * ignored.
 * Replaces ngram_repeat_block_forward
 * (oslo/fused_kernels/bindings/pybind_kernels.cpp:129-157,
 *  oslo/fused_kernels/fused_ngram_repeat_block.cu:18-75); `rows` is its
 * bsz * beam_size.
 */
int oslo_ngram_repeat_block(float *lprobs, const int64_t *tokens, int64_t rows,
                            int64_t max_len, int64_t step, int64_t vocab, int n,
                            oslo_stream_t stream);

/* Dataset index builders (host memory, no device work) ------------------------ */

/*
 * Rows of the array oslo_build_sample_idx fills:
 * (num_epochs * tokens_per_epoch - 1) / seq_length + 1, or -1 for arguments the
 * builder rejects (seq_length <= 1, num_epochs <= 0, tokens_per_epoch <= 1).
 */
int64_t oslo_sample_idx_rows(int32_t seq_length, int32_t num_epochs,
                             int64_t tokens_per_epoch);

/*
 * sample_idx: int32 [rows, 2], host memory. The documents, taken in doc_idx
 * order, form one token stream (document d has sizes[d] tokens); sample k is
 * seq_length + 1 tokens of it and starts on the last token of sample k-1.
 * Row k = (position in doc_idx, offset inside that document) of the first
 * token of sample k; the last row is the end of the last sample. Fails with
 * OSLO_E_BAD_ARG, leaving sample_idx partly written, if doc_idx names a
 * document outside [0, num_docs) or runs out of tokens.
 * Replaces build_sample_idx
 * (oslo/fused_kernels/bindings/pybind_datasets.cpp:85-160), which allocates
 * the array itself and checks nothing.
 */
int oslo_build_sample_idx(int32_t *sample_idx, int64_t rows, const int32_t *sizes,
                          int64_t num_docs, const int32_t *doc_idx,
                          int64_t doc_idx_len, int32_t seq_length,
                          int32_t num_epochs, int64_t tokens_per_epoch);

/*
 * dataset_index: int32 [size]; dataset_sample_index: int64 [size]; weights:
 * double [num_datasets]; host memory. Sample i is given to the dataset d that
 * maximises weights[d] * max(i, 1) - (samples given to d so far), lowest d on
 * ties; dataset_sample_index[i] is that dataset's count before the sample.
 * Replaces build_blending_indices
 * (oslo/fused_kernels/bindings/pybind_datasets.cpp:35-82).
 */
int oslo_build_blending_indices(int32_t *dataset_index,
                                int64_t *dataset_sample_index,
                                const double *weights, int32_t num_datasets,
                                int64_t size);

/*
 * Samples of consecutive sentences for a BERT-style dataset. docs: int64
 * [docs_len], document d is the sentences docs[d] .. docs[d+1]-1; sizes: int32
 * [sizes_len], tokens per sentence; host memory. Every epoch walks the
 * documents in order; a document with fewer than min_num_sent sentences, or
 * (if it has at least two) with a sentence of more than 512 tokens, is skipped;
 * sentences are added to a sample until its length reaches the target and at
 * least min_num_sent sentences are in it and more than one is left in the
 * document, or until the document ends. The target is max_seq_length, except
 * that with short_seq_prob > 0 one draw in round(1/short_seq_prob) of
 * mt19937(seed) gives a short one, 2 + draw mod (max_seq_length - 1). An epoch
 * is not started once max_num_samples rows exist. The rows of all epochs are
 * shuffled with mt19937_64(seed + 1), from the last row down.
 * With maps == NULL the call returns the number of rows; otherwise maps must
 * hold exactly that many rows of 3 indices (first sentence, one past the last,
 * target length), uint32 (index_bytes 4) or uint64 (8; needed beyond 2^32
 * sentences), and the same number is returned. A negative return value is an
 * oslo_status.
 * Replaces build_mapping
 * (oslo/fused_kernels/bindings/pybind_datasets.cpp:163-372), which allocates
 * the array itself and does not check docs against sizes.
 */
int64_t oslo_build_mapping(void *maps, int64_t rows, int index_bytes,
                           const int64_t *docs, int64_t docs_len,
                           const int32_t *sizes, int64_t sizes_len,
                           int32_t num_epochs, uint64_t max_num_samples,
                           int32_t max_seq_length, double short_seq_prob,
                           int32_t seed, int32_t min_num_sent);

/*
 * Blocks of consecutive sentences for a retrieval dataset: as above with the
 * target max_seq_length - titles_sizes[d] (int32 [docs_len - 1], the tokens of
 * document d's title), at least two sentences per block and behind a block that
 * ends early (one with use_one_sent_blocks), no random lengths. Rows of 4
 * indices: first sentence, one past the last, the document, and the block's
 * serial number within its epoch.
 * Replaces build_blocks_mapping
 * (oslo/fused_kernels/bindings/pybind_datasets.cpp:374-574).
 */
int64_t oslo_build_blocks_mapping(void *maps, int64_t rows, int index_bytes,
                                  const int64_t *docs, int64_t docs_len,
                                  const int32_t *sizes, int64_t sizes_len,
                                  const int32_t *titles_sizes, int32_t num_epochs,
                                  uint64_t max_num_samples, int32_t max_seq_length,
                                  int32_t seed, int use_one_sent_blocks);

#ifdef __cplusplus
}
#endif
#endif /* OSLO_AMD_H_ */
