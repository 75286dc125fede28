// Bias + dropout (+ residual add), forward and backward, for gfx950:
// out = dropout(x + bias, p) + residual, the arithmetic of bias_dropout /
// bias_dropout_residual (oslo/fused_kernels_utils.py:259-292). A second
// residual can be added in the same pass (GPT-J's block sums attention output,
// feed-forward output and the residual stream,
// oslo/models/gptj/modeling_gptj.py:319-320): the three-term sum is formed in
// fp32 and rounded once, where two passes would round the sum twice at the
// magnitude of the residual stream. The keep mask
// is never stored: forward and backward both derive it from
// (seed, offset, element index) with Philox4x32-10, so the backward reads only
// the incoming gradient.

#include "dropout.hpp"
#include "elementwise.hpp"

namespace oslo {
namespace {

// RES: how many residual tensors are added (0, 1 or 2)
template <typename T, int VEC, int U, bool DROP, bool HAS_BIAS, int RES, int OUT>
__global__ __launch_bounds__(kBlockThreads) void bias_dropout_add_fwd_kernel(
    T *out, const T *x, const T *__restrict__ bias, const T *residual, const T *residual2,
    float keep_scale, uint32_t threshold, uint64_t seed, uint64_t offset,
    int64_t rows, int64_t cols, int col_tiles, int rows_per_block) {
  const EwPos pos = ew_position<VEC>(col_tiles, rows_per_block);
  if (pos.c0 >= cols) return; // no barrier in this kernel
  const int TY = blockDim.y;
  const BufRsrc xrs = ew_rsrc<T>(x, pos, rows_per_block, rows, cols);
  constexpr bool HAS_RES = RES >= 1, HAS_RES2 = RES >= 2;
  RawVec<T, VEC> xraw[U], rraw[HAS_RES ? U : 1], r2raw[HAS_RES2 ? U : 1];
#pragma unroll
  for (int u = 0; u < U; ++u)
    xraw[u] = buffer_load_raw<T, VEC, true>(xrs, ew_offset<T>(pos, u, cols));
  if constexpr (HAS_RES) {
    const BufRsrc rrs = ew_rsrc<T>(residual, pos, rows_per_block, rows, cols);
#pragma unroll
    for (int u = 0; u < U; ++u)
      rraw[u] = buffer_load_raw<T, VEC, true>(rrs, ew_offset<T>(pos, u, cols));
  }
  if constexpr (HAS_RES2) {
    const BufRsrc rrs = ew_rsrc<T>(residual2, pos, rows_per_block, rows, cols);
#pragma unroll
    for (int u = 0; u < U; ++u)
      r2raw[u] = buffer_load_raw<T, VEC, true>(rrs, ew_offset<T>(pos, u, cols));
  }
  float b[VEC];
  if constexpr (HAS_BIAS) load_f32_cached<T, VEC>(b, bias + pos.c0);
  // rows past the end were read as zeros and their stores are dropped by the
  // same bound, so the body has no branch
  const BufRsrc ors = ew_rsrc<T>(out, pos, rows_per_block, rows, cols);
  float tx[U][VEC], tr[U][VEC], tr2[VEC];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int64_t r = pos.r_base + (int64_t)u * TY;
    raw_to_f32<T, VEC>(tx[u], xraw[u]);
    if constexpr (HAS_RES) raw_to_f32<T, VEC>(tr[u], rraw[u]);
    if constexpr (HAS_RES2) raw_to_f32<T, VEC>(tr2, r2raw[u]);
    bool keep[VEC];
    if constexpr (DROP)
      keep_flags<VEC>(keep, seed, offset, (uint64_t)(r * cols + pos.c0), threshold);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      float t = tx[u][j];
      if constexpr (HAS_BIAS) t += b[j];
      if constexpr (DROP) t = keep[j] ? t * keep_scale : 0.f;
      if constexpr (HAS_RES) t += tr[u][j];
      if constexpr (HAS_RES2) t += tr2[j];
      tx[u][j] = t;
    }
    buffer_store_f32<T, VEC, OUT>(ors, ew_offset<T>(pos, u, cols), tx[u]);
  }
}

template <typename T, int VEC, int U, bool DROP, bool WANT_DBIAS, int OUT>
__global__ __launch_bounds__(kBlockThreads) void bias_dropout_add_bwd_kernel(
    T *dx, float *__restrict__ partial, const T *g, float keep_scale,
    uint32_t threshold, uint64_t seed, uint64_t offset, int64_t rows,
    int64_t cols, int col_tiles, int rows_per_block) {
  const EwPos pos = ew_position<VEC>(col_tiles, rows_per_block);
  const bool col_ok = pos.c0 < cols;
  const int TY = blockDim.y;
  float acc[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) acc[j] = 0.f;
  if (col_ok) {
    const BufRsrc grs = ew_rsrc<T>(g, pos, rows_per_block, rows, cols);
    RawVec<T, VEC> graw[U];
#pragma unroll
    for (int u = 0; u < U; ++u)
      graw[u] = buffer_load_raw<T, VEC, true>(grs, ew_offset<T>(pos, u, cols));
    // rows past the end were read as zeros (they add nothing to dbias) and
    // their stores are dropped by the same bound
    const BufRsrc drs = ew_rsrc<T>(dx, pos, rows_per_block, rows, cols);
    float tg[U][VEC];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t r = pos.r_base + (int64_t)u * TY;
      raw_to_f32<T, VEC>(tg[u], graw[u]);
      bool keep[VEC];
      if constexpr (DROP)
        keep_flags<VEC>(keep, seed, offset, (uint64_t)(r * cols + pos.c0), threshold);
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        if constexpr (DROP) tg[u][j] = keep[j] ? tg[u][j] * keep_scale : 0.f;
        if constexpr (WANT_DBIAS) acc[j] += tg[u][j];
      }
      // with no dropout dx == g bit for bit; still written, dx may be a
      // different buffer
      buffer_store_f32<T, VEC, OUT>(drs, ew_offset<T>(pos, u, cols), tg[u]);
    }
  }
  if constexpr (WANT_DBIAS)
    write_colsum_partial<VEC>(acc, partial, cols, pos);
}

constexpr int kDropBwdUnroll = 4;
static_assert(kDropBwdUnroll >= kBwdMinUnroll, "workspace bound");

template <typename T, int VEC>
int launch_fwd(T *out, const T *x, const T *bias, const T *res, const T *res2,
               const DropArgs &a, int64_t rows, int64_t cols,
               hipStream_t stream) {
  const EwPlan p = plan_elementwise(rows, cols / VEC, kFwdMaxTx, kFwdUnroll);
  if (!p.ok) return fail(OSLO_E_UNSUPPORTED, "bias_dropout_add_fwd: tensor too large for one launch");
  const bool keep = keep_output_cached(rows * cols * (int64_t)sizeof(T));
  auto go = [&]<bool DROP, bool HB, int RES>() {
    if (keep)
      bias_dropout_add_fwd_kernel<T, VEC, kFwdUnroll, DROP, HB, RES, kOutKeep>
          <<<p.grid, p.block, 0, stream>>>(out, x, bias, res, res2, a.keep_scale,
                                           a.threshold, a.seed, a.offset, rows,
                                           cols, p.col_tiles, p.rows_per_block);
    else
      bias_dropout_add_fwd_kernel<T, VEC, kFwdUnroll, DROP, HB, RES, kOutStream>
          <<<p.grid, p.block, 0, stream>>>(out, x, bias, res, res2, a.keep_scale,
                                           a.threshold, a.seed, a.offset, rows,
                                           cols, p.col_tiles, p.rows_per_block);
  };
  auto with_residuals = [&]<bool DROP, bool HB>() {
    if (res2) go.template operator()<DROP, HB, 2>();
    else if (res) go.template operator()<DROP, HB, 1>();
    else go.template operator()<DROP, HB, 0>();
  };
  if (a.drop) {
    if (bias) with_residuals.template operator()<true, true>();
    else with_residuals.template operator()<true, false>();
  } else {
    if (bias) with_residuals.template operator()<false, true>();
    else with_residuals.template operator()<false, false>();
  }
  return check_launch("bias_dropout_add_fwd");
}

template <typename T, int VEC>
int launch_bwd(T *dx, T *dbias, float *ws, const T *g, const DropArgs &a,
               int64_t rows, int64_t cols, hipStream_t stream) {
  const EwPlan p = plan_elementwise(rows, cols / VEC, kBwdMaxTx, kDropBwdUnroll);
  if (!p.ok) return fail(OSLO_E_UNSUPPORTED, "bias_dropout_add_bwd: tensor too large for one launch");
  const bool keep = keep_output_cached(rows * cols * (int64_t)sizeof(T));
  auto go = [&]<bool DROP, bool WANT>() {
    if (keep)
      bias_dropout_add_bwd_kernel<T, VEC, kDropBwdUnroll, DROP, WANT, kOutKeep>
          <<<p.grid, p.block, 0, stream>>>(dx, ws, g, a.keep_scale, a.threshold,
                                           a.seed, a.offset, rows, cols,
                                           p.col_tiles, p.rows_per_block);
    else
      bias_dropout_add_bwd_kernel<T, VEC, kDropBwdUnroll, DROP, WANT, kOutStream>
          <<<p.grid, p.block, 0, stream>>>(dx, ws, g, a.keep_scale, a.threshold,
                                           a.seed, a.offset, rows, cols,
                                           p.col_tiles, p.rows_per_block);
  };
  if (a.drop) {
    if (dbias) go.template operator()<true, true>();
    else go.template operator()<true, false>();
  } else {
    if (dbias) go.template operator()<false, true>();
    else go.template operator()<false, false>();
  }
  int s = check_launch("bias_dropout_add_bwd");
  if (s != OSLO_OK || !dbias) return s;
  launch_colsum_finish<T>(dbias, ws, p.row_blocks, cols, stream);
  return check_launch("bias_dropout_add_bwd(dbias)");
}

} // namespace
} // namespace oslo

namespace {
int bias_dropout_add_fwd_entry(void *out, const void *x, const void *bias,
                               const void *residual, const void *residual2, float p,
                               uint64_t philox_seed, uint64_t philox_offset,
                               int64_t rows, int64_t cols, int dtype,
                               oslo_stream_t stream) {
  using namespace oslo;
  if (rows < 0 || cols < 0)
    return fail(OSLO_E_BAD_ARG, "bias_dropout_add_fwd: negative size");
  DropArgs a;
  int s = make_drop_args("bias_dropout_add_fwd", p, philox_seed, philox_offset, &a);
  if (s != OSLO_OK) return s;
  if (rows == 0 || cols == 0) return OSLO_OK;
  if (!out || !x) return fail(OSLO_E_BAD_ARG, "bias_dropout_add_fwd: null tensor");
  if (residual2 && !residual)
    return fail(OSLO_E_BAD_ARG, "bias_dropout_add2_fwd: a second residual without a first");
  hipStream_t st = static_cast<hipStream_t>(stream);
  OSLO_DISPATCH_DTYPE(dtype, {
    constexpr int V = Io<T>::kVec;
    const bool vec = cols % V == 0 && aligned16(out) && aligned16(x) &&
                     aligned16(bias) && aligned16(residual) && aligned16(residual2);
    T *o = static_cast<T *>(out);
    const T *xx = static_cast<const T *>(x);
    const T *bb = static_cast<const T *>(bias);
    const T *rr = static_cast<const T *>(residual);
    const T *r2 = static_cast<const T *>(residual2);
    return vec ? launch_fwd<T, V>(o, xx, bb, rr, r2, a, rows, cols, st)
               : launch_fwd<T, 1>(o, xx, bb, rr, r2, a, rows, cols, st);
  });
  return OSLO_OK;
}
} // namespace

extern "C" int oslo_bias_dropout_add_fwd(void *out, const void *x,
                                         const void *bias, const void *residual,
                                         float p, uint64_t philox_seed,
                                         uint64_t philox_offset, int64_t rows,
                                         int64_t cols, int dtype,
                                         oslo_stream_t stream) {
  return bias_dropout_add_fwd_entry(out, x, bias, residual, nullptr, p, philox_seed,
                                    philox_offset, rows, cols, dtype, stream);
}

extern "C" int oslo_bias_dropout_add2_fwd(void *out, const void *x,
                                          const void *bias, const void *residual,
                                          const void *residual2, float p,
                                          uint64_t philox_seed,
                                          uint64_t philox_offset, int64_t rows,
                                          int64_t cols, int dtype,
                                          oslo_stream_t stream) {
  return bias_dropout_add_fwd_entry(out, x, bias, residual, residual2, p, philox_seed,
                                    philox_offset, rows, cols, dtype, stream);
}

extern "C" int oslo_bias_dropout_add_bwd(void *dx, void *dbias,
                                         float *workspace, const void *g,
                                         float p, uint64_t philox_seed,
                                         uint64_t philox_offset, int64_t rows,
                                         int64_t cols, int dtype,
                                         oslo_stream_t stream) {
  using namespace oslo;
  if (rows < 0 || cols < 0)
    return fail(OSLO_E_BAD_ARG, "bias_dropout_add_bwd: negative size");
  DropArgs a;
  int s = make_drop_args("bias_dropout_add_bwd", p, philox_seed, philox_offset, &a);
  if (s != OSLO_OK) return s;
  if (cols == 0) return OSLO_OK;
  if (dbias && !workspace && rows > 0)
    return fail(OSLO_E_BAD_ARG, "bias_dropout_add_bwd: dbias needs a workspace");
  if (rows > 0 && (!dx || !g))
    return fail(OSLO_E_BAD_ARG, "bias_dropout_add_bwd: null tensor");
  hipStream_t st = static_cast<hipStream_t>(stream);
  OSLO_DISPATCH_DTYPE(dtype, {
    if (rows == 0) {
      if (dbias)
        launch_colsum_finish<T>(static_cast<T *>(dbias), nullptr, 0, cols, st); // writes zeros
      return check_launch("bias_dropout_add_bwd(dbias)");
    }
    constexpr int V = Io<T>::kVec;
    const bool vec = cols % V == 0 && aligned16(dx) && aligned16(g) &&
                     aligned16(workspace);
    T *d = static_cast<T *>(dx);
    T *db = static_cast<T *>(dbias);
    const T *gg = static_cast<const T *>(g);
    return vec ? launch_bwd<T, V>(d, db, workspace, gg, a, rows, cols, st)
               : launch_bwd<T, 1>(d, db, workspace, gg, a, rows, cols, st);
  });
  return OSLO_OK;
}
