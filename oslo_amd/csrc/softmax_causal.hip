// Scale + causal (upper-triangular) mask + softmax, forward and backward, for
// gfx950. Behaviour follows oslo/fused_kernels/includes/fused_triang_softmax.h
// :134-351 of the reference (row r sees keys 0..r, the rest of the output row
// is zero) with the optional additive key mask of the unfused attention
// (oslo/models/gpt2/modeling_gpt2.py:214-216) folded in.
//
// The mask is never materialised: the diagonal position follows from the row
// index. Keys above the diagonal are not read (their lanes are switched off
// for the load), and the zeros of the upper triangle are written by the same
// 128-bit stores as the probabilities.

#include "dropout.hpp"
#include "softmax.hpp"

namespace oslo {
namespace {

// ---------------------------------------------------------------------------
// The padding-mask values of a wave's part of a causal row, as raw vectors
// beside the row's own loads. Every wave of a [batch, heads, S, S] batch reads
// the same mask row, and two of three vector-memory instructions of an fp16
// row are mask loads. With STAGE, for rows of 4 vectors per lane on and at
// least two rows per block, the mask row of the block's batch goes through LDS
// once per block and each wave takes its part from there. Measured on fp16,
// forward without dropout: [8,16,2048,2048] 271 -> 245 us, S=1536 181 -> 157,
// S=4096 544 -> 504. What keeps the direct loads, also measured: shorter rows
// (they lose to the barrier, S=1024: 66 -> 78 us), one row per block (nothing
// is shared, S=8192: 1195 -> 1534 us), and the kernels with dropout, where
// the Philox arithmetic hides the mask loads (S=4096: forward 552 -> 566,
// backward 711 -> 740 us). Every thread of the block must call it (barrier).
// ---------------------------------------------------------------------------
template <int VEC, int NCHUNK, int WPR, bool STAGE>
__device__ __forceinline__ void load_pad_row(RawVec<float, VEC> (&praw)[NCHUNK],
                                             const float *__restrict__ pad,
                                             const RowMap &map, int S, int heads,
                                             int64_t slab, uint32_t keys, int sub,
                                             int lane) {
  using Tile = RowTile<VEC, NCHUNK, WPR>;
  constexpr bool kStage = STAGE && NCHUNK * WPR >= 4 && Tile::kRowsPerBlock >= 2;
  const int batch = (int)slab / heads;
  auto direct = [&]() {
    const BufRsrc prs =
        make_rsrc(pad + (int64_t)batch * S, keys * (uint32_t)sizeof(float));
#pragma unroll
    for (int c = 0; c < NCHUNK; ++c)
      praw[c] = buffer_load_raw<float, VEC, false>(
          prs, (uint32_t)Tile::col(c, sub, lane) * (uint32_t)sizeof(float));
  };
  if constexpr (!kStage) {
    direct();
  } else {
    __shared__ __align__(32) float s_pad[Tile::kMaxCols];
    // Row slots ascend within a block: the first one names the block's batch,
    // the last one how far its longest causal row reaches (all of the mask
    // row if the block runs over the end of its first [S, S] slab). A wave of
    // another batch (a block across a batch boundary) loads its own.
    int64_t row0 = mapped_row(map, Tile::kRowsPerBlock, 0);
    int64_t row1 = mapped_row(map, Tile::kRowsPerBlock, Tile::kRowsPerBlock - 1);
    if (row0 >= map.total_rows) row0 = map.total_rows - 1;
    if (row1 >= map.total_rows) row1 = map.total_rows - 1;
    const int64_t slab0 = row0 / S;
    const int batch0 = (int)slab0 / heads;
    const bool staged = batch == batch0; // wave-uniform
    const int64_t reach = row1 - slab0 * S;
    const int top = reach >= S ? S : ((int)reach / VEC + 1) * VEC;
    const BufRsrc srs = make_rsrc(pad + (int64_t)batch0 * S,
                                  (uint32_t)top * (uint32_t)sizeof(float));
    for (int i = threadIdx.x * VEC; i < top; i += kBlockThreads * VEC)
      *reinterpret_cast<RawVec<float, VEC> *>(&s_pad[i]) =
          buffer_load_raw<float, VEC, false>(srs, (uint32_t)i * (uint32_t)sizeof(float));
    if (!staged) direct();
    __syncthreads();
    if (staged) {
#pragma unroll
      for (int c = 0; c < NCHUNK; ++c)
        praw[c] = *reinterpret_cast<const RawVec<float, VEC> *>(
            &s_pad[Tile::col(c, sub, lane)]);
    }
  }
}

// ---------------------------------------------------------------------------
// Register-resident path: rows up to kSoftmaxMaxCols, S a multiple of VEC.
// ---------------------------------------------------------------------------
// DROP: what is written is y * keep / (1-p), the probabilities after attention
// dropout (the keep flag of element (row, k) is drawn for the flat index
// row*S + k of the [batch*heads*S, S] tensor), and the probabilities themselves
// are not stored: the row's maximum and reciprocal sum go to stats[2*row..+1],
// from which the backward recomputes them.
template <typename T, int VEC, int NCHUNK, int WPR, bool HAS_PAD, bool DROP>
__global__ __launch_bounds__(kBlockThreads) void causal_fwd_kernel(
    T *y, float *stats, const T *x, const float *__restrict__ pad, float scale,
    int S, int heads, RowMap map, DropArgs drop) {
  using Tile = RowTile<VEC, NCHUNK, WPR>;
  __shared__ float s_max[kWavesPerBlock];
  __shared__ float s_sum[kWavesPerBlock];

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int sub = wave % WPR;
  int64_t row = mapped_row(map, Tile::kRowsPerBlock, wave / WPR);
  // A row slot past the end keeps its waves alive (they meet the same
  // barriers) on the last row and only skips the stores.
  const bool live = row < map.total_rows;
  if (!live) row = map.total_rows - 1;
  const int64_t slab = row / S;
  const int r = (int)(row - slab * S);
  const T *xr = x + row * S;
  T *yr = y + row * S;

  // Every load of the row is issued first (raw), conversion comes afterwards.
  // The row is bounded at the vector that holds key r: lanes wholly above the
  // diagonal get zeros without touching memory.
  const uint32_t keys = (uint32_t)(r / VEC + 1) * VEC;
  const BufRsrc xrs = make_rsrc(xr, keys * (uint32_t)sizeof(T));
  RawVec<T, VEC> raw[NCHUNK];
  RawVec<float, VEC> praw[HAS_PAD ? NCHUNK : 1];
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c)
    raw[c] = buffer_load_raw<T, VEC, true>(
        xrs, (uint32_t)Tile::col(c, sub, lane) * (uint32_t)sizeof(T));
  if constexpr (HAS_PAD)
    load_pad_row<VEC, NCHUNK, WPR, !DROP>(praw, pad, map, S, heads, slab, keys, sub, lane);

  pin_loaded(raw);
  if constexpr (HAS_PAD) pin_loaded(praw);

  // With nothing added after scaling the row is kept in log2 units,
  // exp(s*x - max) = exp2(x*(s*log2 e) - max'), which saves a multiply per key.
  // With a padding mask the score is scale*x rounded, then + mask rounded, the
  // two steps of the unfused path (they decide a fully masked row, where the
  // sum is rounded at magnitude 1e4).
  constexpr bool kLog2 = !HAS_PAD;
  const float sc = kLog2 ? scale * kLog2e : scale;
  float v[NCHUNK][VEC];
  float m = -INFINITY;
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    // wave-uniform classification of the chunk against the diagonal
    const int first = Tile::col(c, sub, 0);
    if (first > r) continue; // wholly above: never converted, stored as zeros
    const int k0 = Tile::col(c, sub, lane);
    float t[VEC], pv[VEC];
    raw_to_f32<T, VEC>(t, raw[c]);
    if constexpr (HAS_PAD) raw_to_f32<float, VEC>(pv, praw[c]);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      t[j] = __fmul_rn(t[j], sc);
      if constexpr (HAS_PAD) t[j] = __fadd_rn(t[j], pv[j]);
    }
    if (first + Tile::kSpan - 1 <= r) { // wholly at or below: no masking
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        v[c][j] = t[j];
        m = fmaxf(m, t[j]);
      }
    } else { // the chunk the diagonal crosses
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        v[c][j] = (k0 + j <= r) ? t[j] : -INFINITY;
        m = fmaxf(m, v[c][j]);
      }
    }
  }
  m = row_allreduce<WPR>(m, OpMax(), s_max);

  float sum = 0.f;
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    if (Tile::col(c, sub, 0) <= r) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        v[c][j] = kLog2 ? __builtin_amdgcn_exp2f(v[c][j] - m) : exp_shifted(v[c][j], m);
        sum += v[c][j];
      }
    } else {
#pragma unroll
      for (int j = 0; j < VEC; ++j) v[c][j] = 0.f;
    }
  }
  sum = row_allreduce<WPR>(sum, OpAdd(), s_sum);
  const float inv = 1.0f / sum;

  if (!live) return;
  if constexpr (DROP) {
    if (sub == 0 && lane == 0)
      *reinterpret_cast<float2 *>(stats + 2 * row) = make_float2(m, inv);
  }
  const BufRsrc yrs = make_rsrc(yr, (uint32_t)S * (uint32_t)sizeof(T));
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    const uint32_t off = (uint32_t)Tile::col(c, sub, lane) * (uint32_t)sizeof(T);
    float o[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) o[j] = v[c][j] * inv;
    if constexpr (DROP) {
      if (Tile::col(c, sub, 0) <= r) { // wave-uniform; above the diagonal o is 0 already
        bool keep[VEC];
        keep_flags<VEC>(keep, drop.seed, drop.offset,
                        (uint64_t)row * S + Tile::col(c, sub, lane), drop.threshold);
#pragma unroll
        for (int j = 0; j < VEC; ++j) o[j] = keep[j] ? o[j] * drop.keep_scale : 0.f;
      }
    }
    buffer_store_f32<T, VEC, kStreamOut>(yrs, off, o);
  }
}

template <typename T, int VEC, int NCHUNK, int WPR>
__global__ __launch_bounds__(kBlockThreads) void causal_bwd_kernel(
    T *dx, const T *g, const T *y, float scale, int S, RowMap map) {
  using Tile = RowTile<VEC, NCHUNK, WPR>;
  __shared__ float s_sum[kWavesPerBlock];

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int sub = wave % WPR;
  int64_t row = mapped_row(map, Tile::kRowsPerBlock, wave / WPR);
  const bool live = row < map.total_rows;
  if (!live) row = map.total_rows - 1;
  const int r = (int)(row % S);
  const T *gr = g + row * S;
  const T *yr = y + row * S;
  T *dr = dx + row * S;

  // bounded at the vector that holds key r, all loads issued first
  const uint32_t bytes = (uint32_t)(r / VEC + 1) * VEC * (uint32_t)sizeof(T);
  const BufRsrc grs = make_rsrc(gr, bytes);
  const BufRsrc yrs = make_rsrc(yr, bytes);
  RawVec<T, VEC> graw[NCHUNK], yraw[NCHUNK];
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    const uint32_t off = (uint32_t)Tile::col(c, sub, lane) * (uint32_t)sizeof(T);
    graw[c] = buffer_load_raw<T, VEC, true>(grs, off);
    yraw[c] = buffer_load_raw<T, VEC, true>(yrs, off);
  }

  pin_loaded(graw);
  pin_loaded(yraw);

  float gy[NCHUNK][VEC]; // g*y
  float yy[NCHUNK][VEC]; // y
  float sum = 0.f;
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    // wave-uniform classification of the chunk against the diagonal
    const int first = Tile::col(c, sub, 0);
    if (first > r) { // wholly above: contributes nothing, stored as zeros
#pragma unroll
      for (int j = 0; j < VEC; ++j) gy[c][j] = yy[c][j] = 0.f;
      continue;
    }
    const int k0 = Tile::col(c, sub, lane);
    float tg[VEC];
    raw_to_f32<T, VEC>(tg, graw[c]);
    raw_to_f32<T, VEC>(yy[c], yraw[c]);
    if (first + Tile::kSpan - 1 > r) { // the chunk the diagonal crosses
#pragma unroll
      for (int j = 0; j < VEC; ++j)
        // entries above the diagonal are never used, whatever they hold
        if (k0 + j > r) yy[c][j] = tg[j] = 0.f;
    }
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      gy[c][j] = tg[j] * yy[c][j];
      sum += gy[c][j];
    }
  }
  sum = row_allreduce<WPR>(sum, OpAdd(), s_sum);

  if (!live) return;
  const BufRsrc drs = make_rsrc(dr, (uint32_t)S * (uint32_t)sizeof(T));
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    float o[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) o[j] = scale * (gy[c][j] - yy[c][j] * sum);
    buffer_store_f32<T, VEC, kStreamOut>(
        drs, (uint32_t)Tile::col(c, sub, lane) * (uint32_t)sizeof(T), o);
  }
}

// Backward of the forward with dropout. g is the gradient of the probabilities
// after dropout; the keep mask is regenerated and g' = g * keep / (1-p) takes
// g's place. The probabilities are recomputed from the scores and the row's
// (max, 1/sum) with the forward's own arithmetic, one exp2 per key and no
// reduction, so the forward never had to store them.
template <typename T, int VEC, int NCHUNK, int WPR, bool HAS_PAD>
__global__ __launch_bounds__(kBlockThreads) void causal_dropout_bwd_kernel(
    T *dx, const T *g, const T *x, const float *__restrict__ stats,
    const float *__restrict__ pad, float scale, int S, int heads, RowMap map,
    DropArgs drop) {
  using Tile = RowTile<VEC, NCHUNK, WPR>;
  __shared__ float s_sum[kWavesPerBlock];

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int sub = wave % WPR;
  int64_t row = mapped_row(map, Tile::kRowsPerBlock, wave / WPR);
  const bool live = row < map.total_rows;
  if (!live) row = map.total_rows - 1;
  const int64_t slab = row / S;
  const int r = (int)(row - slab * S);
  const T *gr = g + row * S;
  const T *xr = x + row * S;
  T *dr = dx + row * S;

  const uint32_t keys = (uint32_t)(r / VEC + 1) * VEC;
  const BufRsrc grs = make_rsrc(gr, keys * (uint32_t)sizeof(T));
  const BufRsrc xrs = make_rsrc(xr, keys * (uint32_t)sizeof(T));
  RawVec<T, VEC> graw[NCHUNK], xraw[NCHUNK];
  RawVec<float, VEC> praw[HAS_PAD ? NCHUNK : 1];
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    const uint32_t off = (uint32_t)Tile::col(c, sub, lane) * (uint32_t)sizeof(T);
    graw[c] = buffer_load_raw<T, VEC, true>(grs, off);
    xraw[c] = buffer_load_raw<T, VEC, true>(xrs, off);
  }
  if constexpr (HAS_PAD)
    load_pad_row<VEC, NCHUNK, WPR, false>(praw, pad, map, S, heads, slab, keys, sub, lane);
  const float2 st = *reinterpret_cast<const float2 *>(stats + 2 * row);
  const float m = st.x, inv = st.y;

  pin_loaded(graw);
  pin_loaded(xraw);
  if constexpr (HAS_PAD) pin_loaded(praw);

  constexpr bool kLog2 = !HAS_PAD; // the forward's exponent domain
  const float sc = kLog2 ? scale * kLog2e : scale;
  float gy[NCHUNK][VEC]; // g'*y
  float yy[NCHUNK][VEC]; // y
  float sum = 0.f;
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    const int first = Tile::col(c, sub, 0);
    if (first > r) { // wholly above the diagonal
#pragma unroll
      for (int j = 0; j < VEC; ++j) gy[c][j] = yy[c][j] = 0.f;
      continue;
    }
    const int k0 = Tile::col(c, sub, lane);
    float tg[VEC], t[VEC], pv[VEC];
    raw_to_f32<T, VEC>(tg, graw[c]);
    raw_to_f32<T, VEC>(t, xraw[c]);
    if constexpr (HAS_PAD) raw_to_f32<float, VEC>(pv, praw[c]);
    bool keep[VEC];
    keep_flags<VEC>(keep, drop.seed, drop.offset, (uint64_t)row * S + k0, drop.threshold);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      t[j] = __fmul_rn(t[j], sc);
      if constexpr (HAS_PAD) t[j] = __fadd_rn(t[j], pv[j]);
      yy[c][j] = (kLog2 ? __builtin_amdgcn_exp2f(t[j] - m) : exp_shifted(t[j], m)) * inv;
      tg[j] = keep[j] ? tg[j] * drop.keep_scale : 0.f;
    }
    if (first + Tile::kSpan - 1 > r) { // the chunk the diagonal crosses
#pragma unroll
      for (int j = 0; j < VEC; ++j)
        if (k0 + j > r) yy[c][j] = tg[j] = 0.f;
    }
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      gy[c][j] = tg[j] * yy[c][j];
      sum += gy[c][j];
    }
  }
  sum = row_allreduce<WPR>(sum, OpAdd(), s_sum);

  if (!live) return;
  const BufRsrc drs = make_rsrc(dr, (uint32_t)S * (uint32_t)sizeof(T));
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    float o[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) o[j] = scale * (gy[c][j] - yy[c][j] * sum);
    buffer_store_f32<T, VEC, kStreamOut>(
        drs, (uint32_t)Tile::col(c, sub, lane) * (uint32_t)sizeof(T), o);
  }
}

// ---------------------------------------------------------------------------
// Any-shape path: one wave per row, element-wise accesses, three passes over
// the row (the second and third come from cache). Used when S is not a
// multiple of the vector width or a pointer is not 16-byte aligned.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(kBlockThreads) void causal_fwd_anyshape_kernel(
    T *y, float *stats, const T *x, const float *__restrict__ pad, float scale,
    int S, int heads, int64_t total_rows, DropArgs drop, bool with_dropout) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t row = (int64_t)blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
  if (row >= total_rows) return; // whole wave leaves; no barriers below
  const int64_t slab = row / S;
  const int r = (int)(row - slab * S);
  const T *xr = x + row * S;
  T *yr = y + row * S;
  const float *padr = pad ? pad + (slab / heads) * S : nullptr;

  // the exponent domain of the register-resident kernels: log2 units unless a
  // padding mask is added
  const bool log2_units = padr == nullptr;
  const float sc = log2_units ? scale * kLog2e : scale;
  auto score = [&](int k) {
    float e = __fmul_rn(static_cast<float>(xr[k]), sc);
    if (padr) e = __fadd_rn(e, padr[k]);
    return e;
  };
  auto ex = [&](float e, float m) {
    return log2_units ? __builtin_amdgcn_exp2f(e - m) : exp_shifted(e, m);
  };
  float m = -INFINITY;
  for (int k = lane; k <= r; k += kWave) m = fmaxf(m, score(k));
  m = wave_allreduce(m, OpMax());
  float sum = 0.f;
  for (int k = lane; k <= r; k += kWave) sum += ex(score(k), m);
  sum = wave_allreduce(sum, OpAdd());
  const float inv = 1.0f / sum;
  if (with_dropout && lane == 0) {
    stats[2 * row] = m;
    stats[2 * row + 1] = inv;
  }
  // x is read before y is written at the same index, so y may alias x
  for (int k = lane; k < S; k += kWave) {
    float o = k <= r ? ex(score(k), m) * inv : 0.f;
    if (with_dropout)
      o = keep_one(drop.seed, drop.offset, (uint64_t)row * S + k, drop.threshold)
              ? o * drop.keep_scale : 0.f;
    yr[k] = static_cast<T>(o);
  }
}

template <typename T>
__global__ __launch_bounds__(kBlockThreads) void causal_bwd_anyshape_kernel(
    T *dx, const T *g, const T *y, float scale, int S, int64_t total_rows) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t row = (int64_t)blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
  if (row >= total_rows) return;
  const int r = (int)(row % S);
  const T *gr = g + row * S;
  const T *yr = y + row * S;
  T *dr = dx + row * S;
  float sum = 0.f;
  for (int k = lane; k <= r; k += kWave)
    sum += static_cast<float>(gr[k]) * static_cast<float>(yr[k]);
  sum = wave_allreduce(sum, OpAdd());
  for (int k = lane; k < S; k += kWave) {
    float o = 0.f;
    if (k <= r) {
      const float yk = static_cast<float>(yr[k]);
      o = scale * (static_cast<float>(gr[k]) * yk - yk * sum);
    }
    dr[k] = static_cast<T>(o);
  }
}

template <typename T>
__global__ __launch_bounds__(kBlockThreads) void causal_dropout_bwd_anyshape_kernel(
    T *dx, const T *g, const T *x, const float *__restrict__ stats,
    const float *__restrict__ pad, float scale, int S, int heads,
    int64_t total_rows, DropArgs drop) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t row = (int64_t)blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
  if (row >= total_rows) return;
  const int64_t slab = row / S;
  const int r = (int)(row - slab * S);
  const T *gr = g + row * S;
  const T *xr = x + row * S;
  T *dr = dx + row * S;
  const float *padr = pad ? pad + (slab / heads) * S : nullptr;
  const bool log2_units = padr == nullptr;
  const float sc = log2_units ? scale * kLog2e : scale;
  const float m = stats[2 * row], inv = stats[2 * row + 1];
  auto prob = [&](int k) {
    float e = __fmul_rn(static_cast<float>(xr[k]), sc);
    if (padr) e = __fadd_rn(e, padr[k]);
    return (log2_units ? __builtin_amdgcn_exp2f(e - m) : exp_shifted(e, m)) * inv;
  };
  auto grad = [&](int k) { // gradient of the probabilities before dropout
    const float gk = static_cast<float>(gr[k]);
    return keep_one(drop.seed, drop.offset, (uint64_t)row * S + k, drop.threshold)
               ? gk * drop.keep_scale : 0.f;
  };
  float sum = 0.f;
  for (int k = lane; k <= r; k += kWave) sum += grad(k) * prob(k);
  sum = wave_allreduce(sum, OpAdd());
  // g and x are read before dx is written at the same index
  for (int k = lane; k < S; k += kWave) {
    float o = 0.f;
    if (k <= r) {
      const float yk = prob(k);
      o = scale * (grad(k) * yk - yk * sum);
    }
    dr[k] = static_cast<T>(o);
  }
}

// with_dropout: y receives the probabilities after dropout and stats the
// per-row (max, 1/sum).
template <typename T>
int launch_causal_fwd(T *y, float *stats, const T *x, const float *pad,
                      float scale, int64_t batch, int64_t heads, int64_t S,
                      const DropArgs &drop, bool with_dropout, hipStream_t stream) {
  constexpr int VEC = Io<T>::kVec;
  const int64_t total_rows = batch * heads * S;
  const bool vector_ok = S % VEC == 0 && aligned16(x) && aligned16(y) &&
                         (pad == nullptr || aligned16(pad)) &&
                         (stats == nullptr || (uintptr_t)stats % 8 == 0);
  if (!vector_ok) {
    const int64_t blocks = (total_rows + kWavesPerBlock - 1) / kWavesPerBlock;
    causal_fwd_anyshape_kernel<T><<<dim3((unsigned)blocks), dim3(kBlockThreads),
                                    0, stream>>>(y, stats, x, pad, scale, (int)S,
                                                 (int)heads, total_rows, drop,
                                                 with_dropout);
    return check_launch("softmax_causal_fwd");
  }
  dispatch_row_tile<VEC>(S, [&]<int NCHUNK, int WPR>() {
    constexpr int rpb = RowTile<VEC, NCHUNK, WPR>::kRowsPerBlock;
    const RowMap map = make_row_map(total_rows, rpb, S * (int64_t)sizeof(T), true);
    const dim3 grid((unsigned)(map.blocks_per_xcd * kXcds));
    // the variants with dropout (Philox) or a padding mask (its loads, and one
    // more multiply and add per key) carry more arithmetic per byte and want
    // every wave the registers allow: measured 277 -> 267 us with the mask
    // read directly, and with the mask staged in LDS a cap at 5 or 6 blocks
    // per CU still loses (245 -> 299 and 269 us)
    const unsigned lds = (with_dropout || pad)
                             ? 0u
                             : occupancy_pad_bytes(false, S * (int64_t)sizeof(T));
    auto go = [&]<bool HAS_PAD, bool DROP>() {
      causal_fwd_kernel<T, VEC, NCHUNK, WPR, HAS_PAD, DROP>
          <<<grid, dim3(kBlockThreads), lds, stream>>>(
              y, stats, x, pad, scale, (int)S, (int)heads, map, drop);
    };
    if (with_dropout) {
      if (pad) go.template operator()<true, true>();
      else go.template operator()<false, true>();
    } else {
      if (pad) go.template operator()<true, false>();
      else go.template operator()<false, false>();
    }
  });
  return check_launch("softmax_causal_fwd");
}

template <typename T>
int launch_causal_bwd(T *dx, const T *g, const T *y, float scale, int64_t bh,
                      int64_t S, hipStream_t stream) {
  constexpr int VEC = Io<T>::kVec;
  const int64_t total_rows = bh * S;
  const bool vector_ok =
      S % VEC == 0 && aligned16(dx) && aligned16(g) && aligned16(y);
  if (!vector_ok) {
    const int64_t blocks = (total_rows + kWavesPerBlock - 1) / kWavesPerBlock;
    causal_bwd_anyshape_kernel<T><<<dim3((unsigned)blocks), dim3(kBlockThreads),
                                    0, stream>>>(dx, g, y, scale, (int)S, total_rows);
    return check_launch("softmax_causal_bwd");
  }
  dispatch_row_tile<VEC>(S, [&]<int NCHUNK, int WPR>() {
    constexpr int rpb = RowTile<VEC, NCHUNK, WPR>::kRowsPerBlock;
    const RowMap map = make_row_map(total_rows, rpb, S * (int64_t)sizeof(T), true);
    const dim3 grid((unsigned)(map.blocks_per_xcd * kXcds));
    const unsigned lds = occupancy_pad_bytes(true, S * (int64_t)sizeof(T));
    causal_bwd_kernel<T, VEC, NCHUNK, WPR>
        <<<grid, dim3(kBlockThreads), lds, stream>>>(dx, g, y, scale, (int)S, map);
  });
  return check_launch("softmax_causal_bwd");
}

template <typename T>
int launch_causal_dropout_bwd(T *dx, const T *g, const T *x, const float *stats,
                              const float *pad, float scale, int64_t batch,
                              int64_t heads, int64_t S, const DropArgs &drop,
                              hipStream_t stream) {
  constexpr int VEC = Io<T>::kVec;
  const int64_t total_rows = batch * heads * S;
  const bool vector_ok = S % VEC == 0 && aligned16(dx) && aligned16(g) &&
                         aligned16(x) && (pad == nullptr || aligned16(pad)) &&
                         (uintptr_t)stats % 8 == 0;
  if (!vector_ok) {
    const int64_t blocks = (total_rows + kWavesPerBlock - 1) / kWavesPerBlock;
    causal_dropout_bwd_anyshape_kernel<T>
        <<<dim3((unsigned)blocks), dim3(kBlockThreads), 0, stream>>>(
            dx, g, x, stats, pad, scale, (int)S, (int)heads, total_rows, drop);
    return check_launch("softmax_causal_dropout_bwd");
  }
  dispatch_row_tile<VEC>(S, [&]<int NCHUNK, int WPR>() {
    constexpr int rpb = RowTile<VEC, NCHUNK, WPR>::kRowsPerBlock;
    const RowMap map = make_row_map(total_rows, rpb, S * (int64_t)sizeof(T), true);
    const dim3 grid((unsigned)(map.blocks_per_xcd * kXcds));
    const unsigned lds = 0; // as in the forward with dropout: no occupancy cap
    if (pad)
      causal_dropout_bwd_kernel<T, VEC, NCHUNK, WPR, true>
          <<<grid, dim3(kBlockThreads), lds, stream>>>(
              dx, g, x, stats, pad, scale, (int)S, (int)heads, map, drop);
    else
      causal_dropout_bwd_kernel<T, VEC, NCHUNK, WPR, false>
          <<<grid, dim3(kBlockThreads), lds, stream>>>(
              dx, g, x, stats, pad, scale, (int)S, (int)heads, map, drop);
  });
  return check_launch("softmax_causal_dropout_bwd");
}

// Shared argument screening. Returns 1 when there is nothing to do.
int screen(const char *name, int64_t rows, int64_t S) {
  if (rows < 0 || S < 0)
    return fail(OSLO_E_BAD_ARG, "%s: negative size", name);
  if (S > kSoftmaxMaxCols)
    return fail(OSLO_E_UNSUPPORTED, "%s: row length %lld exceeds %d", name,
                (long long)S, kSoftmaxMaxCols);
  if (S > 0 && rows > (int64_t)INT32_MAX / S)
    return fail(OSLO_E_UNSUPPORTED, "%s: too many rows for one launch", name);
  return (rows == 0 || S == 0) ? 1 : 0;
}

} // namespace
} // namespace oslo

namespace {
int causal_fwd_entry(const char *name, void *y, float *stats, const void *x,
                     const float *pad_add, float scale, const oslo::DropArgs &drop,
                     bool with_dropout, int64_t batch, int64_t heads, int64_t S,
                     int dtype, oslo_stream_t stream) {
  using namespace oslo;
  if (batch < 0 || heads < 0) return fail(OSLO_E_BAD_ARG, "%s: negative size", name);
  const int s = screen(name, batch * heads, S);
  if (s != 0) return s < 0 ? s : OSLO_OK;
  if (!x || !y || (with_dropout && !stats))
    return fail(OSLO_E_BAD_ARG, "%s: null tensor", name);
  OSLO_DISPATCH_DTYPE(dtype, return launch_causal_fwd<T>(
                                 static_cast<T *>(y), stats, static_cast<const T *>(x),
                                 pad_add, scale, batch, heads, S, drop, with_dropout,
                                 static_cast<hipStream_t>(stream)));
  return OSLO_OK;
}
} // namespace

extern "C" int oslo_softmax_causal_fwd(void *y, const void *x,
                                       const float *pad_add, float scale,
                                       int64_t batch, int64_t heads, int64_t S,
                                       int dtype, oslo_stream_t stream) {
  oslo::DropArgs none{};
  return causal_fwd_entry("softmax_causal_fwd", y, nullptr, x, pad_add, scale, none,
                          false, batch, heads, S, dtype, stream);
}

extern "C" int oslo_softmax_causal_bwd(void *dx, const void *g, const void *y,
                                       float scale, int64_t bh, int64_t S,
                                       int dtype, oslo_stream_t stream) {
  using namespace oslo;
  const int s = screen("softmax_causal_bwd", bh, S);
  if (s != 0) return s < 0 ? s : OSLO_OK;
  if (!dx || !g || !y) return fail(OSLO_E_BAD_ARG, "softmax_causal_bwd: null tensor");
  OSLO_DISPATCH_DTYPE(dtype, return launch_causal_bwd<T>(
                                 static_cast<T *>(dx), static_cast<const T *>(g),
                                 static_cast<const T *>(y), scale, bh, S,
                                 static_cast<hipStream_t>(stream)));
  return OSLO_OK;
}

extern "C" int oslo_softmax_causal_dropout_fwd(void *yd, float *row_stats,
                                               const void *x, const float *pad_add,
                                               float scale, float p,
                                               uint64_t philox_seed,
                                               uint64_t philox_offset, int64_t batch,
                                               int64_t heads, int64_t S, int dtype,
                                               oslo_stream_t stream) {
  oslo::DropArgs drop;
  const int s = oslo::make_drop_args("softmax_causal_dropout_fwd", p, philox_seed,
                                     philox_offset, &drop);
  if (s != OSLO_OK) return s;
  return causal_fwd_entry("softmax_causal_dropout_fwd", yd, row_stats, x, pad_add,
                          scale, drop, true, batch, heads, S, dtype, stream);
}

extern "C" int oslo_softmax_causal_dropout_bwd(void *dx, const void *g, const void *x,
                                               const float *row_stats,
                                               const float *pad_add, float scale,
                                               float p, uint64_t philox_seed,
                                               uint64_t philox_offset, int64_t batch,
                                               int64_t heads, int64_t S, int dtype,
                                               oslo_stream_t stream) {
  using namespace oslo;
  const char *name = "softmax_causal_dropout_bwd";
  DropArgs drop;
  int s = make_drop_args(name, p, philox_seed, philox_offset, &drop);
  if (s != OSLO_OK) return s;
  if (batch < 0 || heads < 0) return fail(OSLO_E_BAD_ARG, "%s: negative size", name);
  s = screen(name, batch * heads, S);
  if (s != 0) return s < 0 ? s : OSLO_OK;
  if (!dx || !g || !x || !row_stats) return fail(OSLO_E_BAD_ARG, "%s: null tensor", name);
  OSLO_DISPATCH_DTYPE(dtype, return launch_causal_dropout_bwd<T>(
                                 static_cast<T *>(dx), static_cast<const T *>(g),
                                 static_cast<const T *>(x), row_stats, pad_add, scale,
                                 batch, heads, S, drop,
                                 static_cast<hipStream_t>(stream)));
  return OSLO_OK;
}
