// Scale + key/padding mask + softmax, forward and backward, for gfx950.
// Behaviour follows oslo/fused_kernels/includes/fused_softmax.h:111-325 of the
// reference. The mask is addressed through two strides, so a [B,1,1,Sk] key
// mask is read in place (a few KiB that stay in cache) instead of being
// repeated to [B,1,Sq,Sk] the way the reference's caller does
// (oslo/fused_kernels_utils.py:456-458).

#include "softmax.hpp"

namespace oslo {
namespace {

// One masked score. ADD: scale*x rounded, then + (-10000) rounded, the two
// steps of the unfused path; REPLACE: the constant.
template <bool REPLACE>
__device__ __forceinline__ float masked_score(float x, float scale,
                                              uint8_t masked) {
  const float e = __fmul_rn(x, scale);
  if (!masked) return e;
  return REPLACE ? kMaskValue : __fadd_rn(e, kMaskValue);
}

template <typename T, int VEC, int NCHUNK, int WPR, bool HAS_MASK, bool REPLACE>
__global__ __launch_bounds__(kBlockThreads) void masked_fwd_kernel(
    T *y, const T *x, const uint8_t *__restrict__ mask, int64_t mask_stride_b,
    int64_t mask_stride_q, float scale, int Sq, int Sk, int heads,
    RowMap map) {
  using Tile = RowTile<VEC, NCHUNK, WPR>;
  __shared__ float s_max[kWavesPerBlock];
  __shared__ float s_sum[kWavesPerBlock];

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int sub = wave % WPR;
  int64_t row = mapped_row(map, Tile::kRowsPerBlock, wave / WPR);
  const bool live = row < map.total_rows;
  if (!live) row = map.total_rows - 1;
  const T *xr = x + row * Sk;
  T *yr = y + row * Sk;
  const uint8_t *mr = nullptr;
  if constexpr (HAS_MASK) {
    const int64_t bh = row / Sq;
    const int q = (int)(row - bh * Sq);
    mr = mask + (bh / heads) * mask_stride_b + q * mask_stride_q;
  }

  // every load of the row is issued first (raw, bounded at Sk), conversion
  // comes afterwards
  const BufRsrc xrs = make_rsrc(xr, (uint32_t)Sk * (uint32_t)sizeof(T));
  RawVec<T, VEC> raw[NCHUNK];
  RawVec<uint8_t, VEC> mraw[HAS_MASK ? NCHUNK : 1];
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c)
    raw[c] = buffer_load_raw<T, VEC, true>(
        xrs, (uint32_t)Tile::col(c, sub, lane) * (uint32_t)sizeof(T));
  if constexpr (HAS_MASK) {
    const BufRsrc mrs = make_rsrc(mr, (uint32_t)Sk);
#pragma unroll
    for (int c = 0; c < NCHUNK; ++c)
      mraw[c] = buffer_load_raw<uint8_t, VEC, false>(
          mrs, (uint32_t)Tile::col(c, sub, lane));
  }

  float v[NCHUNK][VEC];
  float m = -INFINITY;
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    const int k0 = Tile::col(c, sub, lane);
    float t[VEC];
    raw_to_f32<T, VEC>(t, raw[c]);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      uint8_t mk = 0;
      if constexpr (HAS_MASK) {
        if constexpr (VEC == 1) mk = mraw[c]; else mk = mraw[c][j];
      }
      const float e = masked_score<REPLACE>(t[j], scale, mk);
      v[c][j] = (k0 < Sk) ? e : -INFINITY;
      m = fmaxf(m, v[c][j]);
    }
  }
  m = row_allreduce<WPR>(m, OpMax(), s_max);

  float sum = 0.f;
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    if (Tile::col(c, sub, 0) < Sk) { // wave-uniform
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        v[c][j] = exp_shifted(v[c][j], m);
        sum += v[c][j];
      }
    }
  }
  sum = row_allreduce<WPR>(sum, OpAdd(), s_sum);
  const float inv = 1.0f / sum;

  if (!live) return;
  const BufRsrc yrs = make_rsrc(yr, (uint32_t)Sk * (uint32_t)sizeof(T));
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    float o[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) o[j] = v[c][j] * inv;
    buffer_store_f32<T, VEC, kStreamOut>(
        yrs, (uint32_t)Tile::col(c, sub, lane) * (uint32_t)sizeof(T), o);
  }
}

template <typename T, int VEC, int NCHUNK, int WPR>
__global__ __launch_bounds__(kBlockThreads) void masked_bwd_kernel(
    T *dx, const T *g, const T *y, float scale, int Sk, RowMap map) {
  using Tile = RowTile<VEC, NCHUNK, WPR>;
  __shared__ float s_sum[kWavesPerBlock];

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int sub = wave % WPR;
  int64_t row = mapped_row(map, Tile::kRowsPerBlock, wave / WPR);
  const bool live = row < map.total_rows;
  if (!live) row = map.total_rows - 1;
  const T *gr = g + row * Sk;
  const T *yr = y + row * Sk;
  T *dr = dx + row * Sk;

  const uint32_t bytes = (uint32_t)Sk * (uint32_t)sizeof(T);
  const BufRsrc grs = make_rsrc(gr, bytes);
  const BufRsrc yrs = make_rsrc(yr, bytes);
  RawVec<T, VEC> graw[NCHUNK], yraw[NCHUNK];
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    const uint32_t off = (uint32_t)Tile::col(c, sub, lane) * (uint32_t)sizeof(T);
    graw[c] = buffer_load_raw<T, VEC, true>(grs, off);
    yraw[c] = buffer_load_raw<T, VEC, true>(yrs, off);
  }

  float gy[NCHUNK][VEC];
  float yy[NCHUNK][VEC];
  float sum = 0.f;
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    float tg[VEC];
    raw_to_f32<T, VEC>(tg, graw[c]);
    raw_to_f32<T, VEC>(yy[c], yraw[c]);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      gy[c][j] = tg[j] * yy[c][j];
      sum += gy[c][j];
    }
  }
  sum = row_allreduce<WPR>(sum, OpAdd(), s_sum);

  if (!live) return;
  const BufRsrc drs = make_rsrc(dr, (uint32_t)Sk * (uint32_t)sizeof(T));
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    float o[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) o[j] = scale * (gy[c][j] - yy[c][j] * sum);
    buffer_store_f32<T, VEC, kStreamOut>(
        drs, (uint32_t)Tile::col(c, sub, lane) * (uint32_t)sizeof(T), o);
  }
}

// Any-shape path (Sk not a multiple of the vector width, odd strides or
// unaligned pointers): one wave per row, element-wise accesses.
template <typename T>
__global__ __launch_bounds__(kBlockThreads) void masked_fwd_anyshape_kernel(
    T *y, const T *x, const uint8_t *__restrict__ mask, int64_t mask_stride_b,
    int64_t mask_stride_q, int replace, float scale, int Sq, int Sk, int heads,
    int64_t total_rows) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t row = (int64_t)blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
  if (row >= total_rows) return;
  const T *xr = x + row * Sk;
  T *yr = y + row * Sk;
  const uint8_t *mr = nullptr;
  if (mask) {
    const int64_t bh = row / Sq;
    mr = mask + (bh / heads) * mask_stride_b + (row - bh * Sq) * mask_stride_q;
  }
  auto score = [&](int k) {
    const float xv = static_cast<float>(xr[k]);
    const uint8_t mk = mr ? mr[k] : 0;
    return replace ? masked_score<true>(xv, scale, mk)
                   : masked_score<false>(xv, scale, mk);
  };
  float m = -INFINITY;
  for (int k = lane; k < Sk; k += kWave) m = fmaxf(m, score(k));
  m = wave_allreduce(m, OpMax());
  float sum = 0.f;
  for (int k = lane; k < Sk; k += kWave) sum += exp_shifted(score(k), m);
  sum = wave_allreduce(sum, OpAdd());
  const float inv = 1.0f / sum;
  for (int k = lane; k < Sk; k += kWave)
    yr[k] = static_cast<T>(exp_shifted(score(k), m) * inv);
}

template <typename T>
__global__ __launch_bounds__(kBlockThreads) void masked_bwd_anyshape_kernel(
    T *dx, const T *g, const T *y, float scale, int Sk, int64_t total_rows) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t row = (int64_t)blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
  if (row >= total_rows) return;
  const T *gr = g + row * Sk;
  const T *yr = y + row * Sk;
  T *dr = dx + row * Sk;
  float sum = 0.f;
  for (int k = lane; k < Sk; k += kWave)
    sum += static_cast<float>(gr[k]) * static_cast<float>(yr[k]);
  sum = wave_allreduce(sum, OpAdd());
  for (int k = lane; k < Sk; k += kWave) {
    const float yk = static_cast<float>(yr[k]);
    dr[k] = static_cast<T>(scale * (static_cast<float>(gr[k]) * yk - yk * sum));
  }
}

template <typename T>
int launch_masked_fwd(T *y, const T *x, const uint8_t *mask, int64_t msb,
                      int64_t msq, bool replace, float scale, int64_t B,
                      int64_t H, int64_t Sq, int64_t Sk, hipStream_t stream) {
  constexpr int VEC = Io<T>::kVec;
  const int64_t total_rows = B * H * Sq;
  // mask vectors are VEC bytes wide: every row start must be VEC-aligned
  const bool mask_ok =
      mask == nullptr || ((reinterpret_cast<uintptr_t>(mask) % VEC) == 0 &&
                          msb % VEC == 0 && msq % VEC == 0);
  const bool vector_ok =
      Sk % VEC == 0 && aligned16(x) && aligned16(y) && mask_ok;
  if (!vector_ok) {
    const int64_t blocks = (total_rows + kWavesPerBlock - 1) / kWavesPerBlock;
    masked_fwd_anyshape_kernel<T>
        <<<dim3((unsigned)blocks), dim3(kBlockThreads), 0, stream>>>(
            y, x, mask, msb, msq, replace ? 1 : 0, scale, (int)Sq, (int)Sk,
            (int)H, total_rows);
    return check_launch("softmax_masked_fwd");
  }
  dispatch_row_tile<VEC>(Sk, [&]<int NCHUNK, int WPR>() {
    constexpr int rpb = RowTile<VEC, NCHUNK, WPR>::kRowsPerBlock;
    const RowMap map = make_row_map(total_rows, rpb, Sk * (int64_t)sizeof(T), false);
    const dim3 grid((unsigned)(map.blocks_per_xcd * kXcds));
    const dim3 block(kBlockThreads);
    const unsigned lds = occupancy_pad_bytes(false, Sk * (int64_t)sizeof(T));
    if (!mask)
      masked_fwd_kernel<T, VEC, NCHUNK, WPR, false, false>
          <<<grid, block, lds, stream>>>(y, x, nullptr, 0, 0, scale, (int)Sq,
                                         (int)Sk, (int)H, map);
    else if (replace)
      masked_fwd_kernel<T, VEC, NCHUNK, WPR, true, true>
          <<<grid, block, lds, stream>>>(y, x, mask, msb, msq, scale, (int)Sq,
                                         (int)Sk, (int)H, map);
    else
      masked_fwd_kernel<T, VEC, NCHUNK, WPR, true, false>
          <<<grid, block, lds, stream>>>(y, x, mask, msb, msq, scale, (int)Sq,
                                         (int)Sk, (int)H, map);
  });
  return check_launch("softmax_masked_fwd");
}

template <typename T>
int launch_masked_bwd(T *dx, const T *g, const T *y, float scale, int64_t rows,
                      int64_t Sk, hipStream_t stream) {
  constexpr int VEC = Io<T>::kVec;
  const bool vector_ok =
      Sk % VEC == 0 && aligned16(dx) && aligned16(g) && aligned16(y);
  if (!vector_ok) {
    const int64_t blocks = (rows + kWavesPerBlock - 1) / kWavesPerBlock;
    masked_bwd_anyshape_kernel<T><<<dim3((unsigned)blocks), dim3(kBlockThreads),
                                    0, stream>>>(dx, g, y, scale, (int)Sk, rows);
    return check_launch("softmax_masked_bwd");
  }
  dispatch_row_tile<VEC>(Sk, [&]<int NCHUNK, int WPR>() {
    constexpr int rpb = RowTile<VEC, NCHUNK, WPR>::kRowsPerBlock;
    const RowMap map = make_row_map(rows, rpb, Sk * (int64_t)sizeof(T), false);
    masked_bwd_kernel<T, VEC, NCHUNK, WPR>
        <<<dim3((unsigned)(map.blocks_per_xcd * kXcds)), dim3(kBlockThreads),
           occupancy_pad_bytes(true, Sk * (int64_t)sizeof(T)), stream>>>(
            dx, g, y, scale, (int)Sk, map);
  });
  return check_launch("softmax_masked_bwd");
}

int screen(const char *name, int64_t rows, int64_t Sk) {
  if (rows < 0 || Sk < 0)
    return fail(OSLO_E_BAD_ARG, "%s: negative size", name);
  if (Sk > kSoftmaxMaxCols)
    return fail(OSLO_E_UNSUPPORTED, "%s: row length %lld exceeds %d", name,
                (long long)Sk, kSoftmaxMaxCols);
  if (rows > INT32_MAX)
    return fail(OSLO_E_UNSUPPORTED, "%s: too many rows for one launch", name);
  return (rows == 0 || Sk == 0) ? 1 : 0;
}

} // namespace
} // namespace oslo

extern "C" int oslo_softmax_masked_fwd(void *y, const void *x,
                                       const uint8_t *mask,
                                       int64_t mask_stride_b,
                                       int64_t mask_stride_q, int mask_mode,
                                       float scale, int64_t B, int64_t H,
                                       int64_t Sq, int64_t Sk, int dtype,
                                       oslo_stream_t stream) {
  using namespace oslo;
  if (B < 0 || H < 0 || Sq < 0)
    return fail(OSLO_E_BAD_ARG, "softmax_masked_fwd: negative size");
  if (mask_mode != OSLO_MASK_ADD && mask_mode != OSLO_MASK_REPLACE)
    return fail(OSLO_E_BAD_ARG, "softmax_masked_fwd: unknown mask_mode %d",
                mask_mode);
  if (mask && (mask_stride_b < 0 || mask_stride_q < 0))
    return fail(OSLO_E_BAD_ARG, "softmax_masked_fwd: negative mask stride");
  if (H > 0 && Sq > 0 && B > INT32_MAX / H / Sq)
    return fail(OSLO_E_UNSUPPORTED,
                "softmax_masked_fwd: too many rows for one launch");
  const int s = screen("softmax_masked_fwd", B * H * Sq, Sk);
  if (s != 0) return s < 0 ? s : OSLO_OK;
  if (!x || !y) return fail(OSLO_E_BAD_ARG, "softmax_masked_fwd: null tensor");
  OSLO_DISPATCH_DTYPE(
      dtype, return launch_masked_fwd<T>(
                 static_cast<T *>(y), static_cast<const T *>(x), mask,
                 mask_stride_b, mask_stride_q, mask_mode == OSLO_MASK_REPLACE,
                 scale, B, H, Sq, Sk, static_cast<hipStream_t>(stream)));
  return OSLO_OK;
}

extern "C" int oslo_softmax_masked_bwd(void *dx, const void *g, const void *y,
                                       float scale, int64_t rows, int64_t Sk,
                                       int dtype, oslo_stream_t stream) {
  using namespace oslo;
  const int s = screen("softmax_masked_bwd", rows, Sk);
  if (s != 0) return s < 0 ? s : OSLO_OK;
  if (!dx || !g || !y)
    return fail(OSLO_E_BAD_ARG, "softmax_masked_bwd: null tensor");
  OSLO_DISPATCH_DTYPE(dtype, return launch_masked_bwd<T>(
                                 static_cast<T *>(dx), static_cast<const T *>(g),
                                 static_cast<const T *>(y), scale, rows, Sk,
                                 static_cast<hipStream_t>(stream)));
  return OSLO_OK;
}
