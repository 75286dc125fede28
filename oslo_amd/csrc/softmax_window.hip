// Scale + sliding-window causal mask + softmax, forward and backward, for
// gfx950: row r sees keys max(0, r-window+1) .. r, the rest of the output row
// is zero. This is the mask of GPT-Neo's "local" attention layers
// (oslo/models/gpt_neo/modeling_gpt_neo.py:153-163: tril(ones) xor
// tril(ones, -window)), which the reference leaves on the unfused path
// (:268-272). A row reads at most `window` keys and writes S, so the kernels
// are close to a fill: lanes outside the window make no memory request, chunks
// outside it are never converted.

#include "softmax.hpp"

namespace oslo {
namespace {

// A byte offset no row reaches (rows are at most 8192 fp32 values): a buffer
// access at it is out of range, the load returns zeros and makes no request.
constexpr uint32_t kOutsideRow = 0x40000000u;

template <typename T, int VEC, int NCHUNK, int WPR, bool HAS_PAD>
__global__ __launch_bounds__(kBlockThreads) void window_fwd_kernel(
    T *y, const T *x, const float *__restrict__ pad, float scale, int window,
    int S, int heads, RowMap map) {
  using Tile = RowTile<VEC, NCHUNK, WPR>;
  __shared__ float s_max[kWavesPerBlock];
  __shared__ float s_sum[kWavesPerBlock];

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int sub = wave % WPR;
  int64_t row = mapped_row(map, Tile::kRowsPerBlock, wave / WPR);
  const bool live = row < map.total_rows;
  if (!live) row = map.total_rows - 1;
  const int64_t slab = row / S;
  const int r = (int)(row - slab * S);
  const int lo = max(r - window + 1, 0);
  const T *xr = x + row * S;
  T *yr = y + row * S;

  // all loads first; a lane wholly outside [lo, r] asks for nothing
  const BufRsrc xrs = make_rsrc(xr, (uint32_t)S * (uint32_t)sizeof(T));
  const BufRsrc prs = make_rsrc(HAS_PAD ? pad + (slab / heads) * S : nullptr,
                                HAS_PAD ? (uint32_t)S * (uint32_t)sizeof(float) : 0u);
  RawVec<T, VEC> raw[NCHUNK];
  RawVec<float, VEC> praw[HAS_PAD ? NCHUNK : 1];
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    const int k0 = Tile::col(c, sub, lane);
    const bool outside = k0 > r || k0 + VEC - 1 < lo;
    raw[c] = buffer_load_raw<T, VEC, true>(
        xrs, outside ? kOutsideRow : (uint32_t)k0 * (uint32_t)sizeof(T));
    if constexpr (HAS_PAD)
      praw[c] = buffer_load_raw<float, VEC, false>(
          prs, outside ? kOutsideRow : (uint32_t)k0 * (uint32_t)sizeof(float));
  }
  // wave-uniform: does chunk c of this wave touch the window at all?
  auto chunk_live = [&](int c) {
    const int first = Tile::col(c, sub, 0);
    return first <= r && first + Tile::kSpan - 1 >= lo;
  };
  // The chunks outside the window, most of the row, are zeros whatever the
  // loads bring: they are stored while the loads are in flight.
  const BufRsrc yrs = make_rsrc(yr, live ? (uint32_t)S * (uint32_t)sizeof(T) : 0u);
  {
    float zero[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) zero[j] = 0.f;
#pragma unroll
    for (int c = 0; c < NCHUNK; ++c)
      if (!chunk_live(c))
        buffer_store_f32<T, VEC, kStreamOut>(
            yrs, (uint32_t)Tile::col(c, sub, lane) * (uint32_t)sizeof(T), zero);
  }
  pin_loaded(raw);
  if constexpr (HAS_PAD) pin_loaded(praw);

  // the arithmetic of the causal kernel: log2 units unless a mask is added
  constexpr bool kLog2 = !HAS_PAD;
  const float sc = kLog2 ? scale * kLog2e : scale;
  float v[NCHUNK][VEC];
  float m = -INFINITY;
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    if (!chunk_live(c)) continue;
    const int k0 = Tile::col(c, sub, lane);
    float t[VEC], pv[VEC];
    raw_to_f32<T, VEC>(t, raw[c]);
    if constexpr (HAS_PAD) raw_to_f32<float, VEC>(pv, praw[c]);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      float e = __fmul_rn(t[j], sc);
      if constexpr (HAS_PAD) e = __fadd_rn(e, pv[j]);
      const int k = k0 + j;
      v[c][j] = (k >= lo && k <= r) ? e : -INFINITY;
      m = fmaxf(m, v[c][j]);
    }
  }
  m = row_allreduce<WPR>(m, OpMax(), s_max);

  float sum = 0.f;
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    if (chunk_live(c)) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        v[c][j] = kLog2 ? __builtin_amdgcn_exp2f(v[c][j] - m) : exp_shifted(v[c][j], m);
        sum += v[c][j];
      }
    }
  }
  sum = row_allreduce<WPR>(sum, OpAdd(), s_sum);
  const float inv = 1.0f / sum;

  // a row slot past the end has an empty descriptor: its stores are dropped
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    if (!chunk_live(c)) continue;
    float o[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) o[j] = v[c][j] * inv;
    buffer_store_f32<T, VEC, kStreamOut>(
        yrs, (uint32_t)Tile::col(c, sub, lane) * (uint32_t)sizeof(T), o);
  }
}

template <typename T, int VEC, int NCHUNK, int WPR>
__global__ __launch_bounds__(kBlockThreads) void window_bwd_kernel(
    T *dx, const T *g, const T *y, float scale, int window, int S, RowMap map) {
  using Tile = RowTile<VEC, NCHUNK, WPR>;
  __shared__ float s_sum[kWavesPerBlock];

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int sub = wave % WPR;
  int64_t row = mapped_row(map, Tile::kRowsPerBlock, wave / WPR);
  const bool live = row < map.total_rows;
  if (!live) row = map.total_rows - 1;
  const int r = (int)(row % S);
  const int lo = max(r - window + 1, 0);

  const uint32_t bytes = (uint32_t)S * (uint32_t)sizeof(T);
  const BufRsrc grs = make_rsrc(g + row * S, bytes);
  const BufRsrc yrs = make_rsrc(y + row * S, bytes);
  RawVec<T, VEC> graw[NCHUNK], yraw[NCHUNK];
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    const int k0 = Tile::col(c, sub, lane);
    const bool outside = k0 > r || k0 + VEC - 1 < lo;
    const uint32_t off = outside ? kOutsideRow : (uint32_t)k0 * (uint32_t)sizeof(T);
    graw[c] = buffer_load_raw<T, VEC, true>(grs, off);
    yraw[c] = buffer_load_raw<T, VEC, true>(yrs, off);
  }
  auto chunk_live = [&](int c) { // wave-uniform
    const int first = Tile::col(c, sub, 0);
    return first <= r && first + Tile::kSpan - 1 >= lo;
  };
  // zeros outside the window go out while the loads are in flight (dx may be g:
  // nothing outside the window is read)
  const BufRsrc drs = make_rsrc(dx + row * S, live ? bytes : 0u);
  {
    float zero[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) zero[j] = 0.f;
#pragma unroll
    for (int c = 0; c < NCHUNK; ++c)
      if (!chunk_live(c))
        buffer_store_f32<T, VEC, kStreamOut>(
            drs, (uint32_t)Tile::col(c, sub, lane) * (uint32_t)sizeof(T), zero);
  }
  pin_loaded(graw);
  pin_loaded(yraw);

  // Only the raw registers are kept across the reduction: a window covers one
  // or two chunks of a row, and converting those twice costs less than fp32
  // copies of the whole row would cost in occupancy.
  auto products = [&](int c, float (&gy)[VEC], float (&yy)[VEC]) {
    const int k0 = Tile::col(c, sub, lane);
    float tg[VEC];
    raw_to_f32<T, VEC>(tg, graw[c]);
    raw_to_f32<T, VEC>(yy, yraw[c]);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const int k = k0 + j;
      // entries outside the window are never used, whatever they hold
      if (k < lo || k > r) yy[j] = tg[j] = 0.f;
      gy[j] = tg[j] * yy[j];
    }
  };
  float sum = 0.f;
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    if (!chunk_live(c)) continue;
    float gy[VEC], yy[VEC];
    products(c, gy, yy);
#pragma unroll
    for (int j = 0; j < VEC; ++j) sum += gy[j];
  }
  sum = row_allreduce<WPR>(sum, OpAdd(), s_sum);

#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    if (!chunk_live(c)) continue;
    float o[VEC], gy[VEC], yy[VEC];
    products(c, gy, yy);
#pragma unroll
    for (int j = 0; j < VEC; ++j) o[j] = scale * (gy[j] - yy[j] * sum);
    buffer_store_f32<T, VEC, kStreamOut>(
        drs, (uint32_t)Tile::col(c, sub, lane) * (uint32_t)sizeof(T), o);
  }
}

// Any-shape path (S not a multiple of the vector, or unaligned pointers): one
// wave per row, element-wise, three passes over the window.
template <typename T>
__global__ __launch_bounds__(kBlockThreads) void window_fwd_anyshape_kernel(
    T *y, const T *x, const float *__restrict__ pad, float scale, int window,
    int S, int heads, int64_t total_rows) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t row = (int64_t)blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
  if (row >= total_rows) return;
  const int64_t slab = row / S;
  const int r = (int)(row - slab * S);
  const int lo = max(r - window + 1, 0);
  const T *xr = x + row * S;
  T *yr = y + row * S;
  const float *padr = pad ? pad + (slab / heads) * S : nullptr;
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
  for (int k = lo + lane; k <= r; k += kWave) m = fmaxf(m, score(k));
  m = wave_allreduce(m, OpMax());
  float sum = 0.f;
  for (int k = lo + lane; k <= r; k += kWave) sum += ex(score(k), m);
  sum = wave_allreduce(sum, OpAdd());
  const float inv = 1.0f / sum;
  // x is read before y is written at the same index, so y may alias x
  for (int k = lane; k < S; k += kWave)
    yr[k] = static_cast<T>((k >= lo && k <= r) ? ex(score(k), m) * inv : 0.f);
}

template <typename T>
__global__ __launch_bounds__(kBlockThreads) void window_bwd_anyshape_kernel(
    T *dx, const T *g, const T *y, float scale, int window, int S,
    int64_t total_rows) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t row = (int64_t)blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
  if (row >= total_rows) return;
  const int r = (int)(row % S);
  const int lo = max(r - window + 1, 0);
  const T *gr = g + row * S;
  const T *yr = y + row * S;
  T *dr = dx + row * S;
  float sum = 0.f;
  for (int k = lo + lane; k <= r; k += kWave)
    sum += static_cast<float>(gr[k]) * static_cast<float>(yr[k]);
  sum = wave_allreduce(sum, OpAdd());
  for (int k = lane; k < S; k += kWave) {
    float o = 0.f;
    if (k >= lo && k <= r) {
      const float yk = static_cast<float>(yr[k]);
      o = scale * (static_cast<float>(gr[k]) * yk - yk * sum);
    }
    dr[k] = static_cast<T>(o);
  }
}

template <typename T>
int launch_window_fwd(T *y, const T *x, const float *pad, float scale, int window,
                      int64_t batch, int64_t heads, int64_t S, hipStream_t stream) {
  constexpr int VEC = Io<T>::kVec;
  const int64_t total_rows = batch * heads * S;
  const bool vector_ok = S % VEC == 0 && aligned16(x) && aligned16(y) &&
                         (pad == nullptr || aligned16(pad));
  if (!vector_ok) {
    const int64_t blocks = (total_rows + kWavesPerBlock - 1) / kWavesPerBlock;
    window_fwd_anyshape_kernel<T><<<dim3((unsigned)blocks), dim3(kBlockThreads), 0, stream>>>(
        y, x, pad, scale, window, (int)S, (int)heads, total_rows);
    return check_launch("softmax_causal_window_fwd");
  }
  dispatch_row_tile<VEC>(S, [&]<int NCHUNK, int WPR>() {
    constexpr int rpb = RowTile<VEC, NCHUNK, WPR>::kRowsPerBlock;
    const RowMap map = make_row_map(total_rows, rpb, S * (int64_t)sizeof(T), false);
    const dim3 grid((unsigned)(map.blocks_per_xcd * kXcds));
    // no occupancy cap: these kernels are fills with a short read in front, and
    // measured best with every wave the registers allow (forward 223 -> 190 us,
    // backward 232 -> 218 us at bf16 [8,16,2048,2048], window 256)
    const unsigned lds = 0;
    if (pad)
      window_fwd_kernel<T, VEC, NCHUNK, WPR, true><<<grid, dim3(kBlockThreads), lds, stream>>>(
          y, x, pad, scale, window, (int)S, (int)heads, map);
    else
      window_fwd_kernel<T, VEC, NCHUNK, WPR, false><<<grid, dim3(kBlockThreads), lds, stream>>>(
          y, x, pad, scale, window, (int)S, (int)heads, map);
  });
  return check_launch("softmax_causal_window_fwd");
}

template <typename T>
int launch_window_bwd(T *dx, const T *g, const T *y, float scale, int window,
                      int64_t bh, int64_t S, hipStream_t stream) {
  constexpr int VEC = Io<T>::kVec;
  const int64_t total_rows = bh * S;
  const bool vector_ok = S % VEC == 0 && aligned16(dx) && aligned16(g) && aligned16(y);
  if (!vector_ok) {
    const int64_t blocks = (total_rows + kWavesPerBlock - 1) / kWavesPerBlock;
    window_bwd_anyshape_kernel<T><<<dim3((unsigned)blocks), dim3(kBlockThreads), 0, stream>>>(
        dx, g, y, scale, window, (int)S, total_rows);
    return check_launch("softmax_causal_window_bwd");
  }
  dispatch_row_tile<VEC>(S, [&]<int NCHUNK, int WPR>() {
    constexpr int rpb = RowTile<VEC, NCHUNK, WPR>::kRowsPerBlock;
    const RowMap map = make_row_map(total_rows, rpb, S * (int64_t)sizeof(T), false);
    const dim3 grid((unsigned)(map.blocks_per_xcd * kXcds));
    const unsigned lds = 0; // as in the forward
    window_bwd_kernel<T, VEC, NCHUNK, WPR><<<grid, dim3(kBlockThreads), lds, stream>>>(
        dx, g, y, scale, window, (int)S, map);
  });
  return check_launch("softmax_causal_window_bwd");
}

int screen_window(const char *name, int64_t window, int64_t rows, int64_t S) {
  if (rows < 0 || S < 0) return fail(OSLO_E_BAD_ARG, "%s: negative size", name);
  if (window < 1) return fail(OSLO_E_BAD_ARG, "%s: window must be at least 1", name);
  if (S > kSoftmaxMaxCols)
    return fail(OSLO_E_UNSUPPORTED, "%s: row length %lld exceeds %d", name, (long long)S,
                kSoftmaxMaxCols);
  if (S > 0 && rows > (int64_t)INT32_MAX / S)
    return fail(OSLO_E_UNSUPPORTED, "%s: too many rows for one launch", name);
  return (rows == 0 || S == 0) ? 1 : 0;
}

} // namespace
} // namespace oslo

extern "C" int oslo_softmax_causal_window_fwd(void *y, const void *x,
                                              const float *pad_add, float scale,
                                              int64_t window, int64_t batch,
                                              int64_t heads, int64_t S, int dtype,
                                              oslo_stream_t stream) {
  using namespace oslo;
  const char *name = "softmax_causal_window_fwd";
  if (batch < 0 || heads < 0) return fail(OSLO_E_BAD_ARG, "%s: negative size", name);
  const int s = screen_window(name, window, batch * heads, S);
  if (s != 0) return s < 0 ? s : OSLO_OK;
  if (window >= S) // the whole lower triangle
    return oslo_softmax_causal_fwd(y, x, pad_add, scale, batch, heads, S, dtype, stream);
  if (!x || !y) return fail(OSLO_E_BAD_ARG, "%s: null tensor", name);
  OSLO_DISPATCH_DTYPE(dtype, return launch_window_fwd<T>(
                                 static_cast<T *>(y), static_cast<const T *>(x), pad_add,
                                 scale, (int)window, batch, heads, S,
                                 static_cast<hipStream_t>(stream)));
  return OSLO_OK;
}

extern "C" int oslo_softmax_causal_window_bwd(void *dx, const void *g, const void *y,
                                              float scale, int64_t window, int64_t bh,
                                              int64_t S, int dtype,
                                              oslo_stream_t stream) {
  using namespace oslo;
  const char *name = "softmax_causal_window_bwd";
  const int s = screen_window(name, window, bh, S);
  if (s != 0) return s < 0 ? s : OSLO_OK;
  if (window >= S) return oslo_softmax_causal_bwd(dx, g, y, scale, bh, S, dtype, stream);
  if (!dx || !g || !y) return fail(OSLO_E_BAD_ARG, "%s: null tensor", name);
  OSLO_DISPATCH_DTYPE(dtype, return launch_window_bwd<T>(
                                 static_cast<T *>(dx), static_cast<const T *>(g),
                                 static_cast<const T *>(y), scale, (int)window, bh, S,
                                 static_cast<hipStream_t>(stream)));
  return OSLO_OK;
}
