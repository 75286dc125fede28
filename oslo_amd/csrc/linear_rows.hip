// Linear layer for a handful of input rows: out[m, n] = act(x[m, :] . w[n, :] +
// bias[n]) with 1 <= m <= 8, as in a decoding step, where the projections of a
// transformer block read every weight once for one token per sequence. That is
// a stream over the weight matrix, bound by HBM like the other kernels of this
// library, not a contraction for the matrix cores: the weight bytes are the
// algorithmic bytes.
//
// A wave owns R output features (rows of w, each k contiguous elements) and
// walks along k in chunks of 64 lanes x one 128-bit vector, U chunks (so R*U
// loads per lane) in flight. One or two input rows come through the vector
// cache, which every wave of the CU shares; three to eight are staged in LDS
// by the block, a segment of k at a time, because their loads would otherwise
// queue behind the weight loads of the same wave and there are m of them per
// weight vector. Products accumulate in fp32, pairs of
// 16-bit elements through v_dot2c_f32_{f16,bf16}. The bias and the tanh-form
// GeLU of the feed-forward layer are applied to the fp32 sums before the one
// rounding to the storage type: this is the reference's
//   x = torch.matmul(x, weight.t()); x = FusedBiasActivation.apply(x, bias, act)
// (oslo/models/gptj/modeling_gptj.py:1049-1053) without the rounded
// intermediate. A second kernel at the end of this file takes the weight in
// GPT-2's [k, n] layout.

#include "common.hpp"
#include "gelu.hpp"

namespace oslo {
namespace {

constexpr uint32_t kOutside = 0x80000000u; // past any descriptor used here
constexpr int kMaxRows = 8;
constexpr int kMaxJobs = 3;

// Up to three layers of the same shape applied to the same input in one launch
// (blockIdx.y picks the layer): the query, key and value projections.
template <typename T>
struct LinearJobs {
  T *out[kMaxJobs];
  const T *w[kMaxJobs];
  const T *bias[kMaxJobs];
  const T *residual; // [m, n], added after the activation; for one layer only
};

template <typename T, int VEC>
__device__ __forceinline__ float dot_acc(float acc, const RawVec<T, VEC> &w,
                                         const RawVec<T, VEC> &x) {
  if constexpr (sizeof(T) == 4) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) acc = __builtin_fmaf(w[j], x[j], acc);
  } else {
    struct Pairs {
      RawVec<T, 2> p[VEC / 2];
    };
    const Pairs wp = __builtin_bit_cast(Pairs, w);
    const Pairs xp = __builtin_bit_cast(Pairs, x);
#pragma unroll
    for (int j = 0; j < VEC / 2; ++j) {
      if constexpr (__is_same(T, bf16))
        acc = __builtin_amdgcn_fdot2_f32_bf16(wp.p[j], xp.p[j], acc, false);
      else
        acc = __builtin_amdgcn_fdot2(wp.p[j], xp.p[j], acc, false);
    }
  }
  return acc;
}

// MT: input rows the kernel is compiled for (m <= MT; the rows past m read as
// zeros and are not stored).
template <typename T, int VEC, int MT, int R, int U>
__global__ __launch_bounds__(kBlockThreads) void linear_rows_kernel(
    LinearJobs<T> jobs, const T *__restrict__ x, int m, int64_t n, int64_t k,
    int chunks, int gelu) {
  T *__restrict__ out = jobs.out[blockIdx.y];
  const T *__restrict__ w = jobs.w[blockIdx.y];
  const T *__restrict__ bias = jobs.bias[blockIdx.y];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int64_t row0 = ((int64_t)blockIdx.x * kWavesPerBlock + wave) * R;
  if (row0 >= n) return; // no barrier in this kernel
  const BufRsrc wrs = make_rsrc(w, (uint32_t)(n * k * (int64_t)sizeof(T)));
  const BufRsrc xrs = make_rsrc(x, (uint32_t)((int64_t)m * k * (int64_t)sizeof(T)));
  const uint32_t row_bytes = (uint32_t)(k * (int64_t)sizeof(T));

  float acc[R][MT];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int i = 0; i < MT; ++i) acc[r][i] = 0.f;

  for (int c0 = 0; c0 < chunks; c0 += U) {
    uint32_t col[U]; // byte offset of the lane's vector inside a row
    bool col_ok[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t e = ((int64_t)(c0 + u) * kWave + lane) * VEC;
      col_ok[u] = e < k; // k is a multiple of VEC: a vector is inside or outside
      col[u] = (uint32_t)(e * (int64_t)sizeof(T));
    }
    RawVec<T, VEC> wv[R][U];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const bool ok = col_ok[u] && row0 + r < n;
        wv[r][u] = buffer_load_raw<T, VEC, true>(
            wrs, ok ? (uint32_t)(row0 + r) * row_bytes + col[u] : kOutside);
      }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        const bool ok = col_ok[u] && i < m;
        const RawVec<T, VEC> xv = buffer_load_raw<T, VEC, false>(
            xrs, ok ? (uint32_t)i * row_bytes + col[u] : kOutside);
#pragma unroll
        for (int r = 0; r < R; ++r)
          acc[r][i] = dot_acc<T, VEC>(acc[r][i], wv[r][u], xv);
      }
  }

#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int i = 0; i < MT; ++i) acc[r][i] = wave_allreduce(acc[r][i], OpAdd());
  if (lane == 0) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      if (row0 + r >= n) break;
      const float b = bias != nullptr ? static_cast<float>(bias[row0 + r]) : 0.f;
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        if (i >= m) break;
        float v = acc[r][i] + b;
        if (gelu) v = gelu_fwd(v);
        const int64_t at = (int64_t)i * n + row0 + r;
        if (jobs.residual != nullptr) v += static_cast<float>(jobs.residual[at]);
        out[at] = static_cast<T>(v);
      }
    }
  }
}

// The same with the input rows in LDS. The block stages a segment of
// kSegBytes / MT bytes of each of the MT rows (so 32 KiB in all), its eight
// waves walk their weight rows over that segment, and so on along k. Rows past
// m and vectors past k are staged as zeros. Every wave stays to the end: there
// are barriers in the loop. EARLY: the first weight loads of a segment go out
// before its staging and barriers (the launcher says per tile where that paid).
constexpr int kSegBytes = 32768;
constexpr int kLdsThreads = 512; // 8 waves share one staged segment

template <typename T, int VEC, int MT, int R, int U, bool EARLY, int THREADS, int SEGBYTES>
__global__ __launch_bounds__(THREADS) void linear_rows_lds_kernel(
    LinearJobs<T> jobs, const T *__restrict__ x, int m, int64_t n, int64_t k,
    int gelu) {
  T *__restrict__ out = jobs.out[blockIdx.y];
  const T *__restrict__ w = jobs.w[blockIdx.y];
  const T *__restrict__ bias = jobs.bias[blockIdx.y];
  using Vec = RawVec<T, VEC>;
  constexpr int kSegVecs = SEGBYTES / 16 / MT;  // vectors of one row per segment
  constexpr int kSegChunks = kSegVecs / kWave;   // chunks of 64 vectors
  static_assert(kSegChunks % U == 0, "a segment is whole unrolled spans");
  __shared__ Vec xs[MT * kSegVecs];

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int64_t row0 = ((int64_t)blockIdx.x * (THREADS / kWave) + wave) * R;
  const BufRsrc wrs = make_rsrc(w, (uint32_t)(n * k * (int64_t)sizeof(T)));
  const BufRsrc xrs = make_rsrc(x, (uint32_t)((int64_t)m * k * (int64_t)sizeof(T)));
  const uint32_t row_bytes = (uint32_t)(k * (int64_t)sizeof(T));
  const int kvec = (int)(k / VEC); // vectors per row

  float acc[R][MT];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int i = 0; i < MT; ++i) acc[r][i] = 0.f;

  // the weight vectors of U chunks starting at chunk c0 of the segment at v0
  auto load_weights = [&](Vec (&wv)[R][U], int v0, int c0) {
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int v = v0 + (c0 + u) * kWave + lane;
        const bool ok = v < kvec && row0 + r < n;
        wv[r][u] = buffer_load_raw<T, VEC, true>(
            wrs, ok ? (uint32_t)(row0 + r) * row_bytes + (uint32_t)v * 16u : kOutside);
      }
  };

  for (int v0 = 0; v0 < kvec; v0 += kSegVecs) {
    // The loads of the segment's inputs go out first and the first weight loads
    // right behind them, before any barrier: loads return in order, so the
    // wait for the inputs leaves the weight loads, whose latency is the long
    // one, in flight across the staging.
    constexpr int kPasses = MT * kSegVecs / THREADS;
    Vec stage[kPasses];
#pragma unroll
    for (int p = 0; p < kPasses; ++p) {
      const int idx = p * THREADS + threadIdx.x;
      const int i = idx / kSegVecs, v = v0 + idx % kSegVecs;
      const bool ok = i < m && v < kvec;
      stage[p] = buffer_load_raw<T, VEC, false>(
          xrs, ok ? (uint32_t)i * row_bytes + (uint32_t)v * 16u : kOutside);
    }
    Vec wv[R][U];
    if constexpr (EARLY) load_weights(wv, v0, 0);
    if (v0 > 0) __syncthreads(); // the previous segment has been read
#pragma unroll
    for (int p = 0; p < kPasses; ++p) xs[p * THREADS + threadIdx.x] = stage[p];
    __syncthreads();

#pragma unroll 1
    for (int c0 = 0; c0 < kSegChunks; c0 += U) {
      if (!EARLY || c0 > 0) load_weights(wv, v0, c0);
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int i = 0; i < MT; ++i) {
          const Vec xv = xs[i * kSegVecs + (c0 + u) * kWave + lane];
#pragma unroll
          for (int r = 0; r < R; ++r)
            acc[r][i] = dot_acc<T, VEC>(acc[r][i], wv[r][u], xv);
        }
    }
  }

#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int i = 0; i < MT; ++i) acc[r][i] = wave_allreduce(acc[r][i], OpAdd());
  if (lane == 0) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      if (row0 + r >= n) break;
      const float b = bias != nullptr ? static_cast<float>(bias[row0 + r]) : 0.f;
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        if (i >= m) break;
        float v = acc[r][i] + b;
        if (gelu) v = gelu_fwd(v);
        const int64_t at = (int64_t)i * n + row0 + r;
        if (jobs.residual != nullptr) v += static_cast<float>(jobs.residual[at]);
        out[at] = static_cast<T>(v);
      }
    }
  }
}

template <typename T>
LinearJobs<T> make_jobs(void *const *out, const void *const *w,
                        const void *const *bias, const void *residual,
                        int count) {
  LinearJobs<T> jobs;
  for (int j = 0; j < kMaxJobs; ++j) {
    const int s = j < count ? j : 0;
    jobs.out[j] = static_cast<T *>(out[s]);
    jobs.w[j] = static_cast<const T *>(w[s]);
    jobs.bias[j] = bias ? static_cast<const T *>(bias[s]) : nullptr;
  }
  jobs.residual = static_cast<const T *>(residual);
  return jobs;
}

template <typename T, int MT, int R, int U, bool EARLY = true, int THREADS = kLdsThreads, int SEGBYTES = kSegBytes>
int launch_lds(const LinearJobs<T> &jobs, int count, const void *x, int m,
               int64_t n, int64_t k, int gelu, hipStream_t stream) {
  constexpr int VEC = Io<T>::kVec;
  const int64_t rows_per_block = (int64_t)(THREADS / kWave) * R;
  const int64_t blocks = (n + rows_per_block - 1) / rows_per_block;
  linear_rows_lds_kernel<T, VEC, MT, R, U, EARLY, THREADS, SEGBYTES>
      <<<dim3((unsigned)blocks, count), dim3(THREADS), 0, stream>>>(
          jobs, static_cast<const T *>(x), m, n, k, gelu);
  return check_launch("oslo_linear_rows_fwd");
}

template <typename T, int MT, int R, int U>
int launch(const LinearJobs<T> &jobs, int count, const void *x, int m, int64_t n,
           int64_t k, int gelu, hipStream_t stream) {
  constexpr int VEC = Io<T>::kVec;
  const int chunks = (int)((k + (int64_t)kWave * VEC - 1) / ((int64_t)kWave * VEC));
  const int64_t rows_per_block = (int64_t)kWavesPerBlock * R;
  const int64_t blocks = (n + rows_per_block - 1) / rows_per_block;
  linear_rows_kernel<T, VEC, MT, R, U>
      <<<dim3((unsigned)blocks, count), dim3(kBlockThreads), 0, stream>>>(
          jobs, static_cast<const T *>(x), m, n, k, chunks, gelu);
  return check_launch("oslo_linear_rows_fwd");
}

int linear_rows(void *const *out, const void *x, const void *const *weight,
                const void *const *bias, const void *residual, int count,
                int64_t m, int64_t n, int64_t k, int epilogue, int dtype,
                hipStream_t s) {
  if (m < 0 || n < 0 || k < 0)
    return fail(OSLO_E_BAD_ARG, "oslo_linear_rows_fwd: negative size");
  if (epilogue != OSLO_EPILOGUE_NONE && epilogue != OSLO_EPILOGUE_GELU_TANH)
    return fail(OSLO_E_BAD_ARG, "oslo_linear_rows_fwd: unknown epilogue %d", epilogue);
  if (dtype != OSLO_F32 && dtype != OSLO_F16 && dtype != OSLO_BF16)
    return fail(OSLO_E_BAD_ARG, "unknown dtype %d", dtype);
  if (m > kMaxRows)
    return fail(OSLO_E_UNSUPPORTED,
                "oslo_linear_rows_fwd: %lld input rows, at most %d (use a GEMM)",
                (long long)m, kMaxRows);
  if (m == 0 || n == 0) return OSLO_OK;
  if (!x) return fail(OSLO_E_BAD_ARG, "oslo_linear_rows_fwd: null pointer");
  const int64_t es = dtype == OSLO_F32 ? 4 : 2;
  if (k == 0 || (k * es) % 16 != 0)
    return fail(OSLO_E_UNSUPPORTED,
                "oslo_linear_rows_fwd: rows of %lld elements are not whole 16-byte vectors",
                (long long)k);
  if (n > (int64_t)0x7fffffff / (k * es) || m > (int64_t)0x7fffffff / (k * es))
    return fail(OSLO_E_UNSUPPORTED,
                "oslo_linear_rows_fwd: weight of 2 GiB or more (32-bit offsets)");
  if (!aligned16(x))
    return fail(OSLO_E_BAD_ARG, "oslo_linear_rows_fwd: x and weight must be 16-byte aligned");
  for (int j = 0; j < count; ++j) {
    if (!out[j] || !weight[j])
      return fail(OSLO_E_BAD_ARG, "oslo_linear_rows_fwd: null pointer");
    if (!aligned16(weight[j]))
      return fail(OSLO_E_BAD_ARG, "oslo_linear_rows_fwd: x and weight must be 16-byte aligned");
    if (out[j] == x || out[j] == weight[j])
      return fail(OSLO_E_BAD_ARG, "oslo_linear_rows_fwd: out must not alias an input");
    for (int i = 0; i < j; ++i)
      if (out[i] == out[j])
        return fail(OSLO_E_BAD_ARG, "oslo_linear_rows_fwd: two layers share an output");
  }
  const int gelu = epilogue == OSLO_EPILOGUE_GELU_TANH;
  const int mi = (int)m;
  OSLO_DISPATCH_DTYPE(dtype, {
    const LinearJobs<T> jobs = make_jobs<T>(out, weight, bias, residual, count);
    if (mi == 1) return launch<T, 1, 1, 8>(jobs, count, x, mi, n, k, gelu, s);
    if (mi == 2) return launch<T, 2, 1, 8>(jobs, count, x, mi, n, k, gelu, s);
    // two weight rows per wave halve the LDS reads per weight byte, but leave
    // too few blocks when there are few output features
    const bool few = n * count < 8192;
    if (mi <= 4)
      return few ? launch_lds<T, 4, 1, 8>(jobs, count, x, mi, n, k, gelu, s)
                 : launch_lds<T, 4, 2, 4>(jobs, count, x, mi, n, k, gelu, s);
    // (with 8 input rows and two weight rows per wave the early weight loads
    // measured 6-11 % slower than loading inside the loop: that one keeps them there)
    return few ? launch_lds<T, 8, 1, 4>(jobs, count, x, mi, n, k, gelu, s)
               : launch_lds<T, 8, 2, 4, false>(jobs, count, x, mi, n, k, gelu, s);
  });
  return OSLO_OK;
}

// The same layer with the weight stored [k, n] (in_features major), the layout
// of GPT-2's Conv1D: out[i, j] = sum_c x[i, c] * w[c, j]. Here a row of w holds
// one input feature for all outputs, so the lanes go along j: a block owns a
// strip of 4 lanes x one vector of output features (64 bytes of every weight
// row; narrow, because these matrices have few output features and every strip
// is a block) and its 16 waves share the k rows. A wave-wide load covers 16
// rows of the strip; a lane takes VEC consecutive rows per step, so that its
// inputs x[i, c..c+VEC) are one vector load per input row. The 16 row groups
// of a wave are the 16 lanes of a DPP row (lane % 16), so that their sums meet
// by DPP in the vector ALU; the 16 waves then meet in LDS.
// These matrices are small (a few MB): the launch is bound by latency, and one
// block per strip keeps it to a single launch with a fixed summation order.
constexpr int kKnThreads = 1024;
constexpr int kKnWaves = kKnThreads / kWave;
constexpr int kStripLanes = 4; // lanes along the output features

template <typename T, int VEC, int MT>
__global__ __launch_bounds__(kKnThreads) void linear_rows_kn_kernel(
    T *__restrict__ out, const T *__restrict__ x, const T *__restrict__ w,
    const T *__restrict__ bias, const T *residual, int m, int64_t n, int64_t k,
    int gelu) {
  constexpr int kRowGroups = kWave / kStripLanes; // 16 rows per load instruction
  constexpr int kStrip = kStripLanes * VEC;       // output features per block
  __shared__ float red[kKnWaves][MT][kStrip];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int group = lane % kRowGroups, cl = lane / kRowGroups; // rows by lane % 16, features by lane / 16
  const int64_t col = (int64_t)blockIdx.x * kStrip + cl * VEC;
  const bool col_ok = col < n; // n is a multiple of VEC
  const BufRsrc wrs = make_rsrc(w, (uint32_t)(n * k * (int64_t)sizeof(T)));
  const BufRsrc xrs = make_rsrc(x, (uint32_t)((int64_t)m * k * (int64_t)sizeof(T)));
  const uint32_t wrow_bytes = (uint32_t)(n * (int64_t)sizeof(T));
  const uint32_t xrow_bytes = (uint32_t)(k * (int64_t)sizeof(T));

  float acc[MT][VEC];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < VEC; ++j) acc[i][j] = 0.f;

  constexpr int kRowsPerWave = kRowGroups * VEC; // rows of one wave per step
  for (int64_t k0 = (int64_t)wave * kRowsPerWave; k0 < k; k0 += (int64_t)kKnWaves * kRowsPerWave) {
    const int64_t row = k0 + group * VEC; // the lane's VEC consecutive rows (k is a multiple of VEC)
    const bool row_ok = row < k;
    RawVec<T, VEC> wv[VEC];
#pragma unroll
    for (int u = 0; u < VEC; ++u)
      wv[u] = buffer_load_raw<T, VEC, true>(
          wrs, row_ok && col_ok ? (uint32_t)(row + u) * wrow_bytes + (uint32_t)col * (uint32_t)sizeof(T) : kOutside);
    RawVec<T, VEC> xv[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i)
      xv[i] = buffer_load_raw<T, VEC, false>(
          xrs, row_ok && i < m ? (uint32_t)i * xrow_bytes + (uint32_t)row * (uint32_t)sizeof(T) : kOutside);
#pragma unroll
    for (int u = 0; u < VEC; ++u) {
      float wf[VEC];
      raw_to_f32<T, VEC>(wf, wv[u]);
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        const float xi = static_cast<float>(xv[i][u]);
#pragma unroll
        for (int j = 0; j < VEC; ++j) acc[i][j] = __builtin_fmaf(xi, wf[j], acc[i][j]);
      }
    }
  }

  // the 16 row groups of the wave, then the 16 waves
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      static_assert(kRowGroups == 16, "the row groups are the 16 lanes of a DPP row");
      acc[i][j] = sum_over_row(acc[i][j]);
    }
  if (group == 0) {
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int j = 0; j < VEC; ++j) red[wave][i][cl * VEC + j] = acc[i][j];
  }
  __syncthreads();
  for (int t = threadIdx.x; t < m * kStrip; t += kKnThreads) {
    const int i = t / kStrip, c = t % kStrip;
    const int64_t j = (int64_t)blockIdx.x * kStrip + c;
    if (j >= n) continue;
    float v = 0.f;
#pragma unroll
    for (int wv_ = 0; wv_ < kKnWaves; ++wv_) v += red[wv_][i][c];
    if (bias != nullptr) v += static_cast<float>(bias[j]);
    if (gelu) v = gelu_fwd(v);
    if (residual != nullptr) v += static_cast<float>(residual[(int64_t)i * n + j]);
    out[(int64_t)i * n + j] = static_cast<T>(v);
  }
}

template <typename T, int MT>
int launch_kn(void *out, const void *x, const void *w, const void *bias,
              const void *residual, int m, int64_t n, int64_t k, int gelu,
              hipStream_t stream) {
  constexpr int VEC = Io<T>::kVec;
  constexpr int kStrip = kStripLanes * VEC;
  const int64_t blocks = (n + kStrip - 1) / kStrip;
  linear_rows_kn_kernel<T, VEC, MT>
      <<<dim3((unsigned)blocks), dim3(kKnThreads), 0, stream>>>(
          static_cast<T *>(out), static_cast<const T *>(x),
          static_cast<const T *>(w), static_cast<const T *>(bias),
          static_cast<const T *>(residual), m, n, k, gelu);
  return check_launch("oslo_linear_rows_kn_fwd");
}

} // namespace
} // namespace oslo

extern "C" int oslo_linear_rows_kn_fwd(void *out, const void *x, const void *weight,
                                       const void *bias, const void *residual,
                                       int64_t m, int64_t n, int64_t k,
                                       int epilogue, int dtype,
                                       oslo_stream_t stream) {
  using namespace oslo;
  if (m < 0 || n < 0 || k < 0)
    return fail(OSLO_E_BAD_ARG, "oslo_linear_rows_kn_fwd: negative size");
  if (epilogue != OSLO_EPILOGUE_NONE && epilogue != OSLO_EPILOGUE_GELU_TANH)
    return fail(OSLO_E_BAD_ARG, "oslo_linear_rows_kn_fwd: unknown epilogue %d", epilogue);
  if (dtype != OSLO_F32 && dtype != OSLO_F16 && dtype != OSLO_BF16)
    return fail(OSLO_E_BAD_ARG, "unknown dtype %d", dtype);
  if (m > kMaxRows)
    return fail(OSLO_E_UNSUPPORTED,
                "oslo_linear_rows_kn_fwd: %lld input rows, at most %d (use a GEMM)",
                (long long)m, kMaxRows);
  if (m == 0 || n == 0) return OSLO_OK;
  if (!out || !x || !weight)
    return fail(OSLO_E_BAD_ARG, "oslo_linear_rows_kn_fwd: null pointer");
  const int64_t es = dtype == OSLO_F32 ? 4 : 2;
  if (k == 0 || (k * es) % 16 != 0 || (n * es) % 16 != 0)
    return fail(OSLO_E_UNSUPPORTED,
                "oslo_linear_rows_kn_fwd: %lld x %lld: rows of x and of the weight must be whole 16-byte vectors",
                (long long)k, (long long)n);
  if (!aligned16(x) || !aligned16(weight))
    return fail(OSLO_E_BAD_ARG, "oslo_linear_rows_kn_fwd: x and weight must be 16-byte aligned");
  if (n > (int64_t)0x7fffffff / (k * es) || m > (int64_t)0x7fffffff / (k * es))
    return fail(OSLO_E_UNSUPPORTED,
                "oslo_linear_rows_kn_fwd: weight of 2 GiB or more (32-bit offsets)");
  if (out == x || out == weight)
    return fail(OSLO_E_BAD_ARG, "oslo_linear_rows_kn_fwd: out must not alias an input");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int gelu = epilogue == OSLO_EPILOGUE_GELU_TANH;
  const int mi = (int)m;
  OSLO_DISPATCH_DTYPE(dtype, {
    // compiled for the exact row count: a block does all the arithmetic of its
    // strip, and rows padded up to a power of two showed in the time
    switch (mi) {
    case 1: return launch_kn<T, 1>(out, x, weight, bias, residual, mi, n, k, gelu, s);
    case 2: return launch_kn<T, 2>(out, x, weight, bias, residual, mi, n, k, gelu, s);
    case 3: return launch_kn<T, 3>(out, x, weight, bias, residual, mi, n, k, gelu, s);
    case 4: return launch_kn<T, 4>(out, x, weight, bias, residual, mi, n, k, gelu, s);
    case 5: return launch_kn<T, 5>(out, x, weight, bias, residual, mi, n, k, gelu, s);
    case 6: return launch_kn<T, 6>(out, x, weight, bias, residual, mi, n, k, gelu, s);
    case 7: return launch_kn<T, 7>(out, x, weight, bias, residual, mi, n, k, gelu, s);
    default: return launch_kn<T, 8>(out, x, weight, bias, residual, mi, n, k, gelu, s);
    }
  });
  return OSLO_OK;
}

extern "C" int oslo_linear_rows_max(void) { return oslo::kMaxRows; }

extern "C" int oslo_linear_rows_fwd(void *out, const void *x, const void *weight,
                                    const void *bias, const void *residual,
                                    int64_t m, int64_t n, int64_t k, int epilogue,
                                    int dtype, oslo_stream_t stream) {
  void *const outs[1] = {out};
  const void *const weights[1] = {weight};
  const void *const biases[1] = {bias};
  return oslo::linear_rows(outs, x, weights, biases, residual, 1, m, n, k,
                           epilogue, dtype, static_cast<hipStream_t>(stream));
}

extern "C" int oslo_linear_rows_fwd_multi(void *const *out, const void *x,
                                          const void *const *weight,
                                          const void *const *bias, int count,
                                          int64_t m, int64_t n, int64_t k,
                                          int epilogue, int dtype,
                                          oslo_stream_t stream) {
  if (count < 1 || count > oslo::kMaxJobs)
    return oslo::fail(OSLO_E_BAD_ARG, "oslo_linear_rows_fwd_multi: %d layers, 1 to %d are taken",
                      count, oslo::kMaxJobs);
  if (!out || !weight)
    return oslo::fail(OSLO_E_BAD_ARG, "oslo_linear_rows_fwd_multi: null pointer table");
  return oslo::linear_rows(out, x, weight, bias, nullptr, count, m, n, k, epilogue,
                           dtype, static_cast<hipStream_t>(stream));
}
