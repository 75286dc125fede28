// Attention of a decoding step: one query per sequence and head over a
// key/value cache,
//   out[h, :] = sum_s softmax_s(scale * q[h, :] . K[h, s, :]) * V[h, s, :]
// over the visible keys s (those up to the query's own position, and for a
// sliding window only the last `window` of them). With one query this is two
// matrix-vector products around a softmax: every byte of the visible keys and
// values is read once and nothing else moves, so it is bound by HBM like the
// softmax kernels, and a GEMM library spends three launches and most of its
// time on set-up for it (measured at 16 heads x 1024 keys x 256 features in
// bf16, inside a replayed graph: 24 us for batched matmul, softmax kernel and
// batched matmul, 10 us for the two launches here).
//
// The keys of a (sequence, head) pair are cut into splits of one block, about
// as many as fill the device; a wave takes 16 keys in one shot (2 keys per
// 128-bit load instruction at 512 bytes per key, 8 loads of K and 8 of V in
// flight per lane), computes their scores, the exponentials and the weighted
// sum of their values under a running maximum, tile after tile; the four waves
// of a block meet in LDS and write one partial result (maximum, sum, fp32
// accumulator) per split; a second small kernel merges the splits. The position of the query may come from device memory, so that a
// captured step can be replayed while the position advances: splits wholly past
// it write an empty partial without touching the cache.
//
// Replaces, for sq = 1, matmul(q, k^T) -> FusedScaleMaskSoftmax -> matmul(p, v)
// of the fused attention (oslo/models/gptj/modeling_gptj.py:936-951,
// oslo/models/gpt2/modeling_gpt2.py:1435-1459).

#include <algorithm>

#include "common.hpp"

namespace oslo {
namespace {

constexpr uint32_t kOutside = 0x80000000u;
constexpr float kLog2e = 1.4426950408889634f;

__device__ __forceinline__ float lane_xor(float v, int mask) {
  return __shfl_xor(v, mask, kWave);
}

// Keys one wave takes: LPK lanes hold one key (a 128-bit vector each).
template <int LPK>
struct DecodeTile {
  static constexpr int kKeysPerLoad = kWave / LPK;
  static constexpr int kLoads = LPK == 64 ? 8 : 16 / kKeysPerLoad;
  static constexpr int kKeysPerWave = kKeysPerLoad * kLoads;
  static constexpr int kKeysPerBlock = kKeysPerWave * kWavesPerBlock;
};

// Partial results: [rows_heads][splits][2 + head_dim] floats: maximum (log2
// domain), sum of exponentials, accumulator.
template <typename T, int LPK>
__global__ __launch_bounds__(kBlockThreads) void attention_decode_partial_kernel(
    float *__restrict__ ws, const T *__restrict__ q, T *k, T *v,
    const T *__restrict__ k_new, const T *__restrict__ v_new, int heads,
    int64_t new_seq_stride, const int64_t *__restrict__ pos_dev,
    int64_t pos_host, int window, float scale_log2e, int capacity,
    int head_dim, int splits, int tiles) {
  constexpr int VEC = Io<T>::kVec;
  using Tile = DecodeTile<LPK>;
  constexpr int U = Tile::kLoads;
  __shared__ float part[kWavesPerBlock][LPK * VEC];
  __shared__ float part_m[kWavesPerBlock], part_l[kWavesPerBlock];

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int split = blockIdx.x % splits;
  const int64_t bh = blockIdx.x / splits;
  const int sub = lane / LPK; // key within a load
  const int dl = lane % LPK;  // vector within the key

  int64_t last = pos_dev != nullptr ? *pos_dev : pos_host; // last visible key
  if (last > capacity - 1) last = capacity - 1;
  const int64_t first = window > 0 && last - window + 1 > 0 ? last - window + 1 : 0;
  float *out = ws + (bh * splits + split) * (int64_t)(2 + head_dim);

  // a block covers `tiles` tiles of kKeysPerBlock keys
  const int block_key0 = split * tiles * Tile::kKeysPerBlock;
  if (block_key0 > last || block_key0 + tiles * Tile::kKeysPerBlock <= first) {
    // nothing visible in this split (uniform over the block)
    if (threadIdx.x == 0) {
      out[0] = -INFINITY;
      out[1] = 0.f;
    }
    return;
  }

  const uint32_t key_bytes = (uint32_t)head_dim * (uint32_t)sizeof(T);
  const uint32_t cache_bytes = (uint32_t)capacity * key_bytes;
  const BufRsrc krs = make_rsrc(k + bh * (int64_t)capacity * head_dim, cache_bytes);
  const BufRsrc vrs = make_rsrc(v + bh * (int64_t)capacity * head_dim, cache_bytes);
  const BufRsrc qrs = make_rsrc(q + bh * (int64_t)head_dim, key_bytes);
  float qf[VEC];
  raw_to_f32<T, VEC>(qf, buffer_load_raw<T, VEC, false>(qrs, (uint32_t)dl * 16u));
  // The key and value of the query's own position may still be outside the
  // cache: they are used from where they are and written into their slot by
  // the one wave that owns it.
  const bool fresh = k_new != nullptr;
  RawVec<T, VEC> knew, vnew;
  if (fresh) {
    // [sequence, head, head_dim] with a stride between sequences (dense, or
    // slices of a packed q|k|v projection)
    const int64_t at = (bh / heads) * new_seq_stride + (bh % heads) * (int64_t)head_dim;
    knew = buffer_load_raw<T, VEC, false>(make_rsrc(k_new + at, key_bytes), (uint32_t)dl * 16u);
    vnew = buffer_load_raw<T, VEC, false>(make_rsrc(v_new + at, key_bytes), (uint32_t)dl * 16u);
  }

  // running maximum, sum and accumulator of the wave (over its tiles)
  float m = -INFINITY, l = 0.f;
  float acc[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) acc[j] = 0.f;

#pragma unroll 1
  for (int tile = 0; tile < tiles; ++tile) {
    const int key0 = block_key0 + (tile * kWavesPerBlock + wave) * Tile::kKeysPerWave;
    if (key0 > last) break; // wave-uniform: later tiles are past the query too
    RawVec<T, VEC> kraw[U], vraw[U];
    bool vis[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int s = key0 + u * Tile::kKeysPerLoad + sub;
      vis[u] = s >= first && s <= last;
      const bool from_cache = vis[u] && !(fresh && s == last);
      const uint32_t off = from_cache ? (uint32_t)s * key_bytes + (uint32_t)dl * 16u : kOutside;
      kraw[u] = buffer_load_raw<T, VEC, true>(krs, off);
      vraw[u] = buffer_load_raw<T, VEC, true>(vrs, off);
    }
    if (fresh) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int s = key0 + u * Tile::kKeysPerLoad + sub;
        if (s == last) {
          kraw[u] = knew;
          vraw[u] = vnew;
          const int64_t slot = (bh * capacity + s) * (int64_t)head_dim + dl * VEC;
          *reinterpret_cast<RawVec<T, VEC> *>(k + slot) = knew;
          *reinterpret_cast<RawVec<T, VEC> *>(v + slot) = vnew;
        }
      }
    }

    // scores of the tile's keys, in log2 units; every lane of a key gets its score
    float score[U];
    float mt = -INFINITY;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      float kf[VEC];
      raw_to_f32<T, VEC>(kf, kraw[u]);
      float d = 0.f;
#pragma unroll
      for (int j = 0; j < VEC; ++j) d = __builtin_fmaf(kf[j], qf[j], d);
      d = sum_over_lanes<LPK>(d); // the lanes of the key
      score[u] = vis[u] ? d * scale_log2e : -INFINITY;
      mt = fmaxf(mt, score[u]);
    }
    mt = wave_allreduce(mt, OpMax());
    const float m_new = fmaxf(m, mt);
    const float shift = m_new == -INFINITY ? 0.f : m_new; // nothing visible so far
    const float keep = __builtin_amdgcn_exp2f(m - shift);  // rescales what was summed before; exp2(-inf) = 0
    m = m_new;
    l *= keep;
#pragma unroll
    for (int j = 0; j < VEC; ++j) acc[j] *= keep;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const float p = __builtin_amdgcn_exp2f(score[u] - shift);
      l += dl == 0 ? p : 0.f; // one lane per key counts it
      float vf[VEC];
      raw_to_f32<T, VEC>(vf, vraw[u]);
#pragma unroll
      for (int j = 0; j < VEC; ++j) acc[j] = __builtin_fmaf(p, vf[j], acc[j]);
    }
  }
  // the keys of one load sit in different lane groups: add the groups up
  l = wave_allreduce(l, OpAdd());
#pragma unroll
  for (int s = LPK; s < kWave; s <<= 1) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) acc[j] += lane_xor(acc[j], s);
  }
  if (sub == 0) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) part[wave][dl * VEC + j] = acc[j];
  }
  if (lane == 0) {
    part_m[wave] = m;
    part_l[wave] = l;
  }
  __syncthreads();

  // the four waves' partials -> one per split
  float big = part_m[0];
#pragma unroll
  for (int w = 1; w < kWavesPerBlock; ++w) big = fmaxf(big, part_m[w]);
  float wgt[kWavesPerBlock];
  float sum = 0.f;
#pragma unroll
  for (int w = 0; w < kWavesPerBlock; ++w) {
    wgt[w] = part_m[w] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(part_m[w] - big);
    sum += wgt[w] * part_l[w];
  }
  if (threadIdx.x == 0) {
    out[0] = big;
    out[1] = sum;
  }
  for (int t = threadIdx.x; t < head_dim; t += kBlockThreads) {
    float a = 0.f;
#pragma unroll
    for (int w = 0; w < kWavesPerBlock; ++w) a = __builtin_fmaf(wgt[w], part[w][t], a);
    out[2 + t] = a;
  }
}

// One block of 1024 threads per (sequence, head): the first wave reads the
// maxima and sums of all splits (a lane per split), reduces them and leaves
// each split's weight exp2(m_s - max) / total in LDS; then the threads, as
// 1024 / head_dim groups of head_dim, add up the weighted accumulators (group
// g takes the splits s = g mod groups, eight independent loads at a time) and
// meet in LDS. head_dim is a power of two up to 512.
constexpr int kMaxSplits = 2048;
constexpr int kMergeThreads = 1024;

template <typename T>
__global__ __launch_bounds__(kMergeThreads) void attention_decode_merge_kernel(
    T *__restrict__ out, const float *__restrict__ ws, int head_dim, int splits) {
  __shared__ float weight[kMaxSplits];
  __shared__ float red[kMergeThreads];
  const int64_t bh = blockIdx.x;
  const int64_t stride = 2 + head_dim;
  const float *base = ws + bh * splits * stride;
  if (threadIdx.x < kWave) {
    float big = -INFINITY;
    for (int s = threadIdx.x; s < splits; s += kWave) big = fmaxf(big, base[s * stride]);
    big = wave_allreduce(big, OpMax());
    float sum = 0.f;
    for (int s = threadIdx.x; s < splits; s += kWave) {
      const float ms = base[s * stride];
      const float w = ms == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(ms - big);
      weight[s] = w;
      sum = __builtin_fmaf(w, base[s * stride + 1], sum);
    }
    sum = wave_allreduce(sum, OpAdd());
    // no visible key at all (a position below 0 read from device memory): every
    // weight stays 0 and the output is zeros, never an unwritten accumulator
    const float inv = sum > 0.f ? 1.0f / sum : 0.f;
    for (int s = threadIdx.x; s < splits; s += kWave) weight[s] *= inv;
  }
  __syncthreads();
  const int groups = kMergeThreads / head_dim;
  const int g = threadIdx.x / head_dim, t = threadIdx.x % head_dim;
  float a = 0.f;
#pragma unroll 8
  for (int s = g; s < splits; s += groups) {
    const float w = weight[s];
    // an empty split has weight 0 and an accumulator that was never written
    a += w != 0.f ? w * base[s * stride + 2 + t] : 0.f;
  }
  red[threadIdx.x] = a;
  __syncthreads();
  if (g == 0) {
    for (int j = 1; j < groups; ++j) a += red[j * head_dim + t];
    out[bh * head_dim + t] = static_cast<T>(a);
  }
}

template <typename T, int LPK>
int launch(void *out, const void *q, void *k, void *v, const void *k_new,
           const void *v_new, int heads, int64_t new_seq_stride, float *ws,
           const int64_t *pos_dev, int64_t pos, int window, float scale,
           int64_t rows_heads, int capacity, int head_dim, hipStream_t stream) {
  // As many splits as fill the device (about four blocks per CU), not more:
  // every split is a partial result the merge has to read. A block then covers
  // `tiles` tiles of keys.
  const int most = (capacity + DecodeTile<LPK>::kKeysPerBlock - 1) / DecodeTile<LPK>::kKeysPerBlock;
  const int64_t wanted = (1024 + rows_heads - 1) / rows_heads;
  int splits = (int)std::min<int64_t>(most, std::max<int64_t>(wanted, 1));
  const int tiles = (most + splits - 1) / splits;
  splits = (most + tiles - 1) / tiles;
  attention_decode_partial_kernel<T, LPK>
      <<<dim3((unsigned)(rows_heads * splits)), dim3(kBlockThreads), 0, stream>>>(
          ws, static_cast<const T *>(q), static_cast<T *>(k), static_cast<T *>(v),
          static_cast<const T *>(k_new), static_cast<const T *>(v_new), heads,
          new_seq_stride, pos_dev, pos, window, scale * kLog2e, capacity,
          head_dim, splits, tiles);
  attention_decode_merge_kernel<T>
      <<<dim3((unsigned)rows_heads), dim3(kMergeThreads), 0, stream>>>(
          static_cast<T *>(out), ws, head_dim, splits);
  return check_launch("oslo_attention_decode_fwd");
}

// Lanes per key for a head of `bytes` bytes, 0 if unsupported.
int lanes_per_key(int64_t bytes) {
  switch (bytes) {
  case 128: return 8;
  case 256: return 16;
  case 512: return 32;
  case 1024: return 64;
  default: return 0;
  }
}

int keys_per_block(int lpk) {
  switch (lpk) {
  case 8: return DecodeTile<8>::kKeysPerBlock;
  case 16: return DecodeTile<16>::kKeysPerBlock;
  case 32: return DecodeTile<32>::kKeysPerBlock;
  default: return DecodeTile<64>::kKeysPerBlock;
  }
}

} // namespace
} // namespace oslo

extern "C" size_t oslo_attention_decode_workspace_bytes(int64_t rows_heads,
                                                        int64_t capacity,
                                                        int64_t head_dim,
                                                        int dtype) {
  const int64_t es = dtype == OSLO_F32 ? 4 : 2;
  const int lpk = oslo::lanes_per_key(head_dim * es);
  if (rows_heads <= 0 || capacity <= 0 || lpk == 0) return 0;
  const int kpb = oslo::keys_per_block(lpk);
  const int64_t splits = (capacity + kpb - 1) / kpb;
  return (size_t)rows_heads * (size_t)splits * (size_t)(2 + head_dim) * sizeof(float);
}

extern "C" int oslo_attention_decode_fwd(void *out, const void *q, void *k,
                                         void *v, const void *k_new,
                                         const void *v_new, int64_t heads,
                                         int64_t new_seq_stride,
                                         float *workspace,
                                         const int64_t *pos_dev, int64_t pos,
                                         int64_t window, float scale,
                                         int64_t rows_heads, int64_t capacity,
                                         int64_t head_dim, int dtype,
                                         oslo_stream_t stream) {
  using namespace oslo;
  if (rows_heads < 0 || capacity < 0 || head_dim < 0 || window < 0)
    return fail(OSLO_E_BAD_ARG, "oslo_attention_decode_fwd: negative size");
  if (dtype != OSLO_F32 && dtype != OSLO_F16 && dtype != OSLO_BF16)
    return fail(OSLO_E_BAD_ARG, "unknown dtype %d", dtype);
  if (rows_heads == 0) return OSLO_OK;
  const int64_t es = dtype == OSLO_F32 ? 4 : 2;
  const int lpk = lanes_per_key(head_dim * es);
  if (lpk == 0)
    return fail(OSLO_E_UNSUPPORTED,
                "oslo_attention_decode_fwd: heads of %lld bytes (128, 256, 512 or 1024 are taken)",
                (long long)(head_dim * es));
  if (capacity == 0 || capacity * head_dim * es > (int64_t)0x7fffffff)
    return fail(OSLO_E_UNSUPPORTED,
                "oslo_attention_decode_fwd: a cache of %lld keys per head (1 key to 2 GiB are taken)",
                (long long)capacity);
  const int64_t splits = (capacity + keys_per_block(lpk) - 1) / keys_per_block(lpk);
  if (splits > kMaxSplits)
    return fail(OSLO_E_UNSUPPORTED, "oslo_attention_decode_fwd: a cache of %lld keys per head (at most %d are taken)",
                (long long)capacity, kMaxSplits * keys_per_block(lpk));
  if (rows_heads > (int64_t)0x7fffffff / splits)
    return fail(OSLO_E_UNSUPPORTED, "oslo_attention_decode_fwd: too many heads for one launch");
  if (pos_dev == nullptr && (pos < 0 || pos >= capacity))
    return fail(OSLO_E_BAD_ARG, "oslo_attention_decode_fwd: position %lld outside the cache of %lld keys",
                (long long)pos, (long long)capacity);
  if (!out || !q || !k || !v || !workspace)
    return fail(OSLO_E_BAD_ARG, "oslo_attention_decode_fwd: null pointer");
  if ((k_new == nullptr) != (v_new == nullptr))
    return fail(OSLO_E_BAD_ARG, "oslo_attention_decode_fwd: k_new and v_new go together");
  if (k_new != nullptr) {
    if (heads <= 0 || rows_heads % heads != 0)
      return fail(OSLO_E_BAD_ARG, "oslo_attention_decode_fwd: %lld heads do not divide %lld rows",
                  (long long)heads, (long long)rows_heads);
    if (new_seq_stride == 0) new_seq_stride = heads * head_dim;
    if (new_seq_stride < heads * head_dim || (new_seq_stride * es) % 16 != 0)
      return fail(OSLO_E_BAD_ARG, "oslo_attention_decode_fwd: new_seq_stride %lld (whole 16-byte vectors, at least heads*head_dim)",
                  (long long)new_seq_stride);
  } else {
    heads = 1;
  }
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(k_new) || !aligned16(v_new))
    return fail(OSLO_E_BAD_ARG, "oslo_attention_decode_fwd: q, k, v, k_new and v_new must be 16-byte aligned");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int win = window > capacity ? (int)capacity : (int)window;
  OSLO_DISPATCH_DTYPE(dtype, {
    switch (lpk) {
    case 8: return launch<T, 8>(out, q, k, v, k_new, v_new, (int)heads, new_seq_stride, workspace, pos_dev, pos, win, scale, rows_heads, (int)capacity, (int)head_dim, s);
    case 16: return launch<T, 16>(out, q, k, v, k_new, v_new, (int)heads, new_seq_stride, workspace, pos_dev, pos, win, scale, rows_heads, (int)capacity, (int)head_dim, s);
    case 32: return launch<T, 32>(out, q, k, v, k_new, v_new, (int)heads, new_seq_stride, workspace, pos_dev, pos, win, scale, rows_heads, (int)capacity, (int)head_dim, s);
    default: return launch<T, 64>(out, q, k, v, k_new, v_new, (int)heads, new_seq_stride, workspace, pos_dev, pos, win, scale, rows_heads, (int)capacity, (int)head_dim, s);
    }
  });
  return OSLO_OK;
}
