// Rotary position embedding of the query and key projections, fused with the
// split-heads transposition, for gfx950.
//
// GPT-J's attention (oslo/models/gptj/modeling_gptj.py:49-80, :205-233 of the
// reference) views the q/k/v projections as [B, S, H, D], rotates consecutive
// feature pairs (2i, 2i+1) of the first `rotary_dim` features of q and k by the
// angle of position s, concatenates with the untouched features and permutes
// to [B, H, S, D]: about ten elementwise torch kernels and three strided
// copies per layer. Here it is one launch: every element is read once and
// written once, straight into the [B, H, S, D] layout the score GEMM wants.
//
// The arithmetic is the reference's, in fp32 and in its order:
//   out[2i]   = x[2i]  *cos_i + (-x[2i+1])*sin_i
//   out[2i+1] = x[2i+1]*cos_i +   x[2i]   *sin_i
// with sin/cos read from the caller's fp32 tables (the reference's
// fixed_pos_embedding), so the result equals the reference's fp32 value rounded
// once to the storage type. `inverse` runs the transposed map (the backward):
// layouts swapped, rotation by the opposite angle.

#include "common.hpp"

namespace oslo {
namespace {

constexpr int kRotaryUnroll = 4;
// Byte offset no tensor reaches (one batch entry stays under 2 GiB): a buffer
// access at it is out of range, so the load returns zeros and the store is
// dropped.
constexpr uint32_t kOutside = 0x80000000u;

struct RotaryArgs {
  const void *in[3];
  void *out[3];
  int rotate[3]; // 1: rotary features are rotated; 0: tensor is only transposed
  int count;     // tensors in this launch
};

// One work item = one 128-bit vector. Items are numbered feature vector
// fastest, then position within a tile of `ts` positions, then head: a wave
// writes (forward) or reads (inverse) contiguous pieces of the [B,H,S,D] side
// and pieces of one D-row of the [B,S,H,D] side.
template <typename T, int VEC, bool INVERSE, bool TABLE_VEC>
__global__ __launch_bounds__(kBlockThreads) void rotary_transpose_kernel(
    RotaryArgs a, const float *__restrict__ sin_t, const float *__restrict__ cos_t,
    int S, int H, int D, int64_t row_stride, int rotary_dim, int offset, int ts,
    int items_per_tile, int blocks_per_tile, int s_tiles) {
  const int which = blockIdx.y;
  const T *in = static_cast<const T *>(a.in[which]);
  T *out = static_cast<T *>(a.out[which]);
  const bool rotate = a.rotate[which] != 0;

  const int tile = blockIdx.x / blocks_per_tile; // (batch, position tile)
  const int part = blockIdx.x - tile * blocks_per_tile;
  const int b = tile / s_tiles;
  const int s0 = (tile - b * s_tiles) * ts;
  const int lpr = D / VEC; // lanes per D-row

  // [B,S,H,D] side (a position every row_stride elements: H*D when dense, more
  // when q, k, v are slices of one packed projection) and dense [B,H,S,D] side
  // of batch b
  const int64_t dense_slab = (int64_t)S * H * D;
  const int64_t strided_slab = (int64_t)S * row_stride;
  const uint32_t dense_bytes = (uint32_t)dense_slab * (uint32_t)sizeof(T);
  const uint32_t strided_bytes =
      (uint32_t)((int64_t)(S - 1) * row_stride + (int64_t)H * D) * (uint32_t)sizeof(T);
  const BufRsrc irs = make_rsrc(in + b * (INVERSE ? dense_slab : strided_slab),
                                INVERSE ? dense_bytes : strided_bytes);
  const BufRsrc ors = make_rsrc(out + b * (INVERSE ? strided_slab : dense_slab),
                                INVERSE ? strided_bytes : dense_bytes);

  RawVec<T, VEC> raw[kRotaryUnroll];
  uint32_t off_out[kRotaryUnroll];
  int col[kRotaryUnroll], pos[kRotaryUnroll];
#pragma unroll
  for (int u = 0; u < kRotaryUnroll; ++u) {
    const int item = (part * kRotaryUnroll + u) * kBlockThreads + threadIdx.x;
    const int d8 = item % lpr;
    const int rest = item / lpr;
    const int sl = rest % ts;
    const int h = rest / ts;
    const int s = s0 + sl;
    const bool ok = item < items_per_tile && s < S;
    col[u] = d8 * VEC;
    pos[u] = (ok ? s : 0) + offset; // a table row that exists
    const uint32_t bshd = (uint32_t)((int64_t)s * row_stride + h * D + col[u]) * (uint32_t)sizeof(T);
    const uint32_t bhsd = (uint32_t)(((int64_t)h * S + s) * D + col[u]) * (uint32_t)sizeof(T);
    const uint32_t off_in = ok ? (INVERSE ? bhsd : bshd) : kOutside;
    off_out[u] = ok ? (INVERSE ? bshd : bhsd) : kOutside;
    raw[u] = buffer_load_raw<T, VEC, true>(irs, off_in);
  }

  // sin/cos of the thread's pairs, issued before the data is waited for. A
  // vector past the rotary features reads the row's first entries (cached,
  // unused) so that the loads sit outside any branch.
  constexpr int HALF = VEC / 2;
  float sn[kRotaryUnroll][HALF], cs[kRotaryUnroll][HALF];
  const int half_rot = rotary_dim / 2;
  if (rotate) {
#pragma unroll
    for (int u = 0; u < kRotaryUnroll; ++u) {
      const int64_t row = (int64_t)pos[u] * half_rot;
      if constexpr (TABLE_VEC) {
        // rotary_dim/2 is a multiple of HALF and the tables are aligned: the
        // thread's entries are one aligned vector, wholly inside the row or not
        const int i = col[u] / 2;
        if (i < half_rot) {
          load_f32_cached<float, HALF>(sn[u], sin_t + row + i);
          load_f32_cached<float, HALF>(cs[u], cos_t + row + i);
        } else {
#pragma unroll
          for (int j = 0; j < HALF; ++j) sn[u][j] = cs[u][j] = 0.f;
        }
      } else {
#pragma unroll
        for (int j = 0; j < HALF; ++j) {
          const int i = col[u] / 2 + j;
          const int64_t at = row + (i < half_rot ? i : 0);
          sn[u][j] = sin_t[at];
          cs[u][j] = cos_t[at];
        }
      }
    }
  }

#pragma unroll
  for (int u = 0; u < kRotaryUnroll; ++u) {
    float x[VEC];
    raw_to_f32<T, VEC>(x, raw[u]);
    if (rotate) {
#pragma unroll
      for (int j = 0; j < HALF; ++j) {
        if (col[u] + 2 * j < rotary_dim) { // rotary_dim is even, so the pair is whole
          const float s1 = INVERSE ? -sn[u][j] : sn[u][j];
          const float x0 = x[2 * j], x1 = x[2 * j + 1];
          x[2 * j] = __fadd_rn(__fmul_rn(x0, cs[u][j]), __fmul_rn(-x1, s1));
          x[2 * j + 1] = __fadd_rn(__fmul_rn(x1, cs[u][j]), __fmul_rn(x0, s1));
        }
      }
    }
    buffer_store_f32<T, VEC, 0>(ors, off_out[u], x);
  }
}

template <typename T>
int launch_rotary(const RotaryArgs &a, const float *sin_t, const float *cos_t,
                  int64_t B, int64_t S, int64_t H, int64_t D, int64_t row_stride,
                  int64_t rotary_dim, int64_t offset, bool inverse, hipStream_t stream) {
  constexpr int VEC = Io<T>::kVec;
  const int lpr = (int)(D / VEC);
  // positions per tile: enough for a wave to cover whole D-rows, at least 8
  int ts = 8;
  while (ts * lpr < kBlockThreads) ts *= 2;
  const int s_tiles = (int)((S + ts - 1) / ts);
  const int64_t items_per_tile = (int64_t)H * ts * lpr;
  const int per_block = kBlockThreads * kRotaryUnroll;
  const int blocks_per_tile = (int)((items_per_tile + per_block - 1) / per_block);
  const int64_t blocks = B * s_tiles * blocks_per_tile;
  if (blocks > INT32_MAX || items_per_tile > INT32_MAX)
    return fail(OSLO_E_UNSUPPORTED, "rotary_qkv: tensor too large for one launch");
  const dim3 grid((unsigned)blocks, (unsigned)a.count);
  const bool table_vec = rotary_dim > 0 && (rotary_dim / 2) % (VEC / 2) == 0 &&
                         aligned16(sin_t) && aligned16(cos_t);
  auto go = [&]<bool INVERSE, bool TABLE_VEC>() {
    rotary_transpose_kernel<T, VEC, INVERSE, TABLE_VEC>
        <<<grid, dim3(kBlockThreads), 0, stream>>>(
            a, sin_t, cos_t, (int)S, (int)H, (int)D, row_stride, (int)rotary_dim, (int)offset,
            ts, (int)items_per_tile, blocks_per_tile, s_tiles);
  };
  if (inverse) {
    if (table_vec) go.template operator()<true, true>();
    else go.template operator()<true, false>();
  } else {
    if (table_vec) go.template operator()<false, true>();
    else go.template operator()<false, false>();
  }
  return check_launch("rotary_qkv");
}

} // namespace
} // namespace oslo

extern "C" int oslo_rotary_qkv(void *q_out, void *k_out, void *v_out,
                               const void *q_in, const void *k_in, const void *v_in,
                               const float *sin_table, const float *cos_table,
                               int64_t table_positions, int64_t batch, int64_t seq,
                               int64_t heads, int64_t head_dim, int64_t row_stride,
                               int64_t rotary_dim, int64_t offset, int inverse, int dtype,
                               oslo_stream_t stream) {
  using namespace oslo;
  const char *name = "rotary_qkv";
  if (batch < 0 || seq < 0 || heads < 0 || head_dim < 0 || row_stride < 0 || rotary_dim < 0 ||
      offset < 0)
    return fail(OSLO_E_BAD_ARG, "%s: negative size", name);
  if (rotary_dim > head_dim || rotary_dim % 2 != 0)
    return fail(OSLO_E_BAD_ARG, "%s: rotary_dim %lld must be even and <= head_dim %lld", name,
                (long long)rotary_dim, (long long)head_dim);
  if (dtype != OSLO_F32 && dtype != OSLO_F16 && dtype != OSLO_BF16)
    return fail(OSLO_E_BAD_ARG, "%s: unknown dtype %d", name, dtype);
  const int64_t es = dtype == OSLO_F32 ? 4 : 2;
  const int64_t vec = 16 / es;
  if (batch == 0 || seq == 0 || heads == 0 || head_dim == 0) return OSLO_OK;
  if (head_dim % vec != 0)
    return fail(OSLO_E_UNSUPPORTED, "%s: head_dim %lld is not a multiple of %lld", name,
                (long long)head_dim, (long long)vec);
  if (row_stride == 0) row_stride = heads * head_dim; // dense
  if (row_stride < heads * head_dim || row_stride % vec != 0)
    return fail(OSLO_E_BAD_ARG, "%s: row_stride %lld must be a multiple of %lld and at least heads*head_dim",
                name, (long long)row_stride, (long long)vec);
  if (seq > INT32_MAX / row_stride || seq * row_stride * es >= (int64_t)kOutside)
    return fail(OSLO_E_UNSUPPORTED, "%s: one batch entry must stay under 2 GiB", name);
  RotaryArgs a{};
  const void *ins[3] = {q_in, k_in, v_in};
  void *outs[3] = {q_out, k_out, v_out};
  for (int i = 0; i < 3; ++i) {
    if ((ins[i] == nullptr) != (outs[i] == nullptr))
      return fail(OSLO_E_BAD_ARG, "%s: tensor %d has only one of input and output", name, i);
    if (!ins[i]) continue;
    if (!aligned16(ins[i]) || !aligned16(outs[i]))
      return fail(OSLO_E_UNSUPPORTED, "%s: tensors must be 16-byte aligned", name);
    if (ins[i] == outs[i])
      return fail(OSLO_E_BAD_ARG, "%s: the transposition cannot run in place", name);
    a.in[a.count] = ins[i];
    a.out[a.count] = outs[i];
    a.rotate[a.count] = i < 2 && rotary_dim > 0;
    ++a.count;
  }
  if (a.count == 0) return OSLO_OK;
  if (rotary_dim > 0 && (q_in || k_in)) {
    if (!sin_table || !cos_table) return fail(OSLO_E_BAD_ARG, "%s: null sin/cos table", name);
    if (offset + seq > table_positions)
      return fail(OSLO_E_BAD_ARG, "%s: positions %lld..%lld exceed the table's %lld", name,
                  (long long)offset, (long long)(offset + seq - 1), (long long)table_positions);
  }
  OSLO_DISPATCH_DTYPE(dtype, return launch_rotary<T>(a, sin_table, cos_table, batch, seq, heads,
                                                     head_dim, row_stride, rotary_dim, offset,
                                                     inverse != 0,
                                                     static_cast<hipStream_t>(stream)));
  return OSLO_OK;
}
