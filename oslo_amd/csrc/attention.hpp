// Pieces shared by the one-kernel prompt attention and its backward: the
// matrix-core operation per storage type and the operand types of
// v_mfma_f32_32x32x16 (A and B operands: 8 values per lane; accumulator: 16
// fp32 per lane, lane = column, rows 8j + 4*(lane/32) + t).
#pragma once

#include "common.hpp"
#include "dropout.hpp"

namespace oslo {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

template <typename T>
struct MatrixOp;
template <>
struct MatrixOp<bf16> {
  typedef bf16 Frag __attribute__((ext_vector_type(8)));
  static __device__ __forceinline__ f32x16 run(Frag a, Frag b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};
template <>
struct MatrixOp<f16> {
  typedef f16 Frag __attribute__((ext_vector_type(8)));
  static __device__ __forceinline__ f32x16 run(Frag a, Frag b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};

// The value the other half of the wave (lane ^ 32) holds.
__device__ __forceinline__ float other_half(float v) {
  return __shfl_xor(v, 32, kWave);
}

// Maximum and sum of the values lanes l and l ^ 32 hold, in both lanes, on the
// vector ALU (no LDS queue involved): v_permlane32_swap exchanges the upper
// half of its first register with the lower half of its second; given two
// copies of a value it leaves the lower half's value in every lane of the
// first and the upper half's in every lane of the second. (Written out, with
// idle cycles either side for the instruction's register hazards: through the
// builtin the two results came back as one register.)
__device__ __forceinline__ void halves_split(float v, float &lower, float &upper) {
  lower = v, upper = v;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(lower), "+v"(upper));
}
__device__ __forceinline__ float halves_max(float v) {
  float lo, hi;
  halves_split(v, lo, hi);
  return fmaxf(lo, hi);
}
__device__ __forceinline__ float halves_sum(float v) {
  float lo, hi;
  halves_split(v, lo, hi);
  return lo + hi;
}

// Calls f with four pointers the compiler may take to address distinct memory
// (the two buffers a tile reads and the two it writes while it is computed):
// without that it keeps every LDS read behind every LDS write that precedes it
// in the source.
template <typename T, typename F>
__device__ __forceinline__ void with_distinct_buffers(const T *__restrict__ read_a, T *__restrict__ write_a,
                                                      const T *__restrict__ read_b, T *__restrict__ write_b,
                                                      F &&f) {
  f(read_a, write_a, read_b, write_b);
}

// Loads from global memory straight into LDS, for kernels that stream tiles
// of [position][feature] rows. A tile is loaded through a descriptor of its
// own (base = the tile's first row, size = what is left of the head's slice
// from there, nothing for tiles outside [0, end): rows past the slice and
// whole tiles that are not needed read as zeros without a memory access),
// kept as scalars and stepped from tile to tile.
struct TileStream {
  uint64_t base; // the tile's first row
  uint32_t left; // bytes from there to the end of the slice
  uint32_t step; // bytes from a tile to the next
  int tile, end;
  __device__ __forceinline__ void start(const void *p, uint32_t bytes, uint32_t row_bytes, int rows_per_tile, int t,
                                        int tiles_end) {
    step = (uint32_t)rows_per_tile * row_bytes;
    tile = t;
    end = tiles_end;
    const uint32_t skip = (uint32_t)(t < 0 ? 0 : t) * step;
    base = reinterpret_cast<uint64_t>(p) + skip;
    left = skip < bytes ? bytes - skip : 0u;
  }
  __device__ __forceinline__ void advance() {
    base += step;
    left = left > step ? left - step : 0u;
    ++tile;
  }
  // raw 32-bit buffer descriptor (word 3 = 0x00020000, as make_rsrc builds it),
  // read as scalars: the hand-written loads take it in scalar registers
  __device__ __forceinline__ u32x4 descriptor() const {
    u32x4 d;
    d[0] = __builtin_amdgcn_readfirstlane((uint32_t)base);
    d[1] = __builtin_amdgcn_readfirstlane((uint32_t)(base >> 32) & 0xffffu);
    d[2] = __builtin_amdgcn_readfirstlane(tile >= 0 && tile < end ? left : 0u);
    d[3] = 0x00020000u;
    return d;
  }
};
// The loads themselves are written out: the compiler, told of a load into LDS
// (the builtin), waits for every such load before the next LDS read of any
// buffer. These are waited for by count (wait_vm). A wave's instruction puts
// its 64 x 16 (or 64 x 4) bytes at consecutive LDS addresses from `dst` on.
// The LDS address travels in M0, written inside the same asm statement: on
// this family a scalar write of M0 needs one wait state before a load into LDS
// reads it, which the compiler inserts for its own code and not inside inline
// asm, hence the s_nop. Nothing else in the attention kernels uses M0 (LDS
// reads and writes, lane reads and the matrix products do not; there is no
// indirect register indexing, message or interpolation instruction), and every
// statement that needs it sets it itself, so no value of M0 has to survive
// from one statement to the next, whatever the compiler makes of the clobber.
__device__ __forceinline__ void lds_load_b128(const u32x4 &desc, const void *dst, uint32_t offset) {
  const uint32_t at = __builtin_amdgcn_readfirstlane((uint32_t)reinterpret_cast<uintptr_t>(dst));
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds" : : "s"(at), "v"(offset), "s"(desc) : "m0");
}
// The same load with the non-temporal hint: data that is read once.
__device__ __forceinline__ void lds_load_b128_once(const u32x4 &desc, const void *dst, uint32_t offset) {
  const uint32_t at = __builtin_amdgcn_readfirstlane((uint32_t)reinterpret_cast<uintptr_t>(dst));
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen nt lds" : : "s"(at), "v"(offset), "s"(desc) : "m0");
}
__device__ __forceinline__ void lds_load_b32(const u32x4 &desc, const void *dst, uint32_t offset) {
  const uint32_t at = __builtin_amdgcn_readfirstlane((uint32_t)reinterpret_cast<uintptr_t>(dst));
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, 0 offen lds" : : "s"(at), "v"(offset), "s"(desc) : "m0");
}
// vmcnt <= N, nothing else: all but the N most recent loads have arrived
template <int N>
__device__ __forceinline__ void wait_vm() {
  __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
}

// Additive mask values below kMaskFloor act as kMaskFloor, in the forward and in
// every pass of the backward (one constant, applied to the value in natural
// units before anything else). Callers build masks of -10000, of -inf or of the
// most negative finite number; the last two would make every score of a row
// -inf (0/0 in the softmax), and any value of magnitude above about 2^31 breaks
// the kernels' arithmetic even on rows that see valid keys: a row's reference
// maximum is the rounded product score * log2(e), an exponent is the exact
// fma(score, log2(e), -maximum), and their difference is the product's rounding
// error, up to half an ulp of the maximum: 6e22 at 1e30, whose exp2 is inf (and
// inf * 0 = NaN at the next rescaling). At -2^22 that error is at most 0.25, a
// masked key's probability still underflows to exactly 0 beside any score a
// 16-bit model produces (|scaled score| far below 4e6), and a row whose every
// visible key is masked comes out finite (close to the softmax of the scores
// alone, like a -10000 mask).
constexpr float kMaskFloor = -4194304.0f; // -2^22

// Attention dropout inside the attention kernels. The keep flag of the
// probability of (query q, key k) of head bh is the one the softmax kernel with
// fused dropout draws for the flat index ((bh*S + q)*S + k) of a
// [batch, heads, S, S] tensor: Philox4x32-10, one draw per group of eight
// consecutive keys, 16 bits per key (S must be a multiple of 8, so that a
// group lies inside one row). A wave needs the flags of a 32 x 32 tile of
// (query, key) pairs per step: 128 draws, two per lane. Lane (query q0 + lane %
// 32, pair lane / 32) draws the groups of keys k0 + 16*(lane/32) .. +15, turns
// each into a byte of keep bits and puts the two bytes into the wave's own 128
// bytes of LDS, [query][key / 8]; every lane then reads back the bits of the
// pairs its accumulator registers hold, whichever of query and key is the lane.
__device__ __forceinline__ void stage_keep_bits(uint32_t *wave_bits /* 32 words */, const DropArgs &d,
                                                int64_t bh, int S, int q0, int k0, int lane) {
  const int qi = lane & 31, pair = lane >> 5;
  const uint64_t group = ((uint64_t)bh * S + (uint64_t)(q0 + qi)) * (uint64_t)(S >> 3) +
                         (uint64_t)((k0 >> 3) + 2 * pair);
  uint32_t two = 0;
#pragma unroll
  for (int e = 0; e < 2; ++e) {
    const Philox4 w = dropout_draw(d.seed, d.offset, group + e);
    uint32_t byte = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      byte |= ((w.w[j] & 0xFFFFu) >= d.threshold ? 1u : 0u) << (2 * j);
      byte |= ((w.w[j] >> 16) >= d.threshold ? 1u : 0u) << (2 * j + 1);
    }
    two |= byte << (8 * e);
  }
  // all lanes of the wave have read the previous step's bits before these stores
  __builtin_amdgcn_wave_barrier();
  reinterpret_cast<unsigned short *>(wave_bits)[2 * qi + pair] = (unsigned short)two;
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Keep bits of accumulator register r (row 8*(r/4) + 4*half + r%4 of the tile)
// when the lane is the query and the rows are keys: one word per lane, bit =
// the key's index in the tile.
__device__ __forceinline__ uint32_t keep_word_query_lane(const uint32_t *wave_bits, int col) {
  return wave_bits[col];
}
// ... and when the lane is the key (column `col` of the tile) and the rows are
// queries: four words (queries 8j + 4*half .. + 3) per j, bit = col.
__device__ __forceinline__ u32x4 keep_words_key_lane(const uint32_t *wave_bits, int j, int half) {
  return *reinterpret_cast<const u32x4 *>(&wave_bits[8 * j + 4 * half]);
}

} // namespace oslo
