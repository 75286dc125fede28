// Row-softmax machinery shared by the causal and the key-mask kernels.
//
// A row of scores lives in registers as fp32 for the whole kernel: it is read
// from HBM once and written once. WPR waves of a 256-thread block share one
// row (1 for rows up to 64*VEC*NCHUNK elements, 2 or 4 beyond); a lane owns
// NCHUNK vectors of VEC consecutive elements, and the vectors of one chunk are
// consecutive across the lanes of a wave, so every access is a full 128-bit
// per lane, 1 KiB per wave, coalesced request. Waves that share a row exchange
// their partial max / sum through a few floats of LDS.
#pragma once

#include "common.hpp"

namespace oslo {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kMaskValue = -10000.0f;

template <int VEC, int NCHUNK, int WPR>
struct RowTile {
  static_assert(kWavesPerBlock % WPR == 0, "waves of a row must fill a block");
  static constexpr int kSpan = kWave * VEC;             // elements per chunk
  static constexpr int kMaxCols = kSpan * NCHUNK * WPR; // longest row
  static constexpr int kRowsPerBlock = kWavesPerBlock / WPR;
  // First column of chunk c for lane `lane` of the `sub`-th wave of a row.
  // Chunks are dealt round-robin to the waves of a row so that a short causal
  // prefix still spreads over all of them.
  static __device__ __forceinline__ int col(int c, int sub, int lane) {
    return (c * WPR + sub) * kSpan + lane * VEC;
  }
};

// All-reduce over the WPR waves that share a row. `slots` is kWavesPerBlock
// floats of LDS used by this one reduction only (no reuse, so one barrier).
template <int WPR, typename Op>
__device__ __forceinline__ float row_allreduce(float v, Op op, float *slots) {
  v = wave_allreduce(v, op);
  if constexpr (WPR > 1) {
    const int wave = threadIdx.x / kWave;
    if ((threadIdx.x & (kWave - 1)) == 0) slots[wave] = v;
    __syncthreads();
    const int base = wave / WPR * WPR;
    float r = slots[base];
#pragma unroll
    for (int i = 1; i < WPR; ++i) r = op(r, slots[base + i]);
    v = r;
  }
  return v;
}

// Block order for the causal kernels. Row r of a slab reads r+1 keys and writes
// S, so blocks taken in memory order alternate between write-only phases
// (start of a slab) and read-heavy ones (end). Dealing blocks from both ends of
// the launch alternately keeps the read:write mix of the work in flight
// constant, which measured 5-6 % faster on MI355X than memory order.
__device__ __forceinline__ int64_t paired_block(int64_t b, int64_t nblocks) {
  return (b & 1) ? nblocks - 1 - (b >> 1) : (b >> 1);
}

// exp(v - m) for a score v and row max m, both in natural-log units.
__device__ __forceinline__ float exp_shifted(float v, float m) {
  return __builtin_amdgcn_exp2f((v - m) * kLog2e);
}

// Picks <NCHUNK, WPR> for a row length and calls fn.template operator()<...>().
// Rows are kept at <= 32 fp32 values per lane (NCHUNK*VEC <= 32).
template <int VEC, typename Fn>
inline bool dispatch_row_tile(int64_t cols, Fn &&fn) {
  constexpr int kSpan = kWave * VEC;
  constexpr int kMaxChunk = 32 / VEC;
  if (cols <= kSpan * 1) {
    fn.template operator()<1, 1>();
  } else if (cols <= kSpan * 2) {
    fn.template operator()<2, 1>();
  } else if (cols <= kSpan * kMaxChunk) {
    fn.template operator()<kMaxChunk, 1>();
  } else if (cols <= kSpan * kMaxChunk * 2) {
    fn.template operator()<kMaxChunk, 2>();
  } else if (cols <= kSpan * kMaxChunk * 4) {
    fn.template operator()<kMaxChunk, 4>();
  } else {
    return false;
  }
  return true;
}

// Longest row: 4 waves x 64 lanes x 32 values.
constexpr int kSoftmaxMaxCols = kWave * 32 * 4;

} // namespace oslo
