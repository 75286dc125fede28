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

// ---------------------------------------------------------------------------
// Which rows a block works on.
//
// Two measured facts about MI355X set this map:
//  * Workgroups go round-robin to the 8 XCDs (workgroup b runs on XCD b % 8),
//    and HBM bandwidth is best when each XCD keeps to one residue class of
//    4 KiB address chunks modulo 8 (a 1 GiB fill: 166 us when every XCD writes
//    one class, 180 us when each writes four). So the rows are cut into units
//    of one 4 KiB chunk (or one row, if rows are longer) and XCD x gets the
//    units u with u % 8 == x.
//  * A causal row r reads r+1 keys and writes S, so in memory order the work
//    in flight swings between write-only (start of a slab) and read-heavy (its
//    end). Taking the units of an XCD alternately from both ends of its list
//    keeps the mix constant (causal forward: 72 % -> 78 % of peak).
// ---------------------------------------------------------------------------
struct RowMap {
  int64_t total_rows;
  int64_t blocks_per_xcd; // launch = 8 * blocks_per_xcd blocks
  int unit_rows;          // rows per unit: 1, 2 or 4, divides the rows of a block
  int paired;             // alternate from both ends (causal kernels)
};

constexpr int kXcds = 8;
constexpr int kChunkBytes = 4096;

inline RowMap make_row_map(int64_t total_rows, int rows_per_block,
                           int64_t row_bytes, bool paired) {
  RowMap m;
  m.total_rows = total_rows;
  m.unit_rows = 1;
  while (m.unit_rows * 2 <= rows_per_block &&
         (int64_t)m.unit_rows * 2 * row_bytes <= kChunkBytes)
    m.unit_rows *= 2;
  const int64_t units = (total_rows + m.unit_rows - 1) / m.unit_rows;
  const int64_t units_per_xcd = (units + kXcds - 1) / kXcds;
  const int units_per_block = rows_per_block / m.unit_rows;
  m.blocks_per_xcd = (units_per_xcd + units_per_block - 1) / units_per_block;
  m.paired = paired ? 1 : 0;
  return m;
}

// Row of the `w`-th row slot (0 .. rows_per_block-1) of workgroup `block`; may
// be >= total_rows (a slot past the end).
__host__ __device__ inline int64_t mapped_row_of(const RowMap &m, int rows_per_block,
                                                 int64_t block, int w) {
  const int64_t xcd = block % kXcds;
  int64_t q = block / kXcds;
  if (m.paired) q = (q & 1) ? m.blocks_per_xcd - 1 - (q >> 1) : (q >> 1);
  const int units_per_block = rows_per_block / m.unit_rows;
  const int64_t unit = xcd + kXcds * (q * units_per_block + w / m.unit_rows);
  return unit * m.unit_rows + w % m.unit_rows;
}
__device__ __forceinline__ int64_t mapped_row(const RowMap &m, int rows_per_block,
                                              int w) {
  return mapped_row_of(m, rows_per_block, blockIdx.x, w);
}

// Dynamic LDS a softmax launch asks for without using it, to cap the blocks
// resident per CU at 4 (16 waves). With long rows fewer waves in flight keep
// the stream of writes compact: measured on [8,16,2048,2048] fp16, forward
// 257 -> 249 us and backward 337 -> 330 us against the 8 blocks per CU the
// register count would allow; 3 blocks per CU is too few for the forward
// (294 us). Short rows keep full occupancy, they need it to hide latency: the
// forward from 4 KiB rows on is capped, the backward (two loads per element
// in flight) from 2 KiB rows on.
constexpr unsigned kLdsPerCu = 160u * 1024u;
inline unsigned occupancy_pad_bytes(bool backward, int64_t row_bytes) {
  const int64_t from = backward ? kChunkBytes / 2 : kChunkBytes;
  return row_bytes >= from ? kLdsPerCu / 4 - 64 : 0u; // 64: the kernels' own LDS
}

// exp(v - m) for a score v and row max m, both in natural-log units.
__device__ __forceinline__ float exp_shifted(float v, float m) {
  return __builtin_amdgcn_exp2f((v - m) * kLog2e);
}

// Picks <NCHUNK, WPR> for a row length and calls fn.template operator()<...>().
// A lane holds at most four vectors wherever the row length allows it: four
// 128-bit loads in flight per lane, 4 KiB per wave, measured best (fp32 rows of
// 2048 as one wave x 8 vectors: 76 % of HBM peak forward, as two waves x 4: 84
// %). Only fp32 rows beyond 4096 take eight (32 fp32 values per lane).
template <int VEC, typename Fn>
inline bool dispatch_row_tile(int64_t cols, Fn &&fn) {
  constexpr int kSpan = kWave * VEC;
  if (cols <= kSpan * 1) {
    fn.template operator()<1, 1>();
  } else if (cols <= kSpan * 2) {
    fn.template operator()<2, 1>();
  } else if (cols <= kSpan * 4) {
    fn.template operator()<4, 1>();
  } else if (cols <= kSpan * 8) {
    fn.template operator()<4, 2>();
  } else if (cols <= kSpan * 16) {
    fn.template operator()<4, 4>();
  } else if (VEC * 8 <= 32 && cols <= kSpan * 32) {
    if constexpr (VEC * 8 <= 32) fn.template operator()<8, 4>();
  } else {
    return false;
  }
  return true;
}

// Longest row: 4 waves x 64 lanes x 32 values.
constexpr int kSoftmaxMaxCols = kWave * 32 * 4;

} // namespace oslo
