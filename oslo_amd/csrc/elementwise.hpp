// Tiling shared by the [rows, cols] epilogue kernels (bias-GeLU, bias-dropout-
// add) and the column-sum that produces their bias gradients.
//
// A 256-thread block is laid out as TX x TY. Thread x owns one vector of VEC
// consecutive columns (its bias values stay in registers); thread y and an
// unroll index u pick the row: a block covers TY*U rows of one column tile,
// every thread issues its U loads at once, computes, stores and exits. There
// is no loop over rows: on MI355X short-lived blocks dispatched in memory order
// sustained 82-85 % of HBM peak on these shapes, against 60-75 % for blocks
// that walk many rows (measured with tiles of 32..128 rows, with and without
// software prefetch, and with grid-stride sweeps).
//
// Blocks are numbered column tile first, so blocks in flight together cover a
// band of whole rows, i.e. one contiguous range of memory.
#pragma once

#include <algorithm>

#include "common.hpp"

namespace oslo {

constexpr int kFwdMaxTx = 64;  // threads along a row, forward kernels
constexpr int kFwdUnroll = 2;  // rows per thread, forward kernels
constexpr int kBwdMaxTx = 32;  // backward kernels: narrower and taller tiles,
                               // so that fewer dbias partial rows are written
// Fewest rows a backward block covers (TY = 256/kBwdMaxTx threads x the
// smallest unroll any backward kernel uses): bounds the number of partial rows.
constexpr int kBwdMinUnroll = 4;
constexpr int kBwdMinRowsPerBlock = kBlockThreads / kBwdMaxTx * kBwdMinUnroll;

// Cache policy of the epilogue kernels. Loads are non-temporal. Stores are
// written through at device scope (sc1), with the non-temporal hint only for
// tensors beyond the 256 MB memory-side cache in front of HBM: without it a
// smaller output stays in that cache for the kernel that consumes it next.
// Measured on a scaled copy, bf16, as a fraction of the HBM peak; "warm" = the
// same buffers every launch (what a consumer sees whose input was just
// produced), "cold" = four sets of buffers in turn:
//   [16384,4096]  nt loads + sc1 stores      warm 0.865  cold 0.775
//                 nt loads + sc1 nt stores   warm 0.778  cold 0.779
//                 plain loads + sc1 nt       warm 0.874  cold 0.765
//   [16384,8192]  0.872 / 0.783,  0.787 / 0.789,  0.878 / 0.772
// At [16384,16384] the forward kernels do not care, the backward kernels (which
// also write their dbias partial rows) lose 2-3 % without the hint.
constexpr int kOutKeep = 16;       // sc1
constexpr int kOutStream = 16 | 2; // sc1 nt
inline bool keep_output_cached(int64_t tensor_bytes) {
  return tensor_bytes <= (256ll << 20);
}

struct EwPlan {
  dim3 grid, block;
  int rows_per_block;
  int col_tiles;
  int64_t row_blocks;
  bool ok; // false: more blocks than one launch can hold
};

// cols_vec = cols / VEC (VEC divides cols on the vector path; VEC = 1 else).
inline EwPlan plan_elementwise(int64_t rows, int64_t cols_vec, int max_tx,
                               int unroll) {
  int tx = max_tx;
  while (tx > 1 && tx / 2 >= cols_vec) tx /= 2; // smallest pow2 >= cols_vec
  const int ty = kBlockThreads / tx;
  EwPlan p;
  p.rows_per_block = ty * unroll;
  p.col_tiles = (int)((cols_vec + tx - 1) / tx);
  p.row_blocks = (rows + p.rows_per_block - 1) / p.rows_per_block;
  const int64_t blocks = p.row_blocks * p.col_tiles;
  // one launch holds < 2^31 blocks; a block's rows are addressed with 32-bit
  // byte offsets (a vector of any dtype is at most 16 bytes)
  p.ok = blocks <= INT32_MAX &&
         (int64_t)p.rows_per_block * cols_vec * 16 <= (int64_t)UINT32_MAX;
  p.block = dim3(tx, ty);
  p.grid = dim3((unsigned)(p.ok ? blocks : 1));
  return p;
}

// Position of a thread's data for the plan above.
struct EwPos {
  int64_t c0;     // first column of the thread's vector
  uint32_t c0_in_row; // the same, for 32-bit offset arithmetic
  int64_t r_base; // row of unroll index 0; row u is r_base + u*blockDim.y
  int64_t row_block;
};

// Column tile and row block of workgroup `block`: column tile fastest.
struct EwTile {
  int64_t col_tile, row_block;
};
__host__ __device__ inline EwTile ew_tile(int col_tiles, int64_t block) {
  return EwTile{block % col_tiles, block / col_tiles};
}

template <int VEC>
__device__ __forceinline__ EwPos ew_position(int col_tiles, int rows_per_block) {
  const EwTile t = ew_tile(col_tiles, blockIdx.x);
  EwPos p;
  p.row_block = t.row_block;
  p.c0 = (t.col_tile * blockDim.x + threadIdx.x) * VEC;
  p.c0_in_row = (uint32_t)p.c0;
  p.r_base = p.row_block * rows_per_block + threadIdx.y;
  return p;
}

// Descriptor for the rows of this block in a [rows, cols] tensor of T: rows past
// the end of the tensor read as zeros. Offsets into it come from ew_offset.
template <typename T>
__device__ __forceinline__ BufRsrc ew_rsrc(const T *base, const EwPos &pos,
                                           int rows_per_block, int64_t rows,
                                           int64_t cols) {
  const int64_t first = pos.row_block * rows_per_block;
  const int64_t here = min((int64_t)rows_per_block, rows - first);
  return make_rsrc(base + first * cols,
                   (uint32_t)(here * cols) * (uint32_t)sizeof(T));
}
template <typename T>
__device__ __forceinline__ uint32_t ew_offset(const EwPos &pos, int u,
                                              int64_t cols) {
  const uint32_t row_in_block = threadIdx.y + (uint32_t)u * blockDim.y;
  return (row_in_block * (uint32_t)cols + (uint32_t)pos.c0_in_row) *
         (uint32_t)sizeof(T);
}

// Block-level finish of a per-thread column accumulator: sums acc over the TY
// threads that share a column vector and writes the tile's part of one fp32
// partial row. The accumulators go to LDS as TY rows of the tile's width; then
// every thread adds up one column (consecutive threads, consecutive columns:
// no bank conflicts, one coalesced store per wave), in a fixed order.
// Every thread of the block must call this (it contains a barrier).
template <int VEC>
__device__ __forceinline__ void write_colsum_partial(
    const float (&acc)[VEC], float *__restrict__ partial, int64_t cols,
    const EwPos &pos) {
  __shared__ float red[kBlockThreads * VEC];
  const int TX = blockDim.x, TY = blockDim.y;
  const int width = TX * VEC; // columns of the tile
#pragma unroll
  for (int j = 0; j < VEC; ++j)
    red[threadIdx.y * width + threadIdx.x * VEC + j] = acc[j];
  __syncthreads();
  const int tid = threadIdx.y * TX + threadIdx.x;
  const int64_t tile_c0 = pos.c0 - (int64_t)threadIdx.x * VEC;
  float *dst = partial + pos.row_block * cols + tile_c0;
  for (int c = tid; c < width && tile_c0 + c < cols; c += kBlockThreads) {
    float s = red[c];
    for (int t = 1; t < TY; ++t) s += red[t * width + c];
    dst[c] = s;
  }
}

// dbias[c] = sum of the fp32 partial rows in[p, c]. A block of 1024 threads owns
// 64 columns; its 16 waves take every 16th row with eight rows in flight each
// and meet in LDS, so even a few hundred partial rows are a handful of
// dependent steps. The order of the additions is fixed: the result is
// deterministic.
constexpr int kFinishThreads = 1024;
constexpr int kFinishWaves = kFinishThreads / kWave;

template <typename OutT>
__global__ __launch_bounds__(kFinishThreads) void colsum_finish_kernel(
    OutT *__restrict__ out, const float *__restrict__ in, int64_t nparts,
    int64_t cols) {
  __shared__ float red[kFinishThreads];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int64_t c = (int64_t)blockIdx.x * kWave + lane;
  float s[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) s[i] = 0.f;
  if (c < cols) {
    int64_t p = wave;
    for (; p + 7 * kFinishWaves < nparts; p += 8 * kFinishWaves) {
#pragma unroll
      for (int i = 0; i < 8; ++i) s[i] += in[(p + i * kFinishWaves) * cols + c];
    }
    for (; p < nparts; p += kFinishWaves) s[0] += in[p * cols + c];
  }
  red[threadIdx.x] = ((s[0] + s[1]) + (s[2] + s[3])) + ((s[4] + s[5]) + (s[6] + s[7]));
  __syncthreads();
  if (wave == 0 && c < cols) {
    float t = red[lane];
#pragma unroll
    for (int w = 1; w < kFinishWaves; ++w) t += red[w * kWave + lane];
    out[c] = static_cast<OutT>(t);
  }
}

template <typename T>
inline void launch_colsum_finish(T *dbias, const float *partial, int64_t nparts,
                                 int64_t cols, hipStream_t stream) {
  const unsigned bx = (unsigned)((cols + kWave - 1) / kWave);
  colsum_finish_kernel<T><<<dim3(bx), dim3(kFinishThreads), 0, stream>>>(
      dbias, partial, nparts, cols);
}

} // namespace oslo
