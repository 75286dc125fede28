// Tiling shared by the [rows, cols] epilogue kernels (bias-GeLU, bias-dropout-
// add) and the column-sum that produces their bias gradients.
//
// A 256-thread block is laid out as TX x TY: thread x owns one vector of VEC
// consecutive columns (its bias values stay in registers), thread y strides
// over the rows of the block's row range. Consecutive x are consecutive 128-bit
// vectors of a row, so a wave reads and writes whole 1 KiB row segments.
#pragma once

#include <algorithm>

#include "common.hpp"

namespace oslo {

constexpr int kRowsPerBlockFwd = 32;  // rows a block walks in forward kernels
constexpr int kRowsPerBlockBwd = 128; // ... in backward kernels (one dbias
                                      // partial row per block row range)
constexpr int kRowUnroll = 4;         // independent row loads in flight/thread

struct EwPlan {
  dim3 grid, block;
  int rows_per_block;
};

// cols_vec = cols / VEC (VEC divides cols on the vector path; VEC = 1 else).
inline EwPlan plan_elementwise(int64_t rows, int64_t cols_vec, int base_rpb) {
  int tx = kBlockThreads;
  while (tx > 1 && tx / 2 >= cols_vec) tx /= 2; // smallest pow2 >= cols_vec
  const int ty = kBlockThreads / tx;
  // gridDim.y is limited to 65535
  int64_t rpb = std::max<int64_t>(base_rpb, (rows + 32767) / 32768);
  rpb = (rpb + ty - 1) / ty * ty;
  EwPlan p;
  p.block = dim3(tx, ty);
  p.grid = dim3((unsigned)((cols_vec + tx - 1) / tx),
                (unsigned)((rows + rpb - 1) / rpb));
  p.rows_per_block = (int)rpb;
  return p;
}

// Number of partial rows the backward kernels write for a problem: one per
// block row range of plan_elementwise(..., kRowsPerBlockBwd).
inline int64_t colsum_partials(int64_t rows, int64_t cols_vec) {
  if (rows <= 0) return 0;
  return plan_elementwise(rows, cols_vec, kRowsPerBlockBwd).grid.y;
}

// Block-level finish of a per-thread column accumulator: sums acc over the TY
// threads that share a column vector and writes one fp32 partial row.
// Every thread of the block must call this (it contains a barrier).
template <int VEC>
__device__ __forceinline__ void write_colsum_partial(
    const float (&acc)[VEC], float *__restrict__ partial, int64_t cols,
    int64_t c0, bool col_ok) {
  __shared__ float red[kBlockThreads * VEC];
  const int tx = threadIdx.x, ty = threadIdx.y;
  const int TX = blockDim.x, TY = blockDim.y;
  if (TY > 1) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) red[(ty * TX + tx) * VEC + j] = acc[j];
    __syncthreads();
  }
  if (ty == 0 && col_ok) {
    float *dst = partial + (int64_t)blockIdx.y * cols + c0;
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      float s = acc[j];
      for (int t = 1; t < TY; ++t) s += red[(t * TX + tx) * VEC + j];
      dst[j] = s;
    }
  }
}

// dbias[c] = sum over the partial rows, in row order (deterministic).
template <typename T>
__global__ __launch_bounds__(kBlockThreads) void colsum_finish_kernel(
    T *__restrict__ dbias, const float *__restrict__ partial, int nparts,
    int64_t cols) {
  const int64_t c = (int64_t)blockIdx.x * kBlockThreads + threadIdx.x;
  if (c >= cols) return;
  float s = 0.f;
  for (int p = 0; p < nparts; ++p) s += partial[(int64_t)p * cols + c];
  dbias[c] = static_cast<T>(s);
}

template <typename T>
inline void launch_colsum_finish(T *dbias, const float *partial, int nparts,
                                 int64_t cols, hipStream_t stream) {
  const unsigned blocks = (unsigned)((cols + kBlockThreads - 1) / kBlockThreads);
  colsum_finish_kernel<T><<<dim3(blocks), dim3(kBlockThreads), 0, stream>>>(
      dbias, partial, nparts, cols);
}

} // namespace oslo
