// Pieces shared by the one-kernel prompt attention and its backward: the
// matrix-core operation per storage type and the operand types of
// v_mfma_f32_32x32x16 (A and B operands: 8 values per lane; accumulator: 16
// fp32 per lane, lane = column, rows 8j + 4*(lane/32) + t).
#pragma once

#include "common.hpp"

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

// Additive mask values travel in log2 units. Masks of -inf or of the most
// negative finite number (as some callers build them) would make every score
// of a row -inf and its softmax 0/0; they are floored at a value that still
// underflows every exponential but keeps the arithmetic finite.
constexpr float kMaskFloorLog2 = -1e30f;

} // namespace oslo
