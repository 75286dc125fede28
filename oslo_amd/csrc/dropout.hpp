// Dropout keep-mask generation shared by the epilogue kernels and the softmax
// kernels with fused attention dropout: Philox4x32-10 keyed by (seed, offset),
// one counter step per group of four consecutive elements of the flat tensor.
#pragma once

#include "common.hpp"
#include "philox.h"

namespace oslo {

struct DropArgs {
  float keep_scale;   // 1/(1-p)
  uint32_t threshold; // keep iff word >= threshold
  uint64_t seed, offset;
  bool drop;          // p > 0
};

// Validates p in [0, 1) and fills the arguments.
inline int make_drop_args(const char *name, float p, uint64_t seed,
                          uint64_t offset, DropArgs *a) {
  if (!(p >= 0.0f) || !(p < 1.0f))
    return fail(OSLO_E_BAD_ARG, "%s: p = %g is outside [0, 1)", name, (double)p);
  a->drop = p > 0.0f;
  a->keep_scale = (float)(1.0 / (1.0 - (double)p));
  a->threshold = dropout_threshold(p);
  a->seed = seed;
  a->offset = offset;
  return OSLO_OK;
}

// keep flags of VEC consecutive elements starting at flat index i0 (a multiple
// of VEC when VEC is 4 or 8; anything when VEC is 1).
template <int VEC>
__device__ __forceinline__ void keep_flags(bool (&keep)[VEC], uint64_t seed,
                                           uint64_t offset, uint64_t i0,
                                           uint32_t threshold) {
  if constexpr (VEC == 1) {
    const Philox4 d = dropout_draw(seed, offset, i0 >> 2);
    keep[0] = d.w[i0 & 3] >= threshold;
  } else {
    static_assert(VEC % 4 == 0, "vector paths draw whole groups of four");
#pragma unroll
    for (int q = 0; q < VEC / 4; ++q) {
      const Philox4 d = dropout_draw(seed, offset, (i0 >> 2) + q);
#pragma unroll
      for (int j = 0; j < 4; ++j) keep[4 * q + j] = d.w[j] >= threshold;
    }
  }
}

__device__ __forceinline__ bool keep_one(uint64_t seed, uint64_t offset,
                                         uint64_t i, uint32_t threshold) {
  return dropout_draw(seed, offset, i >> 2).w[i & 3] >= threshold;
}

} // namespace oslo
