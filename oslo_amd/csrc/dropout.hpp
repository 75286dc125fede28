// Dropout keep-mask generation shared by the epilogue kernels and the softmax
// kernels with fused attention dropout: Philox4x32-10 keyed by (seed, offset),
// one counter step per group of eight consecutive elements of the flat tensor,
// 16 random bits per element.
#pragma once

#include "common.hpp"
#include "philox.h"

namespace oslo {

struct DropArgs {
  float keep_scale;   // 1/(1-p)
  uint32_t threshold; // keep iff the element's 16 bits >= threshold
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
// of VEC when VEC is 4 or a multiple of 8; anything when VEC is 1).
template <int VEC>
__device__ __forceinline__ void keep_flags(bool (&keep)[VEC], uint64_t seed,
                                           uint64_t offset, uint64_t i0,
                                           uint32_t threshold) {
  if constexpr (VEC == 1) {
    keep[0] = dropout_bits(dropout_draw(seed, offset, i0 >> 3), (int)(i0 & 7)) >= threshold;
  } else if constexpr (VEC == 4) {
    // half a group: words 0,1 or 2,3 of its draw
    const Philox4 d = dropout_draw(seed, offset, i0 >> 3);
    const bool upper = (i0 & 4) != 0;
    const uint32_t w0 = upper ? d.w[2] : d.w[0], w1 = upper ? d.w[3] : d.w[1];
    keep[0] = (w0 & 0xFFFFu) >= threshold;
    keep[1] = (w0 >> 16) >= threshold;
    keep[2] = (w1 & 0xFFFFu) >= threshold;
    keep[3] = (w1 >> 16) >= threshold;
  } else {
    static_assert(VEC % 8 == 0, "vector paths draw whole groups of eight");
#pragma unroll
    for (int q = 0; q < VEC / 8; ++q) {
      const Philox4 d = dropout_draw(seed, offset, (i0 >> 3) + q);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        keep[8 * q + 2 * j] = (d.w[j] & 0xFFFFu) >= threshold;
        keep[8 * q + 2 * j + 1] = (d.w[j] >> 16) >= threshold;
      }
    }
  }
}

__device__ __forceinline__ bool keep_one(uint64_t seed, uint64_t offset,
                                         uint64_t i, uint32_t threshold) {
  return dropout_bits(dropout_draw(seed, offset, i >> 3), (int)(i & 7)) >= threshold;
}

} // namespace oslo
