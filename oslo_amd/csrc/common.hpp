// Shared device helpers for the gfx950 kernels: storage-type traits, 128-bit
// vector access, wave64 reductions, host-side status plumbing.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/oslo_amd.h"

namespace oslo {

constexpr int kWave = 64;          // CDNA wavefront width
constexpr int kBlockThreads = 256; // 4 waves; every kernel here uses this block
constexpr int kWavesPerBlock = kBlockThreads / kWave;

// ---------------------------------------------------------------------------
// Storage types. fp16 is _Float16, bf16 is __bf16: both convert with single
// hardware instructions on gfx950 (v_cvt_f32_f16 / v_cvt_pk_bf16_f32, RNE).
// ---------------------------------------------------------------------------
using f16 = _Float16;
using bf16 = __bf16;

template <typename T, int N>
struct VecOf {
  typedef T type __attribute__((ext_vector_type(N)));
};
template <typename T>
struct VecOf<T, 1> {
  typedef T type;
};

// Elements of T in one 128-bit access.
template <typename T>
struct Io {
  static constexpr int kVec = 16 / sizeof(T);
};

// Load N consecutive elements (address aligned to N*sizeof(T)) as fp32.
// Streaming data is read once, so loads and stores are marked non-temporal.
template <typename T, int N>
__device__ __forceinline__ void load_f32(float (&dst)[N], const T *p) {
  using V = typename VecOf<T, N>::type;
  if constexpr (N == 1) {
    dst[0] = static_cast<float>(__builtin_nontemporal_load(p));
  } else {
    V v = __builtin_nontemporal_load(reinterpret_cast<const V *>(p));
#pragma unroll
    for (int i = 0; i < N; ++i) dst[i] = static_cast<float>(v[i]);
  }
}

// Same, through the normal cached path (for small operands reused by many
// rows: bias vectors, masks).
template <typename T, int N>
__device__ __forceinline__ void load_f32_cached(float (&dst)[N], const T *p) {
  using V = typename VecOf<T, N>::type;
  if constexpr (N == 1) {
    dst[0] = static_cast<float>(*p);
  } else {
    V v = *reinterpret_cast<const V *>(p);
#pragma unroll
    for (int i = 0; i < N; ++i) dst[i] = static_cast<float>(v[i]);
  }
}

template <typename T, int N>
__device__ __forceinline__ void store_f32(T *p, const float (&src)[N]) {
  using V = typename VecOf<T, N>::type;
  if constexpr (N == 1) {
    __builtin_nontemporal_store(static_cast<T>(src[0]), p);
  } else {
    V v;
#pragma unroll
    for (int i = 0; i < N; ++i) v[i] = static_cast<T>(src[i]);
    __builtin_nontemporal_store(v, reinterpret_cast<V *>(p));
  }
}

template <int N>
__device__ __forceinline__ void load_bytes(uint8_t (&dst)[N], const uint8_t *p) {
  using V = typename VecOf<uint8_t, N>::type;
  if constexpr (N == 1) {
    dst[0] = *p;
  } else {
    V v = *reinterpret_cast<const V *>(p);
#pragma unroll
    for (int i = 0; i < N; ++i) dst[i] = v[i];
  }
}

// ---------------------------------------------------------------------------
// Wave64 all-reduce. Four DPP steps inside each row of 16 lanes (quad swaps,
// half-row mirror, row mirror), one ds_swizzle for lane^16, and two v_readlane
// for the 32-lane halves; the result is wave-uniform. The combining order is
// fixed, so results are deterministic run to run.
// ---------------------------------------------------------------------------
struct OpMax {
  __device__ __forceinline__ float operator()(float a, float b) const {
    return fmaxf(a, b);
  }
};
struct OpAdd {
  __device__ __forceinline__ float operator()(float a, float b) const {
    return a + b;
  }
};

template <int kCtrl>
__device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), kCtrl,
                                         0xf, 0xf, false));
}

template <typename Op>
__device__ __forceinline__ float wave_allreduce(float v, Op op) {
  v = op(v, dpp_move<0xB1>(v));  // quad_perm [1,0,3,2] : lane ^ 1
  v = op(v, dpp_move<0x4E>(v));  // quad_perm [2,3,0,1] : lane ^ 2
  v = op(v, dpp_move<0x141>(v)); // row_half_mirror     : other quad of 8
  v = op(v, dpp_move<0x140>(v)); // row_mirror          : other half of 16
  v = op(v, __builtin_bit_cast(
                float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v),
                                                   0x401F))); // lane ^ 16
  const float lo = __builtin_bit_cast(
      float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
  const float hi = __builtin_bit_cast(
      float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32));
  return op(lo, hi);
}

// ---------------------------------------------------------------------------
// Host side: status + per-thread error text.
// ---------------------------------------------------------------------------
int fail(int status, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
int check_launch(const char *what);

inline bool aligned16(const void *p) {
  return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

#define OSLO_DISPATCH_DTYPE(dtype, ...)                                   \
  switch (dtype) {                                                        \
  case OSLO_F32: {                                                        \
    using T = float;                                                      \
    __VA_ARGS__;                                                          \
  } break;                                                                \
  case OSLO_F16: {                                                        \
    using T = ::oslo::f16;                                                \
    __VA_ARGS__;                                                          \
  } break;                                                                \
  case OSLO_BF16: {                                                       \
    using T = ::oslo::bf16;                                               \
    __VA_ARGS__;                                                          \
  } break;                                                                \
  default:                                                                \
    return ::oslo::fail(OSLO_E_BAD_ARG, "unknown dtype %d", (int)(dtype)); \
  }

} // namespace oslo
