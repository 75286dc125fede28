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

// Loads N consecutive elements (address aligned to N*sizeof(T)) as fp32 through
// the caches: for small operands reused by many rows (bias vectors, tables).
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

// Raw (unconverted) vector access. Kernels issue every load of a thread into
// raw registers first and convert afterwards: a load whose result is consumed
// inside the same conditional block makes the compiler wait for it before the
// next load is issued, which serialises the loads of a wave.
template <typename T, int N>
using RawVec = typename VecOf<T, N>::type;

template <typename T, int N>
__device__ __forceinline__ void raw_to_f32(float (&dst)[N],
                                           const RawVec<T, N> &v) {
  if constexpr (N == 1) {
    dst[0] = static_cast<float>(v);
  } else {
#pragma unroll
    for (int i = 0; i < N; ++i) dst[i] = static_cast<float>(v[i]);
  }
}

// Bounded loads through a buffer descriptor: a lane whose byte offset is at or
// past `bytes` gets zeros and produces no memory request, so ragged edges (the
// diagonal of a causal row, the last rows of a tile) need no branch around the
// load and all loads of a wave are issued back to back. The descriptor must be
// wave-uniform; `bytes` must be a multiple of the access size so that every
// access is wholly inside or wholly outside.
using BufRsrc = __amdgpu_buffer_rsrc_t;

__device__ __forceinline__ BufRsrc make_rsrc(const void *base, uint32_t bytes) {
  // word 3 = 0x00020000: raw 32-bit data format, no swizzle (gfx9 layout)
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0,
                                           (int)bytes, 0x00020000);
}

// NT sets the non-temporal bit of the cache policy (bit 1 on gfx94x/gfx950).
// When the first use of a loaded value sits in a conditional block, follow the
// loads with pin_loaded(): otherwise the optimiser sinks each load into that
// block, next to a wait, and the loads of a wave are serialised again.
template <typename T, int N, bool NT>
__device__ __forceinline__ RawVec<T, N> buffer_load_raw(BufRsrc rs,
                                                        uint32_t byte_offset) {
  using V = RawVec<T, N>;
  typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
  constexpr int kAux = NT ? 2 : 0;
  if constexpr (sizeof(V) == 16) {
    return __builtin_bit_cast(
        V, __builtin_amdgcn_raw_buffer_load_b128(rs, byte_offset, 0, kAux));
  } else if constexpr (sizeof(V) == 32) {
    struct Pair {
      u32x4 lo, hi;
    } p;
    p.lo = __builtin_amdgcn_raw_buffer_load_b128(rs, byte_offset, 0, kAux);
    p.hi = __builtin_amdgcn_raw_buffer_load_b128(rs, byte_offset + 16, 0, kAux);
    return __builtin_bit_cast(V, p);
  } else if constexpr (sizeof(V) == 8) {
    return __builtin_bit_cast(
        V, __builtin_amdgcn_raw_buffer_load_b64(rs, byte_offset, 0, kAux));
  } else if constexpr (sizeof(V) == 4) {
    return __builtin_bit_cast(
        V, __builtin_amdgcn_raw_buffer_load_b32(rs, byte_offset, 0, kAux));
  } else {
    static_assert(sizeof(V) == 2, "unsupported vector size");
    return __builtin_bit_cast(
        V, __builtin_amdgcn_raw_buffer_load_b16(rs, byte_offset, 0, kAux));
  }
}

// An empty asm statement that "uses and redefines" the N raw vectors: every
// load that produces them has to be issued before it and cannot be moved past
// it. (The compiler also waits here for all of them; the waves of the other
// rows cover that.)
template <typename V, int N>
__device__ __forceinline__ void pin_loaded(V (&raw)[N]) {
#pragma unroll
  for (int i = 0; i < N; ++i) asm volatile("" : "+v"(raw[i]));
}

// Store N fp32 values as T through a buffer descriptor (offsets at or past the
// bound are dropped). kStreamOut = sc1 + nt: write-through at device scope,
// non-temporal; on the softmax rows it measured 2-3 % faster than nt alone and
// 6 % faster than the default policy.
constexpr int kStreamOut = 16 | 2;

template <typename T, int N, int AUX>
__device__ __forceinline__ void buffer_store_f32(BufRsrc rs, uint32_t byte_offset,
                                                 const float (&src)[N]) {
  using V = RawVec<T, N>;
  typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
  V v;
  if constexpr (N == 1) {
    v = static_cast<T>(src[0]);
  } else {
#pragma unroll
    for (int i = 0; i < N; ++i) v[i] = static_cast<T>(src[i]);
  }
  if constexpr (sizeof(V) == 16) {
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), rs,
                                           byte_offset, 0, AUX);
  } else if constexpr (sizeof(V) == 4) {
    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned int, v),
                                          rs, byte_offset, 0, AUX);
  } else {
    static_assert(sizeof(V) == 2, "unsupported vector size");
    __builtin_amdgcn_raw_buffer_store_b16(__builtin_bit_cast(unsigned short, v),
                                          rs, byte_offset, 0, AUX);
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

// Sum over the 16 lanes of a DPP row (lane / 16 equal), left in every one of
// them: four DPP steps in the vector ALU, the first four of wave_allreduce. A
// ds_bpermute shuffle would take each value through the LDS crossbar instead.
__device__ __forceinline__ float sum_over_row(float v) {
  v += dpp_move<0xB1>(v);  // lane ^ 1
  v += dpp_move<0x4E>(v);  // lane ^ 2
  v += dpp_move<0x141>(v); // row_half_mirror: the other quad of 8
  v += dpp_move<0x140>(v); // row_mirror: the other half of 16
  return v;
}

// Sum over an aligned group of N lanes (N = 8, 16, 32 or 64), left in every
// lane of the group: DPP inside a row of 16, one ds_swizzle for lane ^ 16, two
// v_readlane for the halves of the wave (the steps of wave_allreduce).
template <int N>
__device__ __forceinline__ float sum_over_lanes(float v) {
  static_assert(N == 8 || N == 16 || N == 32 || N == 64, "aligned lane groups");
  if constexpr (N == 64) {
    return wave_allreduce(v, OpAdd());
  } else {
    v += dpp_move<0xB1>(v);
    v += dpp_move<0x4E>(v);
    v += dpp_move<0x141>(v);
    if constexpr (N >= 16) v += dpp_move<0x140>(v);
    if constexpr (N >= 32)
      v += __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F));
    return v;
  }
}

// ---------------------------------------------------------------------------
// Host side: status + per-thread error text.
// ---------------------------------------------------------------------------
int fail(int status, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
int check_launch(const char *what);
// Lets `kernel` ask for `bytes` of dynamic LDS (more than the 64 KiB a kernel
// gets unasked) on the current device. A host-side setting of the kernel, made
// once per kernel and device and remembered, not per launch.
int raise_lds_limit(const void *kernel, unsigned bytes, const char *what);

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
