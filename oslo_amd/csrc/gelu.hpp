// GeLU (tanh form) and its derivative in fp32, shared by the bias-GeLU kernels
// and the fused epilogue of the few-row linear layer. The arithmetic is that of
// bias_gelu_fwb / bias_gelu_bwd (oslo/fused_kernels_utils.py:295-308) rewritten
// around the identity 0.5*(1 + tanh(u)) = 1/(1 + exp(-2u)): one v_exp_f32 and
// one v_rcp_f32 per element.
#pragma once

#include "common.hpp"

namespace oslo {

// gelu_tanh(x) = x * s(x), s(x) = 1/(1 + exp(-2u)), u = K*x*(1 + A*x^2).
constexpr float kGeluK = 0.79788456f;
constexpr float kGeluA = 0.044715f;
constexpr float kLog2eF = 1.4426950408889634f;
// -2u*log2(e) = x * (kW0 + kW1*x^2)
constexpr float kW0 = -2.0f * kLog2eF * kGeluK;
constexpr float kW1 = kW0 * kGeluA;
// 2*du/dx = kD0 + kD1*x^2   (kD1 = 2*3*A*K; 3*A*K is the reference's 0.1070322243)
constexpr float kD0 = 2.0f * kGeluK;
constexpr float kD1 = 2.0f * 0.1070322243f;

// e = exp(-2u), clamped so that e stays finite (x below about -5.4 gives the
// clamp; the results there are 0 to within 2^-126).
__device__ __forceinline__ float exp_m2u(float x, float x2) {
  const float w = fminf(x * __builtin_fmaf(x2, kW1, kW0), 126.0f);
  return __builtin_amdgcn_exp2f(w);
}

__device__ __forceinline__ float gelu_fwd(float x) {
  const float e = exp_m2u(x, x * x);
  return x * __builtin_amdgcn_rcpf(1.0f + e);
}

// d/dx [x*s] = s + x*s*(1-s)*2u' with s = r = 1/(1+e) and 1-s = e*r: written
// as r + q*(e*r)*r so that no difference of nearly equal numbers is formed
// (the reference's 1 - tanh^2 loses about two digits in fp32 for |x| > 2).
__device__ __forceinline__ float gelu_grad(float x) {
  const float x2 = x * x;
  const float e = exp_m2u(x, x2);
  const float r = __builtin_amdgcn_rcpf(1.0f + e);
  const float q = x * __builtin_fmaf(x2, kD1, kD0);
  return __builtin_fmaf(q * (e * r), r, r);
}

} // namespace oslo
