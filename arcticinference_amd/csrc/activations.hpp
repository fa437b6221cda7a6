// sigmoid and GELU of the speculator operators on gfx950's transcendental unit.
#pragma once
#include <hip/hip_runtime.h>

namespace arctic {

// sigmoid_f / gelu_erf / gelu_tanh of the reference (sum_lstm.cu:14-26), built on
// the hardware exp2 and reciprocal instructions (1 ulp each) instead of library
// calls: per output element the operator needs three sigmoids and two GELUs, and
// with library expf / erff / IEEE division the arithmetic alone would take longer
// than moving the row through HBM.
__device__ __forceinline__ float fast_exp(float x) {            // e^x
  return __builtin_amdgcn_exp2f(x * 1.4426950408889634f);
}
__device__ __forceinline__ float sigmoid_f(float x) {
  return __builtin_amdgcn_rcpf(1.0f + fast_exp(-x));
}
// gelu(x) = x * Phi(x) with Phi from Abramowitz & Stegun 7.1.26
//   erfc(z) = (a1 t + ... + a5 t^5) exp(-z^2),  t = 1 / (1 + 0.3275911 z),  z >= 0
// (|error| <= 1.5e-7, the level of fp32 rounding).  With z = |x| / sqrt(2) and
// q = erfc(z) / 2:   gelu(x) = x - x q  for x >= 0  and  x q  for x < 0,
// i.e. max(x, 0) - |x| q.  One reciprocal and one exp2 per value.
__device__ __forceinline__ float gelu_erf(float x) {
  const float ax = fabsf(x);
  const float t = __builtin_amdgcn_rcpf(fmaf(0.3275911f * 0.70710678118654752440f, ax, 1.0f));
  float poly = fmaf(0.5f * 1.061405429f, t, 0.5f * -1.453152027f);
  poly = fmaf(poly, t, 0.5f * 1.421413741f);
  poly = fmaf(poly, t, 0.5f * -0.284496736f);
  poly = fmaf(poly, t, 0.5f * 0.254829592f);
  poly *= t;
  const float q = poly * __builtin_amdgcn_exp2f((x * (-0.5f * 1.4426950408889634f)) * x);
  return fmaf(-ax, q, fmaxf(x, 0.0f));
}
__device__ __forceinline__ float gelu_tanh(float x) {
  // 0.5 x (1 + tanh(u)) = x * sigmoid(2u),  u = sqrt(2/pi) (x + 0.044715 x^3)
  const float u = 0.79788456080286535588f * fmaf(0.044715f * x * x, x, x);
  return x * sigmoid_f(2.0f * u);
}
template <bool kFastGelu>
__device__ __forceinline__ float gelu(float x) {
  return kFastGelu ? gelu_tanh(x) : gelu_erf(x);
}

}  // namespace arctic
