// Scaled conversion to OCP fp8 with the reference's semantics
// (csrc/custom_ops/quant_utils.cuh:456-489,515-526):
//     code = cvt_float_to_fp8(float(x) / scale, SATFINITE, E4M3 | E5M2)
// i.e. an IEEE fp32 division, then round-to-nearest-even into the 8-bit format,
// with everything above the largest finite value (and +-inf) saturating to it.
//
// Exact division without the division instruction sequence
// ---------------------------------------------------------
// The scale is one number per (layer, K|V), so its reciprocal is computed once,
// in fp64, and each element costs  cvt_f64_f32 . mul_f64 . cvt_f32_f64.
// This reproduces RN32(x / s) bit for bit: with y = RN64(1/s), p = RN64(x*y)
// differs from q = x/s by less than 2^-52 relative, while the quotient of two
// numbers with at most 24 significant bits is further than 2^-49 relative from
// every midpoint between adjacent fp32 values, so p and q lie strictly between
// the same pair of rounding boundaries and round to the same fp32 value.
// Zero, infinite, NaN, negative and subnormal scales need no special case: fp64
// holds 1/s for every fp32 s, and 0*inf / inf*0 give the NaN that 0/0 and
// inf/inf give.  (Results in the fp32 subnormal range may round differently, but
// every such value encodes to fp8 zero.)
#pragma once

#include "common.hpp"

namespace arctic {

struct E4M3 {
  static constexpr float kMax = 448.0f;
  __device__ static __forceinline__ uint32_t cvt_pk(float a, float b, uint32_t old, bool hi) {
    // v_cvt_pk_fp8_f32: two fp32 -> two OCP e4m3fn codes (RNE) into the low or
    // high half of `old`.
    return hi ? (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, (int)old, true)
              : (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, (int)old, false);
  }
};

struct E5M2 {
  static constexpr float kMax = 57344.0f;
  __device__ static __forceinline__ uint32_t cvt_pk(float a, float b, uint32_t old, bool hi) {
    return hi ? (uint32_t)__builtin_amdgcn_cvt_pk_bf8_f32(a, b, (int)old, true)
              : (uint32_t)__builtin_amdgcn_cvt_pk_bf8_f32(a, b, (int)old, false);
  }
};

// RN32(x / s) given inv = RN64(1 / (double)s).
__device__ __forceinline__ float div_by_scale(float x, double inv) {
  return (float)((double)x * inv);
}

// Four quotients -> four codes in one dword.  Finite quotients are clamped to
// the format's range first (the hardware conversion does not saturate by
// itself); a NaN quotient becomes 0x7F with its sign bit.
template <typename F8>
__device__ __forceinline__ uint32_t encode4(float q0, float q1, float q2, float q3) {
  const float c0 = __builtin_amdgcn_fmed3f(q0, -F8::kMax, F8::kMax);
  const float c1 = __builtin_amdgcn_fmed3f(q1, -F8::kMax, F8::kMax);
  const float c2 = __builtin_amdgcn_fmed3f(q2, -F8::kMax, F8::kMax);
  const float c3 = __builtin_amdgcn_fmed3f(q3, -F8::kMax, F8::kMax);
  uint32_t w = F8::cvt_pk(c0, c1, 0u, false);
  w = F8::cvt_pk(c2, c3, w, true);
  // One unordered compare tests two quotients for NaN at once.
  if (__builtin_expect(__builtin_isunordered(q0, q1) | __builtin_isunordered(q2, q3), 0)) {
    const float q[4] = {q0, q1, q2, q3};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      if (q[k] != q[k]) {
        const uint32_t code = 0x7fu | ((__float_as_uint(q[k]) >> 24) & 0x80u);
        w = (w & ~(0xffu << (8 * k))) | (code << (8 * k));
      }
    }
  }
  return w;
}

}  // namespace arctic
