// Shared device helpers for the gfx950 kernels: 16-bit float conversion,
// 16-byte vector access, wave64 DPP reductions and the error channel of the C ABI.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/arctic_mi355x.h"

namespace arctic {

// ---- error channel ---------------------------------------------------------
int fail(int code, const char *fmt, ...);
int check_launch(const char *what);

// A row pitch (in elements) that `rows` rows of a tensor inside a 2^47-byte address space can have: not negative,
// and the last row's byte offset stays inside that space, so that no product of the two formed later, on the host
// or in a kernel, overflows 64 bits.
inline bool pitch_ok(int64_t pitch_elems, int64_t rows, int elem_bytes) {
  if (pitch_elems < 0) return false;
  const int64_t limit = ((int64_t)1 << 47) / elem_bytes;
  return pitch_elems <= limit / (rows > 1 ? rows - 1 : 1);
}

// ---- 16-bit floats ---------------------------------------------------------
// Activation element types. to_float is exact; from_float rounds to nearest
// even (what __float2bfloat16 / __float2half do in the reference,
// csrc/custom_ops/dtype_common.cuh:13-35).
struct BF16 {
  static constexpr int kCode = ARCTIC_DTYPE_BF16;
  __device__ static __forceinline__ float lo(uint32_t w) {
    return __uint_as_float(w << 16);
  }
  __device__ static __forceinline__ float hi(uint32_t w) {
    return __uint_as_float(w & 0xffff0000u);
  }
  // gfx950 rounds fp32 pairs to bf16 in hardware (v_cvt_pk_bf16_f32, RNE)
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  __device__ static __forceinline__ uint32_t pack(float a, float b) {
    const f32x2 v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
  }
  __device__ static __forceinline__ uint32_t round_bits(float f) { return pack(f, 0.f) & 0xffffu; }
  // value of the rounded 16-bit number, as fp32
  __device__ static __forceinline__ float requant(float f) {
    return __uint_as_float(pack(f, 0.f) << 16);
  }
};

struct F16 {
  static constexpr int kCode = ARCTIC_DTYPE_F16;
  __device__ static __forceinline__ float lo(uint32_t w) {
    return __half2float(__ushort_as_half((unsigned short)(w & 0xffffu)));
  }
  __device__ static __forceinline__ float hi(uint32_t w) {
    return __half2float(__ushort_as_half((unsigned short)(w >> 16)));
  }
  __device__ static __forceinline__ uint32_t round_bits(float f) {
    return (uint32_t)__half_as_ushort(__float2half_rn(f));
  }
  __device__ static __forceinline__ uint32_t pack(float a, float b) {
    return round_bits(a) | (round_bits(b) << 16);
  }
  __device__ static __forceinline__ float requant(float f) {
    return __half2float(__float2half_rn(f));
  }
};

// Eight 16-bit elements (one 16-byte lane access) unpacked to fp32 and back.
template <typename T>
__device__ __forceinline__ void unpack8(const uint4 &v, float (&f)[8]) {
  f[0] = T::lo(v.x);
  f[1] = T::hi(v.x);
  f[2] = T::lo(v.y);
  f[3] = T::hi(v.y);
  f[4] = T::lo(v.z);
  f[5] = T::hi(v.z);
  f[6] = T::lo(v.w);
  f[7] = T::hi(v.w);
}

template <typename T>
__device__ __forceinline__ uint4 pack8(const float (&f)[8]) {
  uint4 v;
  v.x = T::pack(f[0], f[1]);
  v.y = T::pack(f[2], f[3]);
  v.z = T::pack(f[4], f[5]);
  v.w = T::pack(f[6], f[7]);
  return v;
}

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// Every tensor on these paths lives in device (global) memory.  Saying so keeps
// the compiler from falling back to flat_* instructions when a pointer has been
// round-tripped through LDS or a struct.
#define ARCTIC_GLOBAL __attribute__((address_space(1)))

__device__ __forceinline__ uint4 load16(const void *p) {
  const u32x4 v = *(const ARCTIC_GLOBAL u32x4 *)p;
  return make_uint4(v.x, v.y, v.z, v.w);
}
// streaming (non-temporal) variants: every byte on these paths is touched exactly once
__device__ __forceinline__ uint4 load16_stream(const void *p) {
  const u32x4 v = __builtin_nontemporal_load((const ARCTIC_GLOBAL u32x4 *)p);
  return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void store16_stream(void *p, const uint4 &v) {
  const u32x4 t = {v.x, v.y, v.z, v.w};
  __builtin_nontemporal_store(t, (ARCTIC_GLOBAL u32x4 *)p);
}
__device__ __forceinline__ void store16(void *p, const uint4 &v) {  // stays in the caches: read again soon
  const u32x4 t = {v.x, v.y, v.z, v.w};
  *(ARCTIC_GLOBAL u32x4 *)p = t;
}
__device__ __forceinline__ void store8_stream(void *p, const uint2 &v) {
  const u32x2 t = {v.x, v.y};
  __builtin_nontemporal_store(t, (ARCTIC_GLOBAL u32x2 *)p);
}
__device__ __forceinline__ void store4_stream(void *p, uint32_t v) {
  __builtin_nontemporal_store(v, (ARCTIC_GLOBAL uint32_t *)p);
}

// A lane's unit of work on the speculator paths: eight consecutive 16-bit elements
// moved with one 16-byte access (narrower units measured slower).
struct Chunk {
  static constexpr int kElems = 8;
  static constexpr int kBytes = 16;
  uint4 v;
  __device__ static __forceinline__ Chunk zero() { return Chunk{make_uint4(0, 0, 0, 0)}; }
  __device__ static __forceinline__ Chunk load(const void *p) { return Chunk{load16(p)}; }
  __device__ static __forceinline__ Chunk load_stream(const void *p) { return Chunk{load16_stream(p)}; }
  __device__ __forceinline__ void store_stream(void *p) const { store16_stream(p, v); }
  __device__ __forceinline__ void store(void *p) const { store16(p, v); }
  template <typename T>
  __device__ __forceinline__ void unpack(float (&f)[8]) const { unpack8<T>(v, f); }
  template <typename T>
  __device__ static __forceinline__ Chunk pack(const float (&f)[8]) { return Chunk{pack8<T>(f)}; }
};

// ---- wave64 / workgroup reductions ------------------------------------------
// DPP butterfly inside each row of 16 lanes, then the four row totals are read
// with v_readlane.  Every lane returns the same wave total.
template <int kCtrl>
__device__ __forceinline__ float dpp_add(float v) {
  int moved = __builtin_amdgcn_update_dpp(0, __float_as_int(v), kCtrl, 0xf, 0xf, true);
  return v + __int_as_float(moved);
}

__device__ __forceinline__ float wave_sum(float v) {
  v = dpp_add<0xB1>(v);   // quad_perm [1,0,3,2]
  v = dpp_add<0x4E>(v);   // quad_perm [2,3,0,1]
  v = dpp_add<0x141>(v);  // row_half_mirror
  v = dpp_add<0x140>(v);  // row_mirror
  const int b = __float_as_int(v);
  float r0 = __int_as_float(__builtin_amdgcn_readlane(b, 0));
  float r1 = __int_as_float(__builtin_amdgcn_readlane(b, 16));
  float r2 = __int_as_float(__builtin_amdgcn_readlane(b, 32));
  float r3 = __int_as_float(__builtin_amdgcn_readlane(b, 48));
  return (r0 + r1) + (r2 + r3);
}

// Sum over the whole workgroup (blockDim.x a multiple of 64, at most 1024 = 16
// waves).  `slots` is LDS for 16 floats, private to this call site.  Each wave
// leaves its total in slots[wave]; after the barrier every row of 16 lanes reads
// the 16 slots (zero beyond the last wave) and folds them with the same DPP
// butterfly, so all lanes of all waves end with the identical total and no loop
// or branch depends on the number of waves.
__device__ __forceinline__ float block_sum(float v, float *slots) {
  v = wave_sum(v);
  const int nwaves = blockDim.x >> 6;
  if (nwaves == 1) return v;
  const int lane = threadIdx.x & 63;
  if (lane == 0) slots[threadIdx.x >> 6] = v;
  __syncthreads();
  float t = ((lane & 15) < nwaves) ? slots[lane & 15] : 0.f;
  t = dpp_add<0xB1>(t);   // quad_perm [1,0,3,2]
  t = dpp_add<0x4E>(t);   // quad_perm [2,3,0,1]
  t = dpp_add<0x141>(t);  // row_half_mirror
  t = dpp_add<0x140>(t);  // row_mirror
  return t;
}

}  // namespace arctic
