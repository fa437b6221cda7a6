// NVFP4-style KV-cache write (e2m1 values, one e4m3 scale per 16 elements), gfx950.
//
// Replaces reshape_and_cache_flash_fp4 (csrc/custom_ops/reshape_and_cache_flash_fp4.cu:104-337
// in the reference).  One lane owns one group of 16 consecutive elements: two
// 16-byte loads, the group maximum, the e4m3 scale (v_cvt_pk_fp8_f32), the
// reciprocal of the decoded scale and eight v_cvt_scalef32_pk_fp4_f32 (two values
// each, round to nearest even, saturating) - no cross-lane traffic.  Consecutive
// lanes take consecutive groups of a token's K row, then its V row, so a wave
// reads 2 KiB and writes 512 B of packed values plus 64 scale bytes, all contiguous
// (NHD) or contiguous per head (HND).
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>


#include <cstdint>

#include "common.hpp"

namespace arctic {

struct Fp4Params {
  const char *key;
  const char *value;
  uint8_t *key_cache;
  uint8_t *value_cache;
  uint8_t *key_scale_cache;
  uint8_t *value_scale_cache;
  const int64_t *slot_mapping;
  int64_t key_stride_bytes;
  int64_t value_stride_bytes;
  int64_t block_stride;  // bytes of packed cache; the scale cache uses these / 8
  int64_t page_stride;
  int64_t head_stride;
  int64_t total_groups;  // num_tokens * 2 * num_heads * groups_per_head
  int64_t num_slots;     // slots at or beyond this move nothing
  int num_heads;
  int groups_per_head;   // head_size / 16
  int block_size;
};

// One group of 16 elements per lane, single-wave workgroups: a wave's 64 lanes stay on 64 consecutive groups (2 KiB
// of source, 512 bytes of packed cache).
constexpr int kFp4Lanes = 64;

template <typename T>
__global__ __launch_bounds__(kFp4Lanes) void kv_write_fp4_kernel(const Fp4Params p) {
  const int groups_per_row = p.num_heads * p.groups_per_head;
  // the slot is requested first and the group's 32 bytes right behind it: their address does not depend on the slot,
  // so one round trip to memory serves both (a padding token throws its group away)
  const int64_t idx = (int64_t)blockIdx.x * kFp4Lanes + threadIdx.x;
  const int64_t at_group = min(idx, p.total_groups - 1);   // lanes past the end read the last group and drop it
  const int64_t row = at_group / groups_per_row;           // token * 2 + (0 = K, 1 = V)
  const int in_row = (int)(at_group - row * groups_per_row);
  const int64_t token = row >> 1;
  const int64_t slot = p.slot_mapping[token];
  const char *src = ((row & 1) ? p.value + token * p.value_stride_bytes : p.key + token * p.key_stride_bytes) +
                    (int64_t)in_row * 32;
  const uint4 lo = load16_stream(src);
  const uint4 hi = load16_stream(src + 16);
  __builtin_amdgcn_sched_barrier(0);   // keeps the loads above the tests of the slot
  if (idx >= p.total_groups) return;
  if (slot < 0 || slot >= p.num_slots) return;  // padding token, or a slot outside the cache
  const int head = in_row / p.groups_per_head;
  const int group = in_row - head * p.groups_per_head;
  const bool is_v = row & 1;
  const int64_t blk = slot / p.block_size;
  const int64_t off = slot - blk * p.block_size;

  float x[16];
  {
    float a[8], b[8];
    unpack8<T>(lo, a);
    unpack8<T>(hi, b);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      x[j] = a[j];
      x[8 + j] = b[j];
    }
  }
  float amax = 0.f;
#pragma unroll
  for (int j = 0; j < 16; ++j) amax = fmaxf(amax, fabsf(x[j]));  // a NaN never becomes the maximum

  // scale = e4m3(amax / 6), saturating; SF = the value that byte decodes to
  const float sf = __builtin_amdgcn_fmed3f(amax * 0.16666667163372039794921875f, 0.0f, 448.0f);
  const uint32_t code = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(sf, 0.0f, 0, false) & 0xffu;
  const float SF = __builtin_amdgcn_cvt_f32_fp8((int)code, 0);
  const float inv = (SF != 0.0f) ? 1.0f / SF : 0.0f;

  uint32_t w0 = 0, w1 = 0;
  w0 = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w0, x[0] * inv, x[1] * inv, 1.0f, 0);
  w0 = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w0, x[2] * inv, x[3] * inv, 1.0f, 1);
  w0 = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w0, x[4] * inv, x[5] * inv, 1.0f, 2);
  w0 = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w0, x[6] * inv, x[7] * inv, 1.0f, 3);
  w1 = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w1, x[8] * inv, x[9] * inv, 1.0f, 0);
  w1 = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w1, x[10] * inv, x[11] * inv, 1.0f, 1);
  w1 = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w1, x[12] * inv, x[13] * inv, 1.0f, 2);
  w1 = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w1, x[14] * inv, x[15] * inv, 1.0f, 3);

  uint8_t *cache = is_v ? p.value_cache : p.key_cache;
  uint8_t *scales = is_v ? p.value_scale_cache : p.key_scale_cache;
  const int64_t at = blk * p.block_stride + off * p.page_stride + (int64_t)head * p.head_stride;
  const int64_t sat = blk * (p.block_stride / 8) + off * (p.page_stride / 8) + (int64_t)head * (p.head_stride / 8);
  store8_stream(cache + at + (int64_t)group * 8, make_uint2(w0, w1));
  ((ARCTIC_GLOBAL uint8_t *)scales)[sat + group] = (uint8_t)code;
}

}  // namespace arctic

using namespace arctic;

extern "C" int arctic_reshape_and_cache_flash_fp4(
    const void *key, const void *value, int64_t key_stride, int64_t value_stride, void *key_cache,
    void *value_cache, void *key_scale_cache, void *value_scale_cache, const int64_t *slot_mapping,
    int64_t num_tokens, int num_heads, int head_size, int block_size, int64_t block_stride,
    int64_t page_stride, int64_t head_stride, int64_t num_blocks, int dtype, void *stream) {
  const char *fn = "reshape_and_cache_flash_fp4";
  if (dtype != ARCTIC_DTYPE_F16 && dtype != ARCTIC_DTYPE_BF16)
    return fail(ARCTIC_ERR_UNSUPPORTED,
                "Unsupported input dtype for reshape_and_cache_fp4. Must be half or bfloat16.");
  if (num_tokens == 0) return ARCTIC_OK;
  if (num_tokens < 0 || num_heads <= 0 || head_size <= 0 || block_size <= 0)
    return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: sizes must be positive", fn);
  if (head_size % 16)
    return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: head_size must be a multiple of 16 (one scale per 16 elements)", fn);
  if (num_tokens > 0x7fffffffLL || (int64_t)num_heads * head_size > (1 << 24) || block_size > (1 << 20) ||
      num_blocks < 0 || num_blocks > ((int64_t)1 << 40))
    return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: num_tokens beyond 2^31, num_heads*head_size beyond 2^24, block_size beyond "
                "2^20 or num_blocks outside [0, 2^40]", fn);
  if (!pitch_ok(key_stride, num_tokens, 2) || !pitch_ok(value_stride, num_tokens, 2) ||
      !pitch_ok(block_stride, num_blocks, 1) || !pitch_ok(page_stride, block_size, 1) ||
      !pitch_ok(head_stride, num_heads, 1))
    return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: row, block, page or head pitch out of range", fn);
  if (!key || !value || !key_cache || !value_cache || !key_scale_cache || !value_scale_cache || !slot_mapping)
    return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: null tensor pointer", fn);
  if (((uintptr_t)key | (uintptr_t)value) & 15 || (num_tokens > 1 && ((key_stride | value_stride) & 7)))
    return fail(ARCTIC_ERR_UNSUPPORTED, "%s: key/value rows must be 16-byte aligned", fn);
  if (((uintptr_t)key_cache | (uintptr_t)value_cache | (uintptr_t)block_stride | (uintptr_t)page_stride |
       (uintptr_t)head_stride) & 7)
    return fail(ARCTIC_ERR_UNSUPPORTED, "%s: cache pointers and strides must be multiples of 8 bytes", fn);
  Fp4Params p;
  p.key = (const char *)key;
  p.value = (const char *)value;
  p.key_cache = (uint8_t *)key_cache;
  p.value_cache = (uint8_t *)value_cache;
  p.key_scale_cache = (uint8_t *)key_scale_cache;
  p.value_scale_cache = (uint8_t *)value_scale_cache;
  p.slot_mapping = slot_mapping;
  p.key_stride_bytes = key_stride * 2;
  p.value_stride_bytes = value_stride * 2;
  p.block_stride = block_stride;
  p.page_stride = page_stride;
  p.head_stride = head_stride;
  p.num_heads = num_heads;
  p.groups_per_head = head_size / 16;
  p.block_size = block_size;
  p.total_groups = num_tokens * 2 * num_heads * p.groups_per_head;
  p.num_slots = num_blocks > 0 ? num_blocks * (int64_t)block_size : INT64_MAX;
  hipStream_t s = (hipStream_t)stream;
  // One group per lane in workgroups of one wave: nothing is shared between lanes, and at 8192 tokens and beyond
  // single-wave workgroups ran 1 to 1.5 % faster than 256-lane ones (equal below); 512 and 1024 lanes and two or
  // four groups per lane all measured slower.
  const int64_t grid = (p.total_groups + kFp4Lanes - 1) / kFp4Lanes;
  if (grid > 0x7fffffffLL) return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: too many tokens", fn);
  if (dtype == ARCTIC_DTYPE_BF16)
    hipLaunchKernelGGL((kv_write_fp4_kernel<BF16>), dim3((unsigned)grid), dim3(kFp4Lanes), 0, s, p);
  else
    hipLaunchKernelGGL((kv_write_fp4_kernel<F16>), dim3((unsigned)grid), dim3(kFp4Lanes), 0, s, p);
  return check_launch(fn);
}
