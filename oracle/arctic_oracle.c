/*
 * CPU oracle for the ArcticInference csrc/custom_ops hot path.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  It is a plain-C restatement
 * of the arithmetic of the reference's CUDA kernels, used only as the checker
 * in tests/, in the smoke test and as the timed CPU baseline of the benchmark.
 * The shipped library never links, loads or calls anything in this file.
 *
 * Each function cites the reference lines it restates (paths relative to the
 * reference checkout).
 *
 * How each function is pinned (see tests/test_oracle_*.py):
 *   ao_f32_to_e4m3fn / ao_f32_to_e5m2   exhaustive over all 65 536 bf16 and fp16
 *        bit patterns x several scales against torch's CPU float8 cast (an
 *        independent table-free implementation), every rounding midpoint +-1 ulp,
 *        decode(encode(v)) == v for all finite codes, monotonicity.
 *        NaN sign/payload: parity unpinned (the reference delegates to the CUDA
 *        toolkit's __nv_cvt_float_to_fp8, which is not part of the reference
 *        tree); this file keeps the sign and emits 0x7F/0xFF like torch does.
 *   ao_reshape_and_cache_flash_bulk     closed form == torch index_copy_ per
 *        layer; sentinel-filled caches prove untouched rows stay untouched.
 *   ao_speculator_ln / ao_sum_lstm      torch fp32 closed forms (rsqrt, mean,
 *        sigmoid, gelu) and algebraic invariants / degenerate cases.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define AO_F32 0
#define AO_F16 1
#define AO_BF16 2

#define AO_KV_AUTO 0
#define AO_KV_FP8_E4M3 1
#define AO_KV_FP8_E5M2 2

static inline uint32_t f32_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}
static inline float bits_f32(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* ---- 16-bit float <-> fp32 (csrc/custom_ops/dtype_common.cuh:13-64) ------ */

/* bf16 -> fp32 is exact: the bf16 bits are the top half of the fp32 bits
 * (dtype_common.cuh:21-30). */
float ao_bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

/* fp32 -> bf16, round to nearest even, as __float2bfloat16 does
 * (dtype_common.cuh:32-35; the truncating branch :36-40 is compiled out in the
 * default build).  NaN maps to the canonical quiet NaN 0x7FFF. */
uint16_t ao_f32_to_bf16(float f) {
  uint32_t u = f32_bits(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fff;
  uint32_t lsb = (u >> 16) & 1u;
  u += 0x7fffu + lsb;
  return (uint16_t)(u >> 16);
}

/* fp16 -> fp32, exact (__half2float, dtype_common.cuh:13-15). */
float ao_f16_to_f32(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t e = (h >> 10) & 0x1fu;
  uint32_t m = h & 0x3ffu;
  if (e == 0x1f) return bits_f32(sign | 0x7f800000u | (m << 13));
  if (e == 0) {
    if (m == 0) return bits_f32(sign);
    /* subnormal: m * 2^-24 */
    float v = (float)m * (1.0f / 16777216.0f);
    return bits_f32(f32_bits(v) | sign);
  }
  return bits_f32(sign | ((e + 112u) << 23) | (m << 13));
}

/* fp32 -> fp16, round to nearest even (__float2half, dtype_common.cuh:17-19). */
uint16_t ao_f32_to_f16(float f) {
  uint32_t u = f32_bits(f);
  uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
  uint32_t a = u & 0x7fffffffu;
  if (a > 0x7f800000u) return (uint16_t)(sign | 0x7fffu);
  if (a >= 0x47800000u) { /* >= 65536 -> inf (65520 rounds up too, below) */
    return (uint16_t)(sign | 0x7c00u);
  }
  int e = (int)(a >> 23) - 127;
  uint32_t m = (a & 0x7fffffu) | 0x800000u;
  int shift = 13 + (e < -14 ? -14 - e : 0);
  if (shift > 24) return sign;
  uint32_t q = m >> shift;
  uint32_t rem = m & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1);
  if (rem > half || (rem == half && (q & 1u))) q++;
  uint32_t code;
  if (e >= -14)
    code = ((uint32_t)(e + 15 - 1) << 10) + q;
  else
    code = q;
  return (uint16_t)(sign | code); /* carries into the exponent, up to inf */
}

static inline float load_as_f32(const void *p, int64_t i, int dtype) {
  switch (dtype) {
  case AO_F32:
    return ((const float *)p)[i];
  case AO_F16:
    return ao_f16_to_f32(((const uint16_t *)p)[i]);
  default:
    return ao_bf16_to_f32(((const uint16_t *)p)[i]);
  }
}

static inline uint16_t store_half(float v, int dtype) {
  return dtype == AO_F16 ? ao_f32_to_f16(v) : ao_f32_to_bf16(v);
}

/* value of v after a round trip through the 16-bit type */
static inline float requant(float v, int dtype) {
  return dtype == AO_F16 ? ao_f16_to_f32(ao_f32_to_f16(v)) : ao_bf16_to_f32(ao_f32_to_bf16(v));
}

/* ---- fp8 encode / decode --------------------------------------------------
 * The reference's scaled_vec_conversion<uint8_t, *> ends in
 *   __nv_cvt_float_to_fp8(x / scale, __NV_SATFINITE, __NV_E4M3 | __NV_E5M2)
 * (csrc/custom_ops/quant_utils.cuh:456-489).  That primitive rounds to nearest
 * even into the OCP format and, with SATFINITE, maps everything above the
 * largest finite value (including +-inf) to that largest finite value.
 */
static uint8_t f32_to_fp8_satfinite(float f, int mbits, int bias,
                                    uint8_t maxcode, float maxval) {
  uint32_t u = f32_bits(f);
  uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
  uint32_t a = u & 0x7fffffffu;
  if (a > 0x7f800000u) return (uint8_t)(sign | 0x7fu); /* NaN */
  if (bits_f32(a) > maxval) return (uint8_t)(sign | maxcode);
  int e = (int)(a >> 23) - 127;
  uint32_t m = (a & 0x7fffffu) | 0x800000u;
  int emin = 1 - bias;
  int shift = 23 - mbits + (e < emin ? emin - e : 0);
  if (shift > 24) return sign; /* below half of the smallest subnormal */
  uint32_t q = m >> shift;
  uint32_t rem = m & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1);
  if (rem > half || (rem == half && (q & 1u))) q++;
  uint32_t code;
  if (e >= emin)
    code = ((uint32_t)(e + bias - 1) << mbits) + q;
  else
    code = q;
  return (uint8_t)(sign | code);
}

uint8_t ao_f32_to_e4m3fn(float f) {
  return f32_to_fp8_satfinite(f, 3, 7, 0x7e, 448.0f);
}
uint8_t ao_f32_to_e5m2(float f) {
  return f32_to_fp8_satfinite(f, 2, 15, 0x7b, 57344.0f);
}

/* e4m3fn decode: restates decode_fp8_e4m3 of the reference's own test
 * (tests/unit_tests/test_reshape_and_cache_flash_nvfp4.py:25-45): bias 7,
 * exponent field 0 = subnormal (m/8 * 2^-6), no infinities, 0x7F/0xFF = NaN. */
float ao_e4m3fn_to_f32(uint8_t c) {
  int s = c >> 7, e = (c >> 3) & 0xf, m = c & 7;
  float v;
  if (e == 0xf && m == 7)
    v = NAN;
  else if (e == 0)
    v = ldexpf((float)m / 8.0f, -6);
  else
    v = ldexpf(1.0f + (float)m / 8.0f, e - 7);
  return s ? -v : v;
}

float ao_e5m2_to_f32(uint8_t c) {
  int s = c >> 7, e = (c >> 2) & 0x1f, m = c & 3;
  float v;
  if (e == 0x1f)
    v = m ? NAN : INFINITY;
  else if (e == 0)
    v = ldexpf((float)m / 4.0f, -14);
  else
    v = ldexpf(1.0f + (float)m / 4.0f, e - 15);
  return s ? -v : v;
}

/* fp8::scaled_convert (quant_utils.cuh:515-526): code = cvt(float(x) / scale).
 * The division is a true IEEE fp32 division (the CMake build has no fast-math).
 */
static inline uint8_t scaled_convert_one(float x, float scale, int kv_dtype) {
  volatile float q = x / scale; /* volatile: keep the fp32 rounding of the quotient */
  return kv_dtype == AO_KV_FP8_E5M2 ? ao_f32_to_e5m2(q) : ao_f32_to_e4m3fn(q);
}

void ao_scaled_convert(const void *src, uint8_t *dst, int64_t count,
                       float scale, int src_dtype, int kv_dtype) {
  for (int64_t i = 0; i < count; ++i)
    dst[i] = scaled_convert_one(load_as_f32(src, i, src_dtype), scale, kv_dtype);
}

static int elem_size(int dtype) { return dtype == AO_F32 ? 4 : 2; }

/* ---- Part A: bulk KV-cache write ------------------------------------------
 * Restates reshape_and_cache_flash_bulk_kernel
 * (csrc/custom_ops/reshape_and_cache_flash_bulk.cu:12-60) and the shape/stride
 * handling of its host launcher (:85-102):
 *   for every layer l and token t with slot = slot_mapping[t] >= 0:
 *     blk = slot / block_size, off = slot % block_size
 *     cache_l[blk*block_stride + off*n + i] = cvt(src[t*stride + l*n + i]),  i < n
 * with n = num_heads*head_size; cvt is the identity for "auto" and
 * scaled_convert(x, *scale_l) otherwise.  Slots < 0 are padding: skipped.
 * Strides are in elements.  Returns 0, or -1 for an unsupported dtype pair.
 */
int ao_reshape_and_cache_flash_bulk(
    const void *keys, const void *values, int64_t key_stride,
    int64_t value_stride, void *const *key_cache_ptrs,
    void *const *value_cache_ptrs, const float *const *k_scale_ptrs,
    const float *const *v_scale_ptrs, const int64_t *slot_mapping,
    int64_t num_tokens, int num_layers, int num_heads, int head_size,
    int block_size, int64_t block_stride, int src_dtype, int kv_dtype) {
  if (src_dtype < 0 || src_dtype > 2 || kv_dtype < 0 || kv_dtype > 2) return -1;
  const int64_t n = (int64_t)num_heads * head_size;
  const int es = elem_size(src_dtype);
#pragma omp parallel for schedule(static)
  for (int64_t t = 0; t < num_tokens; ++t) {
    const int64_t slot = slot_mapping[t];
    if (slot < 0) continue;
    const int64_t blk = slot / block_size;
    const int64_t off = slot % block_size;
    const int64_t dst0 = blk * block_stride + off * n;
    for (int l = 0; l < num_layers; ++l) {
      const int64_t ks = t * key_stride + (int64_t)l * n;
      const int64_t vs = t * value_stride + (int64_t)l * n;
      if (kv_dtype == AO_KV_AUTO) {
        memcpy((char *)key_cache_ptrs[l] + dst0 * es,
               (const char *)keys + ks * es, (size_t)(n * es));
        memcpy((char *)value_cache_ptrs[l] + dst0 * es,
               (const char *)values + vs * es, (size_t)(n * es));
      } else {
        const float k_scale = *k_scale_ptrs[l];
        const float v_scale = *v_scale_ptrs[l];
        uint8_t *kc = (uint8_t *)key_cache_ptrs[l] + dst0;
        uint8_t *vc = (uint8_t *)value_cache_ptrs[l] + dst0;
        for (int64_t i = 0; i < n; ++i) {
          kc[i] = scaled_convert_one(load_as_f32(keys, ks + i, src_dtype),
                                     k_scale, kv_dtype);
          vc[i] = scaled_convert_one(load_as_f32(values, vs + i, src_dtype),
                                     v_scale, kv_dtype);
        }
      }
    }
  }
  return 0;
}

/* ---- next row: NVFP4-style KV-cache write ----------------------------------
 * Restates reshape_and_cache_flash_kernel_fp4 / quantize_16_to_fp4
 * (csrc/custom_ops/reshape_and_cache_flash_fp4.cu:104-147,150-254), sm_100 branch:
 * per group of 16 consecutive elements along head_size
 *   amax   = max |x|                                   (:115-121, NaN ignored by __hmax)
 *   sf     = amax * (1/6)                               (:122)
 *   scale  = e4m3(sf), stored as one byte; SF = float(scale)   (:124-128)
 *   inv    = SF != 0 ? 1/SF : 0                          (:131-132)
 *   nibble = e2m1(x * inv), round to nearest even, saturating at +-6 (:64-76)
 * two nibbles per byte, the first element in the low nibble (:88).
 * The reference takes both reciprocals with rcp.approx.ftz (<= 1 ulp from the
 * correctly rounded value); this restatement uses the correctly rounded ones, so
 * PARITY IS UNPINNED where that last ulp decides a rounding, and for NaN inputs
 * (PTX maps NaN to +6 there, the sm_90 fallback :36-38 to 0; here: +6).
 * k_scale / v_scale / kv_cache_dtype are accepted and ignored, as in the reference.
 * Strides are in bytes of the packed cache; the scale cache uses stride/8 (:185-187).
 */
uint8_t ao_f32_to_e2m1(float v) {
  uint32_t u = f32_bits(v);
  uint8_t sign = (uint8_t)((u >> 28) & 0x8u);
  float x = fabsf(v);
  uint8_t m;
  if (x != x) return 0x7; /* NaN */
  if (x > 5.0f) m = 7;           /* 6 */
  else if (x >= 3.5f) m = 6;     /* 4; 3.5 ties to even (4) */
  else if (x > 2.5f) m = 5;      /* 3; 2.5 ties to even (2) */
  else if (x >= 1.75f) m = 4;    /* 2 */
  else if (x > 1.25f) m = 3;     /* 1.5; 1.25 ties to even (1) */
  else if (x >= 0.75f) m = 2;    /* 1 */
  else if (x > 0.25f) m = 1;     /* 0.5; 0.25 ties to even (0) */
  else m = 0;
  return (uint8_t)(sign | m);
}

float ao_e2m1_to_f32(uint8_t c) {
  static const float lut[8] = {0.f, 0.5f, 1.f, 1.5f, 2.f, 3.f, 4.f, 6.f};
  float v = lut[c & 7];
  return (c & 8) ? -v : v;
}

/* One group of 16: writes 8 packed bytes and 1 scale byte. */
static void quantize_16_to_fp4(const void *src, int64_t first, int dtype, uint8_t *dst, uint8_t *scale_dst) {
  float x[16];
  float amax = 0.f;
  for (int i = 0; i < 16; ++i) {
    x[i] = load_as_f32(src, first + i, dtype);
    float a = fabsf(x[i]);
    if (a > amax) amax = a; /* NaN never wins the comparison */
  }
  volatile float sixth = 1.0f / 6.0f;
  volatile float sf = amax * sixth;
  const uint8_t code = ao_f32_to_e4m3fn(sf);
  *scale_dst = code;
  const float SF = ao_e4m3fn_to_f32(code);
  volatile float inv = (SF != 0.0f) ? 1.0f / SF : 0.0f;
  for (int i = 0; i < 8; ++i) {
    volatile float a = x[2 * i] * inv, b = x[2 * i + 1] * inv;
    dst[i] = (uint8_t)((ao_f32_to_e2m1(b) << 4) | ao_f32_to_e2m1(a));
  }
}

int ao_reshape_and_cache_flash_fp4(const void *key, const void *value, int64_t key_stride, int64_t value_stride,
                                   uint8_t *key_cache, uint8_t *value_cache, uint8_t *key_scale_cache,
                                   uint8_t *value_scale_cache, const int64_t *slot_mapping, int64_t num_tokens,
                                   int num_heads, int head_size, int block_size, int64_t block_stride,
                                   int64_t page_stride, int64_t head_stride, int dtype) {
  if (dtype != AO_F16 && dtype != AO_BF16) return -1;
  if (head_size % 16) return -2;
  const int groups = head_size / 16;
#pragma omp parallel for schedule(static)
  for (int64_t t = 0; t < num_tokens; ++t) {
    const int64_t slot = slot_mapping[t];
    if (slot < 0) continue;
    const int64_t blk = slot / block_size, off = slot % block_size;
    for (int h = 0; h < num_heads; ++h) {
      const int64_t row = blk * block_stride + off * page_stride + (int64_t)h * head_stride;
      const int64_t srow = blk * (block_stride / 8) + off * (page_stride / 8) + (int64_t)h * (head_stride / 8);
      for (int g = 0; g < groups; ++g) {
        quantize_16_to_fp4(key, t * key_stride + (int64_t)h * head_size + g * 16, dtype, key_cache + row + g * 8,
                           key_scale_cache + srow + g);
        quantize_16_to_fp4(value, t * value_stride + (int64_t)h * head_size + g * 16, dtype,
                           value_cache + row + g * 8, value_scale_cache + srow + g);
      }
    }
  }
  return 0;
}

/* ---- Part B: speculator "LayerNorm" (an RMS norm) -------------------------
 * Restates spec_ln_vec_kernel / spec_ln_scalar_kernel
 * (csrc/custom_ops/speculator_ln.cu:21-150):
 *   ss = sum x^2 (fp32); inv = rsqrt(ss / hidden + eps)
 *   y = x * inv; if (w) y *= w; if (b) y += b; out = round_to_16bit(y)
 * Input rows are in_row_stride elements apart, output rows are dense (:37-38).
 */
int ao_speculator_ln(void *out, const void *in, const void *w, const void *b,
                     int64_t rows, int hidden, int64_t in_row_stride, float eps,
                     int dtype) {
  if (dtype != AO_F16 && dtype != AO_BF16) return -1;
  uint16_t *o = (uint16_t *)out;
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    const int64_t base = r * in_row_stride;
    float ss = 0.f;
    for (int j = 0; j < hidden; ++j) {
      float x = load_as_f32(in, base + j, dtype);
      ss += x * x;
    }
    const float inv = 1.0f / sqrtf(ss / (float)hidden + eps);
    for (int j = 0; j < hidden; ++j) {
      float y = load_as_f32(in, base + j, dtype) * inv;
      if (w) y *= load_as_f32(w, j, dtype);
      if (b) y += load_as_f32(b, j, dtype);
      o[r * (int64_t)hidden + j] = store_half(y, dtype);
    }
  }
  return 0;
}

/* ---- Part B: fused LSTM-style gate / cell / state update -------------------
 * sigmoid_f, gelu_erf, gelu_tanh: csrc/custom_ops/sum_lstm.cu:14-26.
 */
static inline float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }
static inline float gelu_erf(float x) {
  return 0.5f * x * (1.0f + erff(x * 0.70710678118654752440f));
}
static inline float gelu_tanh(float x) {
  return 0.5f * x *
         (1.0f + tanhf(0.79788456080286535588f * (x + 0.044715f * x * x * x)));
}

/* The speculator's element-wise steps around its norm, as one function: the
 * PyTorch sequences of arctic_inference/vllm/spec_dec/arctic_speculator.py
 *   :300-307, :809-816   states.add_(z, alpha=a); activation(ln(states))
 *   :296-297, :733-734   ln0(previous_hidden_states) / SQRT2
 * Every PyTorch op of those sequences leaves a 16-bit tensor, so the value is
 * rounded to the 16-bit type after the add, after the norm (ao_speculator_ln's own
 * rounding), after the GELU and after the scaling.  The add is a + alpha*b with a
 * single rounding in fp32 (what the GPU's add kernel computes); nn.GELU() is the
 * erf form evaluated in fp32; a tensor divided by a Python scalar is multiplied by
 * the fp32 reciprocal, which the caller passes as out_scale.
 * activation: 0 none, 1 erf GELU, 2 tanh GELU. */
int ao_speculator_add_ln_act(void *out, const void *in, const void *z, const void *w,
                             const void *b, int64_t rows, int hidden,
                             int64_t in_row_stride, int64_t z_row_stride, float alpha,
                             float eps, int activation, float out_scale, int dtype) {
  if (dtype != AO_F16 && dtype != AO_BF16) return -1;
  if (activation < 0 || activation > 2) return -2;
  uint16_t *o = (uint16_t *)out;
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    float *x = (float *)malloc(sizeof(float) * (size_t)hidden);
    float ss = 0.f;
    for (int j = 0; j < hidden; ++j) {
      float v = load_as_f32(in, r * in_row_stride + j, dtype);
      if (z) v = requant(fmaf(alpha, load_as_f32(z, r * z_row_stride + j, dtype), v), dtype);
      x[j] = v;
      ss += v * v;
    }
    const float inv = 1.0f / sqrtf(ss / (float)hidden + eps);
    for (int j = 0; j < hidden; ++j) {
      float y = x[j] * inv;
      if (w) y *= load_as_f32(w, j, dtype);
      if (b) y += load_as_f32(b, j, dtype);
      y = requant(y, dtype);
      if (activation) y = requant(activation == 1 ? gelu_erf(y) : gelu_tanh(y), dtype);
      if (out_scale != 1.0f) y = requant(y * out_scale, dtype);
      o[r * (int64_t)hidden + j] = store_half(y, dtype);
    }
    free(x);
  }
  return 0;
}

/* Restates sum_lstm_vec_kernel / sum_lstm_scalar_kernel
 * (csrc/custom_ops/sum_lstm.cu:28-291).  Gate order along the last dim of
 * states/z4 is f | i | o | c, each D wide.
 *   pre_g   = s_g + alpha * z_g                              (:118-120)
 *   inv_c   = rsqrt(sum(pre_c^2)/D + eps_cell)               (:65-82)
 *   cn      = pre_c*inv_c [*w_cell] [+b_cell]; cact = gelu(cn)
 *   c_new   = prev_cell*sigmoid(pre_f) + cact*sigmoid(pre_i)   (:134)
 *   out_cell = round_to_16bit(c_new); sum(c_new^2) uses the UNROUNDED value (:136-137)
 *   inv_s   = rsqrt(sum(c_new^2)/D + eps_state)               (:143-149)
 *   the state phase re-reads the ROUNDED out_cell                (:163,174)
 *   st      = gelu(rounded_c*inv_s [*w_state] [+b_state]) * sigmoid(pre_o)
 * Strides are in elements; out_state and out_cell share out_stride (:356-365).
 */
int ao_sum_lstm(void *out_state, void *out_cell, const void *states,
                const void *z4, const void *prev_cell, const void *w_cell,
                const void *b_cell, const void *w_state, const void *b_state,
                int64_t rows, int D, int64_t s_stride, int64_t z_stride,
                int64_t pc_stride, int64_t out_stride, float alpha,
                float eps_cell, float eps_state, int fast_gelu, int dtype) {
  if (dtype != AO_F16 && dtype != AO_BF16) return -1;
  uint16_t *os = (uint16_t *)out_state;
  uint16_t *oc = (uint16_t *)out_cell;
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    const int64_t sb = r * s_stride, zb = r * z_stride, pb = r * pc_stride,
                  ob = r * out_stride;
    float ss_cpre = 0.f;
    for (int j = 0; j < D; ++j) {
      float c = load_as_f32(states, sb + 3 * (int64_t)D + j, dtype) +
                alpha * load_as_f32(z4, zb + 3 * (int64_t)D + j, dtype);
      ss_cpre += c * c;
    }
    const float inv_c = 1.0f / sqrtf(ss_cpre / (float)D + eps_cell);
    float ss_cnew = 0.f;
    for (int j = 0; j < D; ++j) {
      float pre_f = load_as_f32(states, sb + j, dtype) +
                    alpha * load_as_f32(z4, zb + j, dtype);
      float pre_i = load_as_f32(states, sb + D + j, dtype) +
                    alpha * load_as_f32(z4, zb + D + j, dtype);
      float cpre = load_as_f32(states, sb + 3 * (int64_t)D + j, dtype) +
                   alpha * load_as_f32(z4, zb + 3 * (int64_t)D + j, dtype);
      float fg = sigmoid_f(pre_f), ig = sigmoid_f(pre_i);
      float cn = cpre * inv_c;
      if (w_cell) cn *= load_as_f32(w_cell, j, dtype);
      if (b_cell) cn += load_as_f32(b_cell, j, dtype);
      float cact = fast_gelu ? gelu_tanh(cn) : gelu_erf(cn);
      float cnew = load_as_f32(prev_cell, pb + j, dtype) * fg + cact * ig;
      ss_cnew += cnew * cnew;
      oc[ob + j] = store_half(cnew, dtype);
    }
    const float inv_s = 1.0f / sqrtf(ss_cnew / (float)D + eps_state);
    for (int j = 0; j < D; ++j) {
      float cn = load_as_f32(oc, ob + j, dtype) * inv_s;
      if (w_state) cn *= load_as_f32(w_state, j, dtype);
      if (b_state) cn += load_as_f32(b_state, j, dtype);
      float sact = fast_gelu ? gelu_tanh(cn) : gelu_erf(cn);
      float pre_o = load_as_f32(states, sb + 2 * (int64_t)D + j, dtype) +
                    alpha * load_as_f32(z4, zb + 2 * (int64_t)D + j, dtype);
      os[ob + j] = store_half(sact * sigmoid_f(pre_o), dtype);
    }
  }
  return 0;
}

/* Number of threads the parallel loops above use (1 without OpenMP). */
int ao_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

void ao_set_num_threads(int n) {
#ifdef _OPENMP
  if (n > 0) omp_set_num_threads(n);
#else
  (void)n;
#endif
}
