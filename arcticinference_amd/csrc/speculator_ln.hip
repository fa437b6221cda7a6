// Speculator "LayerNorm" (RMS norm with optional scale and shift) for gfx950.
//
// Replaces speculator_ln_cuda and its kernels
// (csrc/custom_ops/speculator_ln.cu:21-252 in the reference).
//
// One workgroup per row.  On the vector path every lane keeps its 16-byte
// chunks of the row in registers between the sum of squares and the scaling, so
// the row is read from HBM once (the reference reads it twice); the sum is a DPP
// wave reduction followed by a small LDS combine.
//
// The same kernel also carries the element-wise steps the speculator runs around
// this norm (arctic_speculator.py:296-307,733-734,809-816), each with the rounding
// of the separate PyTorch op it stands for:
//   x   = round(in + alpha * z)        states.add_(z, alpha=...)      (optional)
//   y   = round(x * inv_rms * w + b)   speculator_ln
//   y   = round(gelu(y))               nn.GELU()                      (optional)
//   out = round(y * out_scale)         ln0(x) / sqrt(2)               (optional)
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <algorithm>

#include "activations.hpp"
#include "common.hpp"

namespace arctic {

// What surrounds the norm; all fields are uniform over the launch.
struct LnGlue {
  const char *z;            // nullptr: no add
  int64_t z_row_stride_bytes;
  const int64_t *z_index;   // row of z to add to each row (an embedding lookup); nullptr = the row itself
  int64_t z_rows;           // rows of z when z_index is given; an index is clamped into [0, z_rows)
  float alpha;
  int activation;           // ARCTIC_ACT_*
  float out_scale;          // applied when != 1
};

template <typename T>
__device__ __forceinline__ float glue_tail(float y, const LnGlue &g) {
  if (g.activation != ARCTIC_ACT_NONE) {
    y = T::requant(y);
    y = g.activation == ARCTIC_ACT_GELU ? gelu_erf(y) : gelu_tanh(y);
  }
  if (g.out_scale != 1.0f) y = T::requant(y) * g.out_scale;
  return y;
}

template <typename T, int kChunksPerThread, bool kGlue>
__global__ __launch_bounds__(1024) void spec_ln_vec_kernel(
    char *__restrict__ out, const char *__restrict__ in, const char *__restrict__ weight,
    const char *__restrict__ bias, int64_t in_row_stride_bytes, int hidden, float inv_hidden, float eps,
    LnGlue glue) {
  __shared__ float slots[16];
  const int chunks = hidden >> 3;
  const char *row_in = in + (int64_t)blockIdx.x * in_row_stride_bytes;
  char *row_out = out + (int64_t)blockIdx.x * hidden * 2;

  uint4 raw[kChunksPerThread], wv[kChunksPerThread], bv[kChunksPerThread];
  float ss = 0.f;
  // scale / shift first: they are cache resident and memory returns loads in issue
  // order, so asking for them after the row sum would add a full round trip
#pragma unroll
  for (int k = 0; k < kChunksPerThread; ++k) {
    const int c = threadIdx.x + k * blockDim.x;
    if (weight && c < chunks) wv[k] = load16(weight + (int64_t)c * 16);
    if (bias && c < chunks) bv[k] = load16(bias + (int64_t)c * 16);
  }
#pragma unroll
  for (int k = 0; k < kChunksPerThread; ++k) {
    const int c = threadIdx.x + k * blockDim.x;
    raw[k] = make_uint4(0, 0, 0, 0);
    if (c < chunks) raw[k] = load16_stream(row_in + (int64_t)c * 16);
  }
  if (kGlue && glue.z) {
    int64_t z_at = blockIdx.x;
    if (glue.z_index) z_at = min(max(glue.z_index[blockIdx.x], (int64_t)0), glue.z_rows - 1);
    const char *row_z = glue.z + z_at * glue.z_row_stride_bytes;
    uint4 zr[kChunksPerThread];
#pragma unroll
    for (int k = 0; k < kChunksPerThread; ++k) {
      const int c = threadIdx.x + k * blockDim.x;
      zr[k] = make_uint4(0, 0, 0, 0);
      if (c < chunks) zr[k] = load16_stream(row_z + (int64_t)c * 16);
    }
#pragma unroll
    for (int k = 0; k < kChunksPerThread; ++k) {
      float x[8], z[8];
      unpack8<T>(raw[k], x);
      unpack8<T>(zr[k], z);
#pragma unroll
      for (int j = 0; j < 8; ++j) x[j] = fmaf(glue.alpha, z[j], x[j]);
      raw[k] = pack8<T>(x);   // the sum stands in the tensor's own type, as after the in-place add
    }
  }
#pragma unroll
  for (int k = 0; k < kChunksPerThread; ++k) {
    float x[8];
    unpack8<T>(raw[k], x);
#pragma unroll
    for (int j = 0; j < 8; ++j) ss += x[j] * x[j];
  }
  const float total = block_sum(ss, slots);
  const float inv = rsqrtf(total * inv_hidden + eps);

#pragma unroll
  for (int k = 0; k < kChunksPerThread; ++k) {
    const int c = threadIdx.x + k * blockDim.x;
    if (c >= chunks) continue;
    float x[8];
    unpack8<T>(raw[k], x);
#pragma unroll
    for (int j = 0; j < 8; ++j) x[j] *= inv;
    if (weight) {
      float w[8];
      unpack8<T>(wv[k], w);
#pragma unroll
      for (int j = 0; j < 8; ++j) x[j] *= w[j];
    }
    if (bias) {
      float b[8];
      unpack8<T>(bv[k], b);
#pragma unroll
      for (int j = 0; j < 8; ++j) x[j] += b[j];
    }
    if (kGlue) {
#pragma unroll
      for (int j = 0; j < 8; ++j) x[j] = glue_tail<T>(x[j], glue);
    }
    store16_stream(row_out + (int64_t)c * 16, pack8<T>(x));
  }
}

// Any hidden size, any alignment: element-wise, two passes over the row.
template <typename T>
__global__ __launch_bounds__(256) void spec_ln_scalar_kernel(
    uint16_t *__restrict__ out, const uint16_t *__restrict__ in, const uint16_t *__restrict__ weight,
    const uint16_t *__restrict__ bias, int64_t in_row_stride, int hidden, float inv_hidden, float eps,
    LnGlue glue) {
  __shared__ float slots[16];
  const uint16_t *row_in = in + (int64_t)blockIdx.x * in_row_stride;
  int64_t z_at = blockIdx.x;
  if (glue.z && glue.z_index) z_at = min(max(glue.z_index[blockIdx.x], (int64_t)0), glue.z_rows - 1);
  const uint16_t *row_z = glue.z ? (const uint16_t *)(glue.z + z_at * glue.z_row_stride_bytes) : nullptr;
  uint16_t *row_out = out + (int64_t)blockIdx.x * hidden;
  auto element = [&](int j) {
    float x = T::lo(row_in[j]);
    if (row_z) x = T::requant(fmaf(glue.alpha, T::lo(row_z[j]), x));
    return x;
  };
  float ss = 0.f;
  for (int j = threadIdx.x; j < hidden; j += blockDim.x) {
    const float x = element(j);
    ss += x * x;
  }
  const float total = block_sum(ss, slots);
  const float inv = rsqrtf(total * inv_hidden + eps);
  for (int j = threadIdx.x; j < hidden; j += blockDim.x) {
    float y = element(j) * inv;
    if (weight) y *= T::lo(weight[j]);
    if (bias) y += T::lo(bias[j]);
    row_out[j] = (uint16_t)T::round_bits(glue_tail<T>(y, glue));
  }
}

static inline bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

template <typename T>
static void launch_ln(void *out, const void *in, const void *w, const void *b, int64_t rows, int hidden,
                      int64_t in_row_stride, float eps, const LnGlue &glue, hipStream_t s) {
  const int chunks = hidden / 8;
  const float inv_hidden = 1.0f / (float)hidden;
  const bool vec = (hidden % 8 == 0) && (in_row_stride % 8 == 0 || rows == 1) && aligned16(in) &&
                   aligned16(out) && (!w || aligned16(w)) && (!b || aligned16(b)) && chunks <= 8 * 1024 &&
                   (!glue.z || (aligned16(glue.z) && (glue.z_row_stride_bytes % 16 == 0 || (rows == 1 && !glue.z_index))));
  const bool plain = !glue.z && glue.activation == ARCTIC_ACT_NONE && glue.out_scale == 1.0f;
  const dim3 grid((unsigned)rows);
  if (vec) {
    int cpt = 1;
    while (cpt < 8 && (chunks + cpt - 1) / cpt > 1024) cpt *= 2;
    int threads = (chunks + cpt - 1) / cpt;
    threads = std::max(64, (threads + 63) & ~63);
    const int64_t stride_bytes = in_row_stride * 2;
#define ARCTIC_LN_LAUNCH(CPT)                                                                              \
  do {                                                                                                     \
    if (plain)                                                                                             \
      hipLaunchKernelGGL((spec_ln_vec_kernel<T, CPT, false>), grid, dim3(threads), 0, s, (char *)out,       \
                         (const char *)in, (const char *)w, (const char *)b, stride_bytes, hidden,          \
                         inv_hidden, eps, glue);                                                           \
    else                                                                                                   \
      hipLaunchKernelGGL((spec_ln_vec_kernel<T, CPT, true>), grid, dim3(threads), 0, s, (char *)out,        \
                         (const char *)in, (const char *)w, (const char *)b, stride_bytes, hidden,          \
                         inv_hidden, eps, glue);                                                           \
  } while (0)
    switch (cpt) {
      case 1: ARCTIC_LN_LAUNCH(1); break;
      case 2: ARCTIC_LN_LAUNCH(2); break;
      case 4: ARCTIC_LN_LAUNCH(4); break;
      default: ARCTIC_LN_LAUNCH(8); break;
    }
#undef ARCTIC_LN_LAUNCH
  } else {
    hipLaunchKernelGGL((spec_ln_scalar_kernel<T>), grid, dim3(256), 0, s, (uint16_t *)out,
                       (const uint16_t *)in, (const uint16_t *)w, (const uint16_t *)b, in_row_stride, hidden,
                       inv_hidden, eps, glue);
  }
}

}  // namespace arctic

using namespace arctic;

static int ln_entry(const char *fn, void *out, const void *in, const void *weight, const void *bias,
                    int64_t rows, int hidden, int64_t in_row_stride, float eps, const LnGlue &glue, int dtype,
                    void *stream) {
  if (dtype != ARCTIC_DTYPE_F16 && dtype != ARCTIC_DTYPE_BF16)
    return fail(ARCTIC_ERR_UNSUPPORTED, "%s: only fp16 and bf16 are supported.", fn);
  if (hidden <= 0) return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: hidden size must be > 0", fn);
  if (hidden > (1 << 30)) return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: hidden size beyond 2^30", fn);
  if (rows < 0 || rows > 0x7fffffffLL) return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: bad row count", fn);
  if (glue.activation != ARCTIC_ACT_NONE && glue.activation != ARCTIC_ACT_GELU &&
      glue.activation != ARCTIC_ACT_GELU_TANH)
    return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: unknown activation %d", fn, glue.activation);
  if (rows == 0) return ARCTIC_OK;
  if (!out || !in) return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: null tensor pointer", fn);
  if (!pitch_ok(in_row_stride, rows, 2) || !pitch_ok(hidden, rows, 2))
    return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: row pitch out of range", fn);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == ARCTIC_DTYPE_BF16)
    launch_ln<BF16>(out, in, weight, bias, rows, hidden, in_row_stride, eps, glue, s);
  else
    launch_ln<F16>(out, in, weight, bias, rows, hidden, in_row_stride, eps, glue, s);
  return check_launch(fn);
}

extern "C" int arctic_speculator_ln(void *out, const void *in, const void *weight, const void *bias,
                                    int64_t rows, int hidden, int64_t in_row_stride, float eps, int dtype,
                                    void *stream) {
  const LnGlue none = {nullptr, 0, nullptr, 0, 0.0f, ARCTIC_ACT_NONE, 1.0f};
  return ln_entry("speculator_ln", out, in, weight, bias, rows, hidden, in_row_stride, eps, none, dtype, stream);
}

extern "C" int arctic_speculator_add_ln_act(void *out, const void *in, const void *z, const void *weight,
                                            const void *bias, int64_t rows, int hidden, int64_t in_row_stride,
                                            int64_t z_row_stride, float alpha, float eps, int activation,
                                            float out_scale, int dtype, void *stream) {
  if (!pitch_ok(z_row_stride, rows, 2))
    return fail(ARCTIC_ERR_INVALID_ARGUMENT, "speculator_add_ln_act: row pitch of z out of range");
  const LnGlue glue = {(const char *)z, z_row_stride * 2, nullptr, 0, alpha, activation, out_scale};
  return ln_entry("speculator_add_ln_act", out, in, weight, bias, rows, hidden, in_row_stride, eps, glue, dtype,
                  stream);
}

extern "C" int arctic_speculator_embed_add_ln_act(void *out, const void *in, const void *emb_table,
                                                  const int64_t *token_ids, const void *weight, const void *bias,
                                                  int64_t rows, int hidden, int64_t in_row_stride, int64_t emb_row_stride,
                                                  int64_t num_embeddings, float alpha, float eps, int activation,
                                                  float out_scale, int dtype, void *stream) {
  const char *fn = "speculator_embed_add_ln_act";
  if (rows > 0 && (!emb_table || !token_ids)) return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: null embedding table or token ids", fn);
  if (rows > 0 && num_embeddings <= 0) return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: the embedding table has no rows", fn);
  if (!pitch_ok(emb_row_stride, num_embeddings, 2))
    return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: row pitch of the embedding table out of range", fn);
  const LnGlue glue = {(const char *)emb_table, emb_row_stride * 2, token_ids, num_embeddings, alpha, activation, out_scale};
  return ln_entry(fn, out, in, weight, bias, rows, hidden, in_row_stride, eps, glue, dtype, stream);
}
