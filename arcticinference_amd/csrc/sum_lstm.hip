// Fused LSTM-style gate / cell / state update of the Arctic speculator, gfx950.
//
// Replaces sum_lstm_cuda and its kernels
// (csrc/custom_ops/sum_lstm.cu:14-473 in the reference).
//
// One workgroup per row.  On the vector path each lane owns 16-byte chunks
// (8 elements) at the same column of all four gates of `states` and `z4` and of
// `prev_cell`: nine 16-byte loads per chunk, issued together.  The row then
// stays in registers across both RMS reductions, so HBM sees 9*D elements read
// and 2*D written per row (the reference re-reads the cell gate and reads
// out_cell back: 12*D).  Sums are DPP wave reductions plus an LDS combine.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <algorithm>

#include "common.hpp"

namespace arctic {

// sigmoid_f / gelu_erf / gelu_tanh of the reference (sum_lstm.cu:14-26).
__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float gelu_erf(float x) {
  return 0.5f * x * (1.0f + erff(x * 0.70710678118654752440f));
}
__device__ __forceinline__ float gelu_tanh(float x) {
  return 0.5f * x * (1.0f + tanhf(0.79788456080286535588f * (x + 0.044715f * x * x * x)));
}
template <bool kFastGelu>
__device__ __forceinline__ float gelu(float x) {
  return kFastGelu ? gelu_tanh(x) : gelu_erf(x);
}

struct LstmParams {
  char *out_state;
  char *out_cell;
  const char *states;
  const char *z4;
  const char *prev_cell;
  const char *w_cell;
  const char *b_cell;
  const char *w_state;
  const char *b_state;
  int64_t s_stride;   // all strides in elements
  int64_t z_stride;
  int64_t pc_stride;
  int64_t out_stride;
  int D;
  float alpha;
  float eps_cell;
  float eps_state;
};

template <typename T, int kChunksPerThread, bool kFastGelu>
__global__ __launch_bounds__(1024) void sum_lstm_vec_kernel(const LstmParams p) {
  __shared__ float slots_cpre[16];
  __shared__ float slots_cnew[16];
  const int D = p.D;
  const int chunks = D >> 3;
  const int64_t row = blockIdx.x;
  const int64_t gate_bytes = (int64_t)D * 2;
  const char *s_row = p.states + row * p.s_stride * 2;
  const char *z_row = p.z4 + row * p.z_stride * 2;
  const char *pc_row = p.prev_cell + row * p.pc_stride * 2;
  char *oc_row = p.out_cell + row * p.out_stride * 2;
  char *os_row = p.out_state + row * p.out_stride * 2;

  uint4 s[kChunksPerThread][4], z[kChunksPerThread][4], pc[kChunksPerThread];
#pragma unroll
  for (int k = 0; k < kChunksPerThread; ++k) {
    const int c = threadIdx.x + k * blockDim.x;
    const int64_t off = (int64_t)c * 16;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      s[k][g] = make_uint4(0, 0, 0, 0);
      z[k][g] = make_uint4(0, 0, 0, 0);
    }
    pc[k] = make_uint4(0, 0, 0, 0);
    if (c < chunks) {
      // cell gate first: the first reduction only needs it
      s[k][3] = load16_stream(s_row + 3 * gate_bytes + off);
      z[k][3] = load16_stream(z_row + 3 * gate_bytes + off);
#pragma unroll
      for (int g = 0; g < 3; ++g) {
        s[k][g] = load16_stream(s_row + g * gate_bytes + off);
        z[k][g] = load16_stream(z_row + g * gate_bytes + off);
      }
      pc[k] = load16_stream(pc_row + off);
    }
  }

  // phase 1: pre_c and its sum of squares (reference :65-82)
  float cpre[kChunksPerThread][8];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < kChunksPerThread; ++k) {
    float a[8], b[8];
    unpack8<T>(s[k][3], a);
    unpack8<T>(z[k][3], b);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      cpre[k][j] = a[j] + p.alpha * b[j];
      ss += cpre[k][j] * cpre[k][j];
    }
  }
  const float inv_cpre = rsqrtf(block_sum(ss, slots_cpre) / (float)D + p.eps_cell);

  // phase 2: gates f, i; cell update; write out_cell (reference :104-140)
  float cell[kChunksPerThread][8];  // the ROUNDED new cell, as the state phase must see it
  ss = 0.f;
#pragma unroll
  for (int k = 0; k < kChunksPerThread; ++k) {
    const int c = threadIdx.x + k * blockDim.x;
    const bool live = c < chunks;
    float sf[8], zf[8], si[8], zi[8], pcv[8], w[8], b[8];
    unpack8<T>(s[k][0], sf);
    unpack8<T>(z[k][0], zf);
    unpack8<T>(s[k][1], si);
    unpack8<T>(z[k][1], zi);
    unpack8<T>(pc[k], pcv);
    if (p.w_cell && live) unpack8<T>(load16(p.w_cell + (int64_t)c * 16), w);
    if (p.b_cell && live) unpack8<T>(load16(p.b_cell + (int64_t)c * 16), b);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float fgate = sigmoid_f(sf[j] + p.alpha * zf[j]);
      const float igate = sigmoid_f(si[j] + p.alpha * zi[j]);
      float cn = cpre[k][j] * inv_cpre;
      if (p.w_cell) cn *= w[j];
      if (p.b_cell) cn += b[j];
      const float cnew = live ? pcv[j] * fgate + gelu<kFastGelu>(cn) * igate : 0.f;
      ss += cnew * cnew;  // unrounded, as in the reference (:136)
      cell[k][j] = cnew;
    }
    const uint4 packed = pack8<T>(cell[k]);
    if (live) store16_stream(oc_row + (int64_t)c * 16, packed);
    unpack8<T>(packed, cell[k]);
  }
  const float inv_cnew = rsqrtf(block_sum(ss, slots_cnew) / (float)D + p.eps_state);

  // phase 3: state = gelu(rmsnorm(rounded cell)) * sigmoid(pre_o) (reference :160-190)
#pragma unroll
  for (int k = 0; k < kChunksPerThread; ++k) {
    const int c = threadIdx.x + k * blockDim.x;
    if (c >= chunks) continue;
    float so[8], zo[8], w[8], b[8], st[8];
    unpack8<T>(s[k][2], so);
    unpack8<T>(z[k][2], zo);
    if (p.w_state) unpack8<T>(load16(p.w_state + (int64_t)c * 16), w);
    if (p.b_state) unpack8<T>(load16(p.b_state + (int64_t)c * 16), b);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      float cn = cell[k][j] * inv_cnew;
      if (p.w_state) cn *= w[j];
      if (p.b_state) cn += b[j];
      st[j] = gelu<kFastGelu>(cn) * sigmoid_f(so[j] + p.alpha * zo[j]);
    }
    store16_stream(os_row + (int64_t)c * 16, pack8<T>(st));
  }
}

// Any D, any alignment: element-wise, three passes like the reference's scalar
// kernel (sum_lstm.cu:193-291).
template <typename T, bool kFastGelu>
__global__ __launch_bounds__(256) void sum_lstm_scalar_kernel(const LstmParams p) {
  __shared__ float slots_cpre[16];
  __shared__ float slots_cnew[16];
  const int D = p.D;
  const int64_t row = blockIdx.x;
  const uint16_t *s = (const uint16_t *)p.states + row * p.s_stride;
  const uint16_t *z = (const uint16_t *)p.z4 + row * p.z_stride;
  const uint16_t *pc = (const uint16_t *)p.prev_cell + row * p.pc_stride;
  uint16_t *oc = (uint16_t *)p.out_cell + row * p.out_stride;
  uint16_t *os = (uint16_t *)p.out_state + row * p.out_stride;
  const uint16_t *wc = (const uint16_t *)p.w_cell, *bc = (const uint16_t *)p.b_cell;
  const uint16_t *ws = (const uint16_t *)p.w_state, *bs = (const uint16_t *)p.b_state;

  float ss = 0.f;
  for (int j = threadIdx.x; j < D; j += blockDim.x) {
    const float c = T::lo(s[3 * (int64_t)D + j]) + p.alpha * T::lo(z[3 * (int64_t)D + j]);
    ss += c * c;
  }
  const float inv_cpre = rsqrtf(block_sum(ss, slots_cpre) / (float)D + p.eps_cell);

  ss = 0.f;
  for (int j = threadIdx.x; j < D; j += blockDim.x) {
    const float pre_f = T::lo(s[j]) + p.alpha * T::lo(z[j]);
    const float pre_i = T::lo(s[(int64_t)D + j]) + p.alpha * T::lo(z[(int64_t)D + j]);
    const float cpre = T::lo(s[3 * (int64_t)D + j]) + p.alpha * T::lo(z[3 * (int64_t)D + j]);
    float cn = cpre * inv_cpre;
    if (wc) cn *= T::lo(wc[j]);
    if (bc) cn += T::lo(bc[j]);
    const float cnew = T::lo(pc[j]) * sigmoid_f(pre_f) + gelu<kFastGelu>(cn) * sigmoid_f(pre_i);
    ss += cnew * cnew;
    oc[j] = (uint16_t)T::round_bits(cnew);
  }
  const float inv_cnew = rsqrtf(block_sum(ss, slots_cnew) / (float)D + p.eps_state);

  // each thread re-reads only the out_cell elements it wrote itself
  for (int j = threadIdx.x; j < D; j += blockDim.x) {
    float cn = T::lo(oc[j]) * inv_cnew;
    if (ws) cn *= T::lo(ws[j]);
    if (bs) cn += T::lo(bs[j]);
    const float pre_o = T::lo(s[2 * (int64_t)D + j]) + p.alpha * T::lo(z[2 * (int64_t)D + j]);
    os[j] = (uint16_t)T::round_bits(gelu<kFastGelu>(cn) * sigmoid_f(pre_o));
  }
}

static inline bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

template <typename T, bool kFastGelu>
static void launch_lstm(const LstmParams &p, int64_t rows, hipStream_t s) {
  const int chunks = p.D / 8;
  const bool multi = rows > 1;
  const bool vec = (p.D % 8 == 0) && chunks <= 2 * 1024 &&
                   (!multi || (p.s_stride % 8 == 0 && p.z_stride % 8 == 0 && p.pc_stride % 8 == 0 &&
                               p.out_stride % 8 == 0)) &&
                   aligned16(p.states) && aligned16(p.z4) && aligned16(p.prev_cell) &&
                   aligned16(p.out_state) && aligned16(p.out_cell) && aligned16(p.w_cell) &&
                   aligned16(p.b_cell) && aligned16(p.w_state) && aligned16(p.b_state);
  const dim3 grid((unsigned)rows);
  if (vec) {
    const int cpt = chunks > 1024 ? 2 : 1;
    int threads = (chunks + cpt - 1) / cpt;
    threads = std::max(64, (threads + 63) & ~63);
    if (cpt == 1)
      hipLaunchKernelGGL((sum_lstm_vec_kernel<T, 1, kFastGelu>), grid, dim3(threads), 0, s, p);
    else
      hipLaunchKernelGGL((sum_lstm_vec_kernel<T, 2, kFastGelu>), grid, dim3(threads), 0, s, p);
  } else {
    hipLaunchKernelGGL((sum_lstm_scalar_kernel<T, kFastGelu>), grid, dim3(256), 0, s, p);
  }
}

}  // namespace arctic

using namespace arctic;

extern "C" int arctic_sum_lstm(void *out_state, void *out_cell, const void *states, const void *z4,
                               const void *prev_cell, const void *w_cell, const void *b_cell,
                               const void *w_state, const void *b_state, int64_t rows, int D,
                               int64_t s_stride, int64_t z_stride, int64_t pc_stride, int64_t out_stride,
                               float alpha, float eps_cell, float eps_state, int fast_gelu, int dtype,
                               void *stream) {
  const char *fn = "sum_lstm";
  if (dtype != ARCTIC_DTYPE_F16 && dtype != ARCTIC_DTYPE_BF16)
    return fail(ARCTIC_ERR_UNSUPPORTED, "%s: only fp16 and bf16 are supported.", fn);
  if (D <= 0) return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: last dim of states must be 4*D_gate", fn);
  if (rows < 0 || rows > 0x7fffffffLL) return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: bad row count", fn);
  if (rows == 0) return ARCTIC_OK;
  if (!out_state || !out_cell || !states || !z4 || !prev_cell)
    return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: null tensor pointer", fn);
  LstmParams p;
  p.out_state = (char *)out_state;
  p.out_cell = (char *)out_cell;
  p.states = (const char *)states;
  p.z4 = (const char *)z4;
  p.prev_cell = (const char *)prev_cell;
  p.w_cell = (const char *)w_cell;
  p.b_cell = (const char *)b_cell;
  p.w_state = (const char *)w_state;
  p.b_state = (const char *)b_state;
  p.s_stride = s_stride;
  p.z_stride = z_stride;
  p.pc_stride = pc_stride;
  p.out_stride = out_stride;
  p.D = D;
  p.alpha = alpha;
  p.eps_cell = eps_cell;
  p.eps_state = eps_state;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == ARCTIC_DTYPE_BF16) {
    if (fast_gelu) launch_lstm<BF16, true>(p, rows, s);
    else launch_lstm<BF16, false>(p, rows, s);
  } else {
    if (fast_gelu) launch_lstm<F16, true>(p, rows, s);
    else launch_lstm<F16, false>(p, rows, s);
  }
  return check_launch(fn);
}
