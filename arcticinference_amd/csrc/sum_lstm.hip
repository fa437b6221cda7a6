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
#include <cstdlib>

#include "activations.hpp"
#include "common.hpp"

namespace arctic {

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
  const int64_t *z_index;  // shared-z only: row of z4 to use for each row (an embedding lookup); nullptr = the row itself
  int64_t z_rows;          // rows of z4 when z_index is given; an index is clamped into [0, z_rows)
  int64_t s_stride;   // all strides in elements
  int64_t z_stride;
  int64_t pc_stride;
  int64_t out_stride;
  int D;
  float inv_D;        // 1 / D
  float alpha;
  float eps_cell;
  float eps_state;
};

// Loads are issued in the order in which the arithmetic needs them - cell gate,
// forget gate, previous cell, input gate, output gate - and memory returns them
// in that order, so the first row sum, the candidate GELU and the early sigmoids
// run while the later gates are still on their way, and only one sigmoid, one
// multiply and the store remain after the last load has landed.
// kSharedZ: `z4` holds ONE gate-wide row per token ([rows, D]) that is added to all four
// gates, as the speculator's z4 = emb.repeat(1, 1, 4) would; it is then read once, not four times.
// kAllVectors: all four scale / shift vectors are given (the speculator always passes them)
// AND every lane of the workgroup owns a chunk, so no select on either is needed.
template <typename T, int E, int kChunksPerThread, bool kFastGelu, int kMaxThreads, bool kSharedZ, bool kAllVectors>
__global__ __launch_bounds__(kMaxThreads) void sum_lstm_vec_kernel(const LstmParams p) {
  __shared__ float slots_cpre[16];
  __shared__ float slots_cnew[16];
  constexpr int K = kChunksPerThread;
  using C = Chunk<E>;
  const int D = p.D;
  const int chunks = D / E;
  const int64_t row = blockIdx.x;
  const int64_t gate_bytes = (int64_t)D * 2;
  const char *s_row = p.states + row * p.s_stride * 2;
  int64_t zr = row;
  if (kSharedZ && p.z_index) zr = min(max(p.z_index[row], (int64_t)0), p.z_rows - 1);
  const char *z_row = p.z4 + zr * p.z_stride * 2;
  const char *pc_row = p.prev_cell + row * p.pc_stride * 2;
  char *oc_row = p.out_cell + row * p.out_stride * 2;
  char *os_row = p.out_state + row * p.out_stride * 2;

  bool live[K];
  int64_t off[K];
  C sc[K], zc[K], sf[K], zf[K], si[K], zi[K], pc[K], so[K], zo[K];
  C wc[K], bc[K], ws[K], bs[K];
#pragma unroll
  for (int k = 0; k < K; ++k) {
    const int c = threadIdx.x + k * blockDim.x;
    live[k] = kAllVectors || c < chunks;
    off[k] = (int64_t)(live[k] ? c : 0) * C::kBytes;  // idle lanes re-read chunk 0 and discard it
  }
  // The scale / shift vectors are the same for every row (cache resident).  They
  // are requested first: memory returns loads in issue order, so asking for them
  // later would park the arithmetic behind the whole row.
#pragma unroll
  for (int k = 0; k < K; ++k) {
    if (kAllVectors || p.w_cell) wc[k] = C::load(p.w_cell + off[k]);
    if (kAllVectors || p.b_cell) bc[k] = C::load(p.b_cell + off[k]);
    if (kAllVectors || p.w_state) ws[k] = C::load(p.w_state + off[k]);
    if (kAllVectors || p.b_state) bs[k] = C::load(p.b_state + off[k]);
  }
#pragma unroll
  for (int k = 0; k < K; ++k) {
    zc[k] = C::load_stream(z_row + (kSharedZ ? 0 : 3 * gate_bytes) + off[k]);
    sc[k] = C::load_stream(s_row + 3 * gate_bytes + off[k]);
  }
#pragma unroll
  for (int k = 0; k < K; ++k) {
    sf[k] = C::load_stream(s_row + off[k]);
    zf[k] = kSharedZ ? zc[k] : C::load_stream(z_row + off[k]);
  }
#pragma unroll
  // the cell comes straight from the previous step's launch and both outputs are read by the next
  // kernels of the step, so these three accesses stay in the caches; the gates are touched once and stream
  for (int k = 0; k < K; ++k) pc[k] = C::load(pc_row + off[k]);
#pragma unroll
  for (int k = 0; k < K; ++k) {
    si[k] = C::load_stream(s_row + gate_bytes + off[k]);
    zi[k] = kSharedZ ? zc[k] : C::load_stream(z_row + gate_bytes + off[k]);
  }
#pragma unroll
  for (int k = 0; k < K; ++k) {
    so[k] = C::load_stream(s_row + 2 * gate_bytes + off[k]);
    zo[k] = kSharedZ ? zc[k] : C::load_stream(z_row + 2 * gate_bytes + off[k]);
  }

  // Lanes beyond the row take part in the sums with zeros.  (Each value is
  // cleared where it is first used, not here: touching pc now would wait for it.)
  // phase 1: pre_c and its sum of squares (reference :65-82); needs the cell gate only
  float cact[K][E];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < K; ++k) {
    float a[E], b[E];
    if (!live[k]) sc[k] = zc[k] = C::zero();
    sc[k].template unpack<T>(a);
    zc[k].template unpack<T>(b);
#pragma unroll
    for (int j = 0; j < E; ++j) {
      cact[k][j] = fmaf(p.alpha, b[j], a[j]);
      ss = fmaf(cact[k][j], cact[k][j], ss);
    }
  }
  const float inv_cpre = rsqrtf(block_sum(ss, slots_cpre) * p.inv_D + p.eps_cell);
  // candidate = gelu(rmsnorm(pre_c)): runs while the other gates are still arriving
#pragma unroll
  for (int k = 0; k < K; ++k) {
    // an absent scale / shift vector acts as 1 / 0 (exact), so the norm is one multiply and
    // one fused multiply-add per element whichever vectors were given
    float w[E], b[E];
#pragma unroll
    for (int j = 0; j < E; ++j) {
      w[j] = 1.f;
      b[j] = 0.f;
    }
    if (kAllVectors || p.w_cell) wc[k].template unpack<T>(w);
    if (kAllVectors || p.b_cell) bc[k].template unpack<T>(b);
    const float mask = live[k] ? 1.f : 0.f;  // idle lanes must add nothing to the second sum
#pragma unroll
    for (int j = 0; j < E; ++j) {
      const float cn = fmaf(cact[k][j] * inv_cpre, w[j], b[j]);
      cact[k][j] = gelu<kFastGelu>(cn) * mask;
    }
  }

  // phase 2: cell update; write out_cell (reference :104-140)
  float cell[K][E];  // ends up as the ROUNDED new cell, as the state phase must see it
  ss = 0.f;
#pragma unroll
  for (int k = 0; k < K; ++k) {
    float a[E], b[E], c[E];
    sf[k].template unpack<T>(a);
    zf[k].template unpack<T>(b);
    if (!live[k]) pc[k] = C::zero();
    pc[k].template unpack<T>(c);
#pragma unroll
    for (int j = 0; j < E; ++j) cell[k][j] = sigmoid_f(fmaf(p.alpha, b[j], a[j])) * c[j];
    // keep the forget-gate arithmetic ahead of the wait for the input gate: it then runs while that gate
    // is still arriving instead of in the short stretch between the last two gates
    __builtin_amdgcn_sched_barrier(0);
    si[k].template unpack<T>(a);
    zi[k].template unpack<T>(b);
#pragma unroll
    for (int j = 0; j < E; ++j) {
      const float cnew = fmaf(cact[k][j], sigmoid_f(fmaf(p.alpha, b[j], a[j])), cell[k][j]);
      ss = fmaf(cnew, cnew, ss);  // unrounded, as in the reference (:136)
      cell[k][j] = cnew;
    }
    const C packed = C::template pack<T>(cell[k]);
    if (live[k]) packed.store(oc_row + off[k]);
    packed.template unpack<T>(cell[k]);
  }
  const float inv_cnew = rsqrtf(block_sum(ss, slots_cnew) * p.inv_D + p.eps_state);

  // phase 3: state = gelu(rmsnorm(rounded cell)) * sigmoid(pre_o) (reference :160-190);
  // the output gate is the last load to arrive and is consumed last
#pragma unroll
  for (int k = 0; k < K; ++k) {
    float w[E], b[E], st[E];
#pragma unroll
    for (int j = 0; j < E; ++j) {
      w[j] = 1.f;
      b[j] = 0.f;
    }
    if (kAllVectors || p.w_state) ws[k].template unpack<T>(w);
    if (kAllVectors || p.b_state) bs[k].template unpack<T>(b);
#pragma unroll
    for (int j = 0; j < E; ++j) st[j] = gelu<kFastGelu>(fmaf(cell[k][j] * inv_cnew, w[j], b[j]));
    float a[E], g[E];
    so[k].template unpack<T>(a);
    zo[k].template unpack<T>(g);
#pragma unroll
    for (int j = 0; j < E; ++j) st[j] *= sigmoid_f(fmaf(p.alpha, g[j], a[j]));
    if (live[k]) C::template pack<T>(st).store(os_row + off[k]);
  }
}

// Any D, any alignment: element-wise, three passes like the reference's scalar
// kernel (sum_lstm.cu:193-291).
template <typename T, bool kFastGelu>
__global__ __launch_bounds__(256) void sum_lstm_scalar_kernel(const LstmParams p, const int z_gate_stride) {
  __shared__ float slots_cpre[16];
  __shared__ float slots_cnew[16];
  const int D = p.D;
  const int64_t row = blockIdx.x;
  const uint16_t *s = (const uint16_t *)p.states + row * p.s_stride;
  int64_t zr = row;
  if (p.z_index) zr = min(max(p.z_index[row], (int64_t)0), p.z_rows - 1);
  const uint16_t *z = (const uint16_t *)p.z4 + zr * p.z_stride;
  const uint16_t *pc = (const uint16_t *)p.prev_cell + row * p.pc_stride;
  uint16_t *oc = (uint16_t *)p.out_cell + row * p.out_stride;
  uint16_t *os = (uint16_t *)p.out_state + row * p.out_stride;
  const uint16_t *wc = (const uint16_t *)p.w_cell, *bc = (const uint16_t *)p.b_cell;
  const uint16_t *ws = (const uint16_t *)p.w_state, *bs = (const uint16_t *)p.b_state;

  float ss = 0.f;
  for (int j = threadIdx.x; j < D; j += blockDim.x) {
    const float c = T::lo(s[3 * (int64_t)D + j]) + p.alpha * T::lo(z[3 * (int64_t)z_gate_stride + j]);
    ss += c * c;
  }
  const float inv_cpre = rsqrtf(block_sum(ss, slots_cpre) * p.inv_D + p.eps_cell);

  ss = 0.f;
  for (int j = threadIdx.x; j < D; j += blockDim.x) {
    const float pre_f = T::lo(s[j]) + p.alpha * T::lo(z[j]);
    const float pre_i = T::lo(s[(int64_t)D + j]) + p.alpha * T::lo(z[(int64_t)z_gate_stride + j]);
    const float cpre = T::lo(s[3 * (int64_t)D + j]) + p.alpha * T::lo(z[3 * (int64_t)z_gate_stride + j]);
    float cn = cpre * inv_cpre;
    if (wc) cn *= T::lo(wc[j]);
    if (bc) cn += T::lo(bc[j]);
    const float cnew = T::lo(pc[j]) * sigmoid_f(pre_f) + gelu<kFastGelu>(cn) * sigmoid_f(pre_i);
    ss += cnew * cnew;
    oc[j] = (uint16_t)T::round_bits(cnew);
  }
  const float inv_cnew = rsqrtf(block_sum(ss, slots_cnew) * p.inv_D + p.eps_state);

  // each thread re-reads only the out_cell elements it wrote itself
  for (int j = threadIdx.x; j < D; j += blockDim.x) {
    float cn = T::lo(oc[j]) * inv_cnew;
    if (ws) cn *= T::lo(ws[j]);
    if (bs) cn += T::lo(bs[j]);
    const float pre_o = T::lo(s[2 * (int64_t)D + j]) + p.alpha * T::lo(z[2 * (int64_t)z_gate_stride + j]);
    os[j] = (uint16_t)T::round_bits(gelu<kFastGelu>(cn) * sigmoid_f(pre_o));
  }
}

static inline bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

template <typename T, bool kFastGelu, bool kSharedZ>
static void launch_lstm(const LstmParams &p, int64_t rows, hipStream_t s) {
  const int chunks = p.D / 8;
  const bool multi = rows > 1;
  const bool vec = (p.D % 8 == 0) && chunks <= 2 * 1024 &&
                   (!multi || (p.s_stride % 8 == 0 && p.z_stride % 8 == 0 && p.pc_stride % 8 == 0 &&
                               p.out_stride % 8 == 0)) &&
                   (!p.z_index || p.z_stride % 8 == 0) &&
                   aligned16(p.states) && aligned16(p.z4) && aligned16(p.prev_cell) &&
                   aligned16(p.out_state) && aligned16(p.out_cell) && aligned16(p.w_cell) &&
                   aligned16(p.b_cell) && aligned16(p.w_state) && aligned16(p.b_state);
  const dim3 grid((unsigned)rows);
  if (vec) {
    const int cpt = chunks > 512 ? 2 : 1;   // one 16-byte chunk per lane up to 512 lanes (D <= 4096)
    int threads = (chunks + cpt - 1) / cpt;
    threads = std::max(64, (threads + 63) & ~63);
    const bool all = p.w_cell && p.b_cell && p.w_state && p.b_state && threads * cpt == chunks;
    if (cpt == 1 && all)
      hipLaunchKernelGGL((sum_lstm_vec_kernel<T, 8, 1, kFastGelu, 512, kSharedZ, true>), grid, dim3(threads), 0, s, p);
    else if (cpt == 1)
      hipLaunchKernelGGL((sum_lstm_vec_kernel<T, 8, 1, kFastGelu, 512, kSharedZ, false>), grid, dim3(threads), 0, s, p);
    else
      hipLaunchKernelGGL((sum_lstm_vec_kernel<T, 8, 2, kFastGelu, 1024, kSharedZ, false>), grid, dim3(threads), 0, s, p);
  } else {
    hipLaunchKernelGGL((sum_lstm_scalar_kernel<T, kFastGelu>), grid, dim3(256), 0, s, p, kSharedZ ? 0 : p.D);
  }
}

}  // namespace arctic

using namespace arctic;

static int sum_lstm_entry(const char *fn, bool shared_z, void *out_state, void *out_cell, const void *states,
                          const void *z, const int64_t *z_index, int64_t z_rows, const void *prev_cell, const void *w_cell, const void *b_cell,
                          const void *w_state, const void *b_state, int64_t rows, int D, int64_t s_stride,
                          int64_t z_stride, int64_t pc_stride, int64_t out_stride, float alpha, float eps_cell,
                          float eps_state, int fast_gelu, int dtype, void *stream) {
  if (dtype != ARCTIC_DTYPE_F16 && dtype != ARCTIC_DTYPE_BF16)
    return fail(ARCTIC_ERR_UNSUPPORTED, "%s: only fp16 and bf16 are supported.", fn);
  if (D <= 0) return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: last dim of states must be 4*D_gate", fn);
  if (rows < 0 || rows > 0x7fffffffLL) return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: bad row count", fn);
  if (rows == 0) return ARCTIC_OK;
  if (!out_state || !out_cell || !states || !z || !prev_cell)
    return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: null tensor pointer", fn);
  if (z_index && z_rows <= 0) return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: the embedding table has no rows", fn);
  LstmParams p;
  p.z_index = z_index;
  p.z_rows = z_rows;
  p.out_state = (char *)out_state;
  p.out_cell = (char *)out_cell;
  p.states = (const char *)states;
  p.z4 = (const char *)z;
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
  p.inv_D = 1.0f / (float)D;
  p.alpha = alpha;
  p.eps_cell = eps_cell;
  p.eps_state = eps_state;
  hipStream_t s = (hipStream_t)stream;
#define ARCTIC_LSTM_DISPATCH(TYPE)                                        \
  do {                                                                    \
    if (shared_z) {                                                       \
      if (fast_gelu) launch_lstm<TYPE, true, true>(p, rows, s);           \
      else launch_lstm<TYPE, false, true>(p, rows, s);                    \
    } else {                                                              \
      if (fast_gelu) launch_lstm<TYPE, true, false>(p, rows, s);          \
      else launch_lstm<TYPE, false, false>(p, rows, s);                   \
    }                                                                     \
  } while (0)
  if (dtype == ARCTIC_DTYPE_BF16) ARCTIC_LSTM_DISPATCH(BF16);
  else ARCTIC_LSTM_DISPATCH(F16);
#undef ARCTIC_LSTM_DISPATCH
  return check_launch(fn);
}

extern "C" int arctic_sum_lstm(void *out_state, void *out_cell, const void *states, const void *z4,
                               const void *prev_cell, const void *w_cell, const void *b_cell,
                               const void *w_state, const void *b_state, int64_t rows, int D,
                               int64_t s_stride, int64_t z_stride, int64_t pc_stride, int64_t out_stride,
                               float alpha, float eps_cell, float eps_state, int fast_gelu, int dtype,
                               void *stream) {
  return sum_lstm_entry("sum_lstm", false, out_state, out_cell, states, z4, nullptr, 0, prev_cell, w_cell, b_cell, w_state,
                        b_state, rows, D, s_stride, z_stride, pc_stride, out_stride, alpha, eps_cell, eps_state,
                        fast_gelu, dtype, stream);
}

extern "C" int arctic_sum_lstm_shared_z(void *out_state, void *out_cell, const void *states, const void *z,
                                        const void *prev_cell, const void *w_cell, const void *b_cell,
                                        const void *w_state, const void *b_state, int64_t rows, int D,
                                        int64_t s_stride, int64_t z_stride, int64_t pc_stride,
                                        int64_t out_stride, float alpha, float eps_cell, float eps_state,
                                        int fast_gelu, int dtype, void *stream) {
  return sum_lstm_entry("sum_lstm_shared_z", true, out_state, out_cell, states, z, nullptr, 0, prev_cell, w_cell, b_cell,
                        w_state, b_state, rows, D, s_stride, z_stride, pc_stride, out_stride, alpha, eps_cell,
                        eps_state, fast_gelu, dtype, stream);
}

extern "C" int arctic_sum_lstm_embedded(void *out_state, void *out_cell, const void *states, const void *emb_table,
                                        const int64_t *token_ids, const void *prev_cell, const void *w_cell,
                                        const void *b_cell, const void *w_state, const void *b_state, int64_t rows,
                                        int D, int64_t s_stride, int64_t emb_stride, int64_t pc_stride,
                                        int64_t out_stride, int64_t num_embeddings, float alpha, float eps_cell,
                                        float eps_state, int fast_gelu, int dtype, void *stream) {
  const char *fn = "sum_lstm_embedded";
  if (rows > 0 && !token_ids) return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: null token ids", fn);
  return sum_lstm_entry(fn, true, out_state, out_cell, states, emb_table, token_ids, num_embeddings, prev_cell, w_cell,
                        b_cell, w_state, b_state, rows, D, s_stride, emb_stride, pc_stride, out_stride, alpha, eps_cell,
                        eps_state, fast_gelu, dtype, stream);
}
