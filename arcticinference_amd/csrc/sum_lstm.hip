// Fused LSTM-style gate / cell / state update of the Arctic speculator, gfx950.
//
// Replaces sum_lstm_cuda and its kernels
// (csrc/custom_ops/sum_lstm.cu:14-473 in the reference).
//
// One workgroup per row.  On the vector paths each lane owns 16-byte chunks
// (8 elements) at the same column of all four gates of `states` and `z4` and of
// `prev_cell`: nine 16-byte loads per chunk.  The row then stays in registers
// across both RMS reductions, so HBM sees 9*D elements read and 2*D written per
// row (the reference re-reads the cell gate and reads out_cell back: 12*D).
// Sums are DPP wave reductions plus an LDS combine.  Three kernels:
// sum_lstm_staged_kernel (the speculator's shapes, rows of up to 8192 elements
// with all four vectors: the nine loads are requested in stages, between the
// stages of the arithmetic, one chunk per lane), sum_lstm_vec_kernel (every
// other shape with 16-byte accesses: the loads are requested together) and
// sum_lstm_scalar_kernel (any size and alignment, element by element).
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <algorithm>
#include <type_traits>

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
  int64_t rows;
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
// kEarlyOutputGate: the output gate's sigmoid runs ahead of the second row sum (rows of up to 4096 elements: by
// then the gate has arrived and the waves would otherwise idle at the barrier); it changes no result bit.
// A null prev_cell stands for a cell of zeros: the lanes then read the forget gate's address a second time and
// discard it.
template <int K>
struct LstmRow {
  Chunk sc[K], zc[K], sf[K], zf[K], si[K], zi[K], pc[K], so[K], zo[K];
};

template <typename T, int kChunksPerThread, bool kFastGelu, int kMaxThreads, bool kSharedZ, bool kEarlyOutputGate>
__global__ __launch_bounds__(kMaxThreads) void sum_lstm_vec_kernel(const LstmParams p) {
  __shared__ float slots_cpre[16];
  __shared__ float slots_cnew[16];
  constexpr int K = kChunksPerThread;
  constexpr int E = Chunk::kElems;
  using C = Chunk;
  const int D = p.D;
  const int chunks = D / E;
  const int64_t gate_bytes = (int64_t)D * 2;

  bool live[K];
  int64_t off[K];
  C wc[K], bc[K], ws[K], bs[K];
#pragma unroll
  for (int k = 0; k < K; ++k) {
    const int c = threadIdx.x + k * blockDim.x;
    live[k] = c < chunks;
    off[k] = (int64_t)(live[k] ? c : 0) * C::kBytes;  // idle lanes re-read chunk 0 and discard it
  }
  // The scale / shift vectors are the same for every row (cache resident).  They
  // are requested first: memory returns loads in issue order, so asking for them
  // later would park the arithmetic behind the whole row.
#pragma unroll
  for (int k = 0; k < K; ++k) {
    if (p.w_cell) wc[k] = C::load(p.w_cell + off[k]);
    if (p.b_cell) bc[k] = C::load(p.b_cell + off[k]);
    if (p.w_state) ws[k] = C::load(p.w_state + off[k]);
    if (p.b_state) bs[k] = C::load(p.b_state + off[k]);
  }

  const int64_t row = blockIdx.x;
  LstmRow<K> r;
  {
    const char *s_row = p.states + row * p.s_stride * 2;
    int64_t zr = row;
    if (kSharedZ && p.z_index) zr = min(max(p.z_index[row], (int64_t)0), p.z_rows - 1);
    const char *z_row = p.z4 + zr * p.z_stride * 2;
    const char *pc_row = p.prev_cell ? p.prev_cell + row * p.pc_stride * 2 : s_row;
#pragma unroll
    for (int k = 0; k < K; ++k) {
      r.zc[k] = C::load_stream(z_row + (kSharedZ ? 0 : 3 * gate_bytes) + off[k]);
      r.sc[k] = C::load_stream(s_row + 3 * gate_bytes + off[k]);
    }
#pragma unroll
    for (int k = 0; k < K; ++k) {
      r.sf[k] = C::load_stream(s_row + off[k]);
      r.zf[k] = kSharedZ ? r.zc[k] : C::load_stream(z_row + off[k]);
    }
    // (the previous cell and both outputs stream like the gates: a launch boundary writes the outputs back anyway,
    // and streaming stores leave the CU earlier - measured on the staged kernel below)
#pragma unroll
    for (int k = 0; k < K; ++k) r.pc[k] = C::load_stream(pc_row + off[k]);
#pragma unroll
    for (int k = 0; k < K; ++k) {
      r.si[k] = C::load_stream(s_row + gate_bytes + off[k]);
      r.zi[k] = kSharedZ ? r.zc[k] : C::load_stream(z_row + gate_bytes + off[k]);
    }
#pragma unroll
    for (int k = 0; k < K; ++k) {
      r.so[k] = C::load_stream(s_row + 2 * gate_bytes + off[k]);
      r.zo[k] = kSharedZ ? r.zc[k] : C::load_stream(z_row + 2 * gate_bytes + off[k]);
    }
  }

  char *oc_row = p.out_cell + row * p.out_stride * 2;
  char *os_row = p.out_state + row * p.out_stride * 2;
  // Lanes beyond the row take part in the sums with zeros.  (Each value is
  // cleared where it is first used, not here: touching pc now would wait for it.)
  // phase 1: pre_c and its sum of squares (reference :65-82); needs the cell gate only
  float cact[K][E];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < K; ++k) {
    float a[E], b[E];
    if (!live[k]) r.sc[k] = r.zc[k] = C::zero();
    r.sc[k].template unpack<T>(a);
    r.zc[k].template unpack<T>(b);
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
    if (p.w_cell) wc[k].template unpack<T>(w);
    if (p.b_cell) bc[k].template unpack<T>(b);
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
    r.sf[k].template unpack<T>(a);
    r.zf[k].template unpack<T>(b);
    if (!live[k] || !p.prev_cell) r.pc[k] = C::zero();
    r.pc[k].template unpack<T>(c);
#pragma unroll
    for (int j = 0; j < E; ++j) cell[k][j] = sigmoid_f(fmaf(p.alpha, b[j], a[j])) * c[j];
    // keep the forget-gate arithmetic ahead of the wait for the input gate: it then runs while that gate
    // is still arriving instead of in the short stretch between the last two gates
    __builtin_amdgcn_sched_barrier(0);
    r.si[k].template unpack<T>(a);
    r.zi[k].template unpack<T>(b);
#pragma unroll
    for (int j = 0; j < E; ++j) {
      const float cnew = fmaf(cact[k][j], sigmoid_f(fmaf(p.alpha, b[j], a[j])), cell[k][j]);
      ss = fmaf(cnew, cnew, ss);  // unrounded, as in the reference (:136)
      cell[k][j] = cnew;
    }
    const C packed = C::template pack<T>(cell[k]);
    if (live[k]) packed.store_stream(oc_row + off[k]);
    packed.template unpack<T>(cell[k]);
  }
  float og[K][E];
  if constexpr (kEarlyOutputGate) {
#pragma unroll
    for (int k = 0; k < K; ++k) {
      float a[E], g[E];
      r.so[k].template unpack<T>(a);
      r.zo[k].template unpack<T>(g);
#pragma unroll
      for (int j = 0; j < E; ++j) og[k][j] = sigmoid_f(fmaf(p.alpha, g[j], a[j]));
    }
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
    if (p.w_state) ws[k].template unpack<T>(w);
    if (p.b_state) bs[k].template unpack<T>(b);
#pragma unroll
    for (int j = 0; j < E; ++j) st[j] = gelu<kFastGelu>(fmaf(cell[k][j] * inv_cnew, w[j], b[j]));
    if constexpr (kEarlyOutputGate) {
#pragma unroll
      for (int j = 0; j < E; ++j) st[j] *= og[k][j];
    } else {
      float a[E], g[E];
      r.so[k].template unpack<T>(a);
      r.zo[k].template unpack<T>(g);
#pragma unroll
      for (int j = 0; j < E; ++j) st[j] *= sigmoid_f(fmaf(p.alpha, g[j], a[j]));
    }
    if (live[k]) C::template pack<T>(st).store_stream(os_row + off[k]);
  }
}

// The speculator's shape (every lane owns one 16-byte chunk of the row, all four scale / shift vectors given) with the
// requests of a row issued in stages.  A CU accepts vector-memory requests only as fast as HBM answers them: a wave
// that asks for its nine chunks at once sits in the ninth request for microseconds, long after the first chunks have
// arrived and with nothing computed, and the younger workgroup of the CU does not get its first request in before
// the older one's last.  Here a wave requests its chunks in the order cell gate z, s; forget gate s, z; previous
// cell; input gate s, z; output gate s, z, at four points of its arithmetic (the best of a sweep over the request
// points at 512 rows of 4096):
//   - the cell gate (2 chunks) at the start, with the cell norm's scale / shift pair right behind it;
//   - the forget gate's s behind the first sum of squares;
//   - the rest of the forget gate, the previous cell and the input gate behind the candidate's GELU, the state
//     norm's pair just ahead of them, and a workgroup barrier that waits for no memory behind them, so that every
//     wave of the row has made these requests before any wave makes the next ones;
//   - the output gate behind the forget gate's part of the cell update; it is consumed last, after the state's GELU.
// Waves that are computing leave the request slots to the others, so both rows of a CU arrive gate by gate and every
// stage's arithmetic runs while the next stage is in flight.  The scale / shift vectors (the same for every row,
// cache resident) are requested where they are needed, not ahead of the row: a wave's requests come back in the order
// they were made.  Both outputs are stored and the previous cell is read with streaming accesses (a step's outputs
// are read by the next launches of the step, but a launch boundary writes them back anyway, and stores that stream
// leave earlier).
//
// Same arithmetic, operation for operation, as sum_lstm_vec_kernel: results are bit-identical.
// kMaxLanes: 512 for rows of up to 4096 elements, 1024 (half the registers per lane) for rows of up to 8192.
// kRagged: the row's chunks do not fill the last wave; the lanes behind the last chunk run along on that chunk (the
// barriers need every wave), add nothing to the row sums and store nothing.
// kZeroCell: the previous cell is all zeros (the first step of a proposal round) and is not read.
template <typename T, bool kFastGelu, bool kSharedZ, bool kZeroCell, int kMaxLanes, bool kRagged>
__global__ __launch_bounds__(kMaxLanes) void sum_lstm_staged_kernel(const LstmParams p) {
  __shared__ float slots_cpre[16];
  __shared__ float slots_cnew[16];
  constexpr int E = Chunk::kElems;
  using C = Chunk;
  using std::integral_constant;
  const int64_t row = blockIdx.x;
  const bool active = !kRagged || (int)threadIdx.x < p.D / E;
  const int64_t off = (int64_t)(kRagged ? min((int)threadIdx.x, p.D / E - 1) : (int)threadIdx.x) * C::kBytes;
  const int64_t gate_bytes = (int64_t)p.D * 2;
  const char *s_row = p.states + row * p.s_stride * 2 + off;
  int64_t zr = row;
  if (kSharedZ && p.z_index) zr = min(max(p.z_index[row], (int64_t)0), p.z_rows - 1);
  const char *z_row = p.z4 + zr * p.z_stride * 2 + off;
  const char *pc_row = kZeroCell ? s_row : p.prev_cell + row * p.pc_stride * 2 + off;
  char *oc_row = p.out_cell + row * p.out_stride * 2 + off;
  char *os_row = p.out_state + row * p.out_stride * 2 + off;

  C in[9];   // zc sc sf zf pc si zi so zo; with kSharedZ the one z chunk stands for all four, with kZeroCell pc is unused
  // requests chunks kFrom ... kTo - 1 of the list above
  auto request = [&](auto from, auto to) {
    constexpr int kFrom = decltype(from)::value, kTo = decltype(to)::value;
    __builtin_amdgcn_sched_barrier(0);   // neither hoisted above the arithmetic in front nor sunk below what follows
    if constexpr (kFrom <= 0 && 0 < kTo) in[0] = C::load_stream(z_row + (kSharedZ ? 0 : 3 * gate_bytes));
    if constexpr (kFrom <= 1 && 1 < kTo) in[1] = C::load_stream(s_row + 3 * gate_bytes);
    if constexpr (kFrom <= 2 && 2 < kTo) in[2] = C::load_stream(s_row);
    if constexpr (kFrom <= 3 && 3 < kTo && !kSharedZ) in[3] = C::load_stream(z_row);
    if constexpr (kFrom <= 4 && 4 < kTo && !kZeroCell) in[4] = C::load_stream(pc_row);
    if constexpr (kFrom <= 5 && 5 < kTo) in[5] = C::load_stream(s_row + gate_bytes);
    if constexpr (kFrom <= 6 && 6 < kTo && !kSharedZ) in[6] = C::load_stream(z_row + gate_bytes);
    if constexpr (kFrom <= 7 && 7 < kTo) in[7] = C::load_stream(s_row + 2 * gate_bytes);
    if constexpr (kFrom <= 8 && 8 < kTo && !kSharedZ) in[8] = C::load_stream(z_row + 2 * gate_bytes);
    __builtin_amdgcn_sched_barrier(0);
  };
  request(integral_constant<int, 0>(), integral_constant<int, 2>());
  const C wc = C::load(p.w_cell + off);
  const C bc = C::load(p.b_cell + off);

  // phase 1: pre_c and its sum of squares (reference :65-82)
  float cact[E], a[E], b[E], c[E];
  float ss = 0.f;
  in[1].template unpack<T>(a);
  in[0].template unpack<T>(b);
#pragma unroll
  for (int j = 0; j < E; ++j) {
    cact[j] = fmaf(p.alpha, b[j], a[j]);
    ss = fmaf(cact[j], cact[j], ss);
  }
  request(integral_constant<int, 2>(), integral_constant<int, 3>());
  const float inv_cpre = rsqrtf(block_sum(active ? ss : 0.f, slots_cpre) * p.inv_D + p.eps_cell);
  {
    float w[E], sh[E];
    wc.template unpack<T>(w);
    bc.template unpack<T>(sh);
#pragma unroll
    for (int j = 0; j < E; ++j) cact[j] = gelu<kFastGelu>(fmaf(cact[j] * inv_cpre, w[j], sh[j]));
  }
  const C ws = C::load(p.w_state + off);
  const C bs = C::load(p.b_state + off);
  request(integral_constant<int, 3>(), integral_constant<int, 7>());
  __builtin_amdgcn_s_barrier();   // waits for no memory: only keeps the row's waves in step at their largest group of requests
  __builtin_amdgcn_sched_barrier(0);

  // phase 2: cell update; write out_cell (reference :104-140)
  float cell[E];
  in[2].template unpack<T>(a);
  (kSharedZ ? in[0] : in[3]).template unpack<T>(b);
  (kZeroCell ? C::zero() : in[4]).template unpack<T>(c);
#pragma unroll
  for (int j = 0; j < E; ++j) cell[j] = sigmoid_f(fmaf(p.alpha, b[j], a[j])) * c[j];
  __builtin_amdgcn_sched_barrier(0);   // the forget gate's part stays ahead of the wait for the input gate
  in[5].template unpack<T>(a);
  (kSharedZ ? in[0] : in[6]).template unpack<T>(b);
  ss = 0.f;
#pragma unroll
  for (int j = 0; j < E; ++j) {
    const float cnew = fmaf(cact[j], sigmoid_f(fmaf(p.alpha, b[j], a[j])), cell[j]);
    ss = fmaf(cnew, cnew, ss);  // unrounded, as in the reference (:136)
    cell[j] = cnew;
  }
  {
    const C packed = C::template pack<T>(cell);
    if (active) packed.store_stream(oc_row);
    packed.template unpack<T>(cell);   // the state phase sees the rounded cell (:163,174)
  }
  request(integral_constant<int, 7>(), integral_constant<int, 9>());
  const float inv_cnew = rsqrtf(block_sum(active ? ss : 0.f, slots_cnew) * p.inv_D + p.eps_state);

  // phase 3: state = gelu(rmsnorm(rounded cell)) * sigmoid(pre_o) (reference :160-190)
  float st[E];
  {
    float w[E], sh[E];
    ws.template unpack<T>(w);
    bs.template unpack<T>(sh);
#pragma unroll
    for (int j = 0; j < E; ++j) st[j] = gelu<kFastGelu>(fmaf(cell[j] * inv_cnew, w[j], sh[j]));
  }
  __builtin_amdgcn_sched_barrier(0);   // the GELU above runs while the output gate is still on its way
  in[7].template unpack<T>(a);
  (kSharedZ ? in[0] : in[8]).template unpack<T>(b);
#pragma unroll
  for (int j = 0; j < E; ++j) st[j] *= sigmoid_f(fmaf(p.alpha, b[j], a[j]));
  if (active) C::template pack<T>(st).store_stream(os_row);
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
    const float cnew = (p.prev_cell ? T::lo(pc[j]) : 0.f) * sigmoid_f(pre_f) + gelu<kFastGelu>(cn) * sigmoid_f(pre_i);
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
                   aligned16(p.states) && aligned16(p.z4) && aligned16(p.prev_cell) &&   /* null counts as aligned */
                   aligned16(p.out_state) && aligned16(p.out_cell) && aligned16(p.w_cell) &&
                   aligned16(p.b_cell) && aligned16(p.w_state) && aligned16(p.b_state);
  const dim3 grid((unsigned)rows);
  if (vec) {
    const int cpt = chunks > 512 ? 2 : 1;   // one 16-byte chunk per lane up to 512 lanes (D <= 4096)
    int threads = (chunks + cpt - 1) / cpt;
    threads = std::max(64, (threads + 63) & ~63);
    // All four vectors given and a row of up to 8192 elements: the staged kernel, one chunk per lane (512 rows of
    // 5120 / 6144 / 8192 elements: 12.0 / 13.9 / 17.9 us against 17.6 / 19.9 / 22.5 us with two chunks per lane in the
    // kernel below), with idle lanes in the last wave when the row is no multiple of 512 elements.
    const bool staged = chunks <= 1024 && p.w_cell && p.b_cell && p.w_state && p.b_state;
    const int lanes = (chunks + 63) & ~63;
#define ARCTIC_LSTM_STAGED_LAUNCH(ZERO, MAX_LANES, RAGGED)                                                \
  hipLaunchKernelGGL((sum_lstm_staged_kernel<T, kFastGelu, kSharedZ, ZERO, MAX_LANES, RAGGED>), grid, dim3(lanes), 0, \
                     s, p)
    if (staged) {
      const bool zero = !p.prev_cell, ragged = lanes != chunks;
      if (chunks <= 512) {
        if (zero && ragged) ARCTIC_LSTM_STAGED_LAUNCH(true, 512, true);
        else if (zero) ARCTIC_LSTM_STAGED_LAUNCH(true, 512, false);
        else if (ragged) ARCTIC_LSTM_STAGED_LAUNCH(false, 512, true);
        else ARCTIC_LSTM_STAGED_LAUNCH(false, 512, false);
      } else {
        if (zero && ragged) ARCTIC_LSTM_STAGED_LAUNCH(true, 1024, true);
        else if (zero) ARCTIC_LSTM_STAGED_LAUNCH(true, 1024, false);
        else if (ragged) ARCTIC_LSTM_STAGED_LAUNCH(false, 1024, true);
        else ARCTIC_LSTM_STAGED_LAUNCH(false, 1024, false);
      }
    }
#undef ARCTIC_LSTM_STAGED_LAUNCH
    else if (cpt == 1)
      hipLaunchKernelGGL((sum_lstm_vec_kernel<T, 1, kFastGelu, 512, kSharedZ, true>), grid, dim3(threads), 0, s, p);
    else
      hipLaunchKernelGGL((sum_lstm_vec_kernel<T, 2, kFastGelu, 1024, kSharedZ, false>), grid, dim3(threads), 0, s, p);
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
  if (!out_state || !out_cell || !states || !z)   // prev_cell may be null: a cell of zeros
    return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: null tensor pointer", fn);
  if (z_index && z_rows <= 0) return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: the embedding table has no rows", fn);
  if (D > (1 << 28)) return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: D_gate beyond 2^28", fn);
  if (!pitch_ok(s_stride, rows, 2) || !pitch_ok(z_stride, z_index ? z_rows : rows, 2) ||
      !pitch_ok(pc_stride, rows, 2) || !pitch_ok(out_stride, rows, 2))
    return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: row pitch out of range", fn);
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
  p.pc_stride = prev_cell ? pc_stride : 0;
  p.out_stride = out_stride;
  p.rows = rows;
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
