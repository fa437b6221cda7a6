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
#include <cstdlib>
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
#ifdef ARCTIC_TUNING
  unsigned long long *trace;   // measurement build: time stamps of sum_lstm_staged_kernel<..., kTrace>, or nullptr
#endif
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
// kRows: rows per workgroup (consecutive).  With two, the second row's loads are issued right behind the
// first row's, so the first row's arithmetic runs while the second row is still arriving.
// kZeroCell: the previous cell is all zeros (the first step of a proposal round) and is not read.  Without this
// flag a null prev_cell is still honoured: the lanes then read the forget gate's address a second time and
// discard it.
// kVariant: bit 0: input gate loaded and consumed before the forget gate and the previous cell; bit 1: the
// output gate's sigmoid ahead of the second row sum (what the library ships for rows of up to 4096: by then the
// gate has arrived and the waves would otherwise idle at the barrier); bit 2: one reciprocal shared by the
// sigmoids and the GELU of a phase; bit 3: a workgroup barrier (no memory wait) between the groups of requests, so
// that every wave of the row has requested a gate before any wave requests the next one.  Built for tuning, the
// combinations that the benchmark times can be selected at run time.
template <typename C, int K>
struct LstmRow {
  C sc[K], zc[K], sf[K], zf[K], si[K], zi[K], pc[K], so[K], zo[K];
};

enum : int { kLstmInputGateFirst = 1, kLstmEarlyOutputGate = 2, kLstmSharedReciprocal = 4, kLstmLoadGroupBarriers = 8 };

template <typename T, int E, int kChunksPerThread, bool kFastGelu, int kMaxThreads, bool kSharedZ, bool kAllVectors,
          int kRows, int kVariant, bool kZeroCell = false>
__global__ __launch_bounds__(kMaxThreads) void sum_lstm_vec_kernel(const LstmParams p) {
  __shared__ float slots_cpre[kRows][16];
  __shared__ float slots_cnew[kRows][16];
  constexpr int K = kChunksPerThread;
  using C = Chunk<E>;
  const int D = p.D;
  const int chunks = D / E;
  const int64_t gate_bytes = (int64_t)D * 2;

  bool live[K];
  int64_t off[K];
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

  LstmRow<C, K> in[kRows];
  auto issue_loads = [&](int64_t row, LstmRow<C, K> &r) {
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
    auto forget_and_cell = [&]() {
#pragma unroll
      for (int k = 0; k < K; ++k) {
        r.sf[k] = C::load_stream(s_row + off[k]);
        r.zf[k] = kSharedZ ? r.zc[k] : C::load_stream(z_row + off[k]);
      }
      // (the previous cell and both outputs stream like the gates: a launch boundary writes the outputs back anyway,
      // and streaming stores leave the CU earlier - measured on the staged kernel below)
      if constexpr (!kZeroCell) {
#pragma unroll
        for (int k = 0; k < K; ++k) r.pc[k] = C::load_stream(pc_row + off[k]);
      }
    };
    auto input_gate = [&]() {
#pragma unroll
      for (int k = 0; k < K; ++k) {
        r.si[k] = C::load_stream(s_row + gate_bytes + off[k]);
        r.zi[k] = kSharedZ ? r.zc[k] : C::load_stream(z_row + gate_bytes + off[k]);
      }
    };
    // the groups must reach memory in this order (it returns loads in issue order); with more than one row per
    // workgroup the compiler would otherwise interleave the rows' loads
    auto fence = [&]() {
      if constexpr (kVariant & kLstmLoadGroupBarriers) {
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_barrier();   // no memory wait: only the order in which the waves issue their requests
        __builtin_amdgcn_sched_barrier(0);
      } else if constexpr (kRows > 1) {
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    fence();
    if constexpr (kVariant & kLstmInputGateFirst) {
      input_gate();
      fence();
      forget_and_cell();
    } else {
      forget_and_cell();
      fence();
      input_gate();
    }
    fence();
#pragma unroll
    for (int k = 0; k < K; ++k) {
      r.so[k] = C::load_stream(s_row + 2 * gate_bytes + off[k]);
      r.zo[k] = kSharedZ ? r.zc[k] : C::load_stream(z_row + 2 * gate_bytes + off[k]);
    }
    if constexpr (kRows > 1) __builtin_amdgcn_sched_barrier(0);
  };

  auto compute = [&](int64_t row, LstmRow<C, K> &r, float *slots_a, float *slots_b) {
    char *oc_row = p.out_cell + row * p.out_stride * 2;
    char *os_row = p.out_state + row * p.out_stride * 2;
    if constexpr (kRows > 1) __builtin_amdgcn_sched_barrier(0);   // one row's arithmetic after the other's
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
    const float inv_cpre = rsqrtf(block_sum(ss, slots_a) * p.inv_D + p.eps_cell);
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
      if constexpr (kVariant & kLstmInputGateFirst) {
        float gi[E];
        r.si[k].template unpack<T>(a);
        r.zi[k].template unpack<T>(b);
#pragma unroll
        for (int j = 0; j < E; ++j) gi[j] = sigmoid_f(fmaf(p.alpha, b[j], a[j]));
        __builtin_amdgcn_sched_barrier(0);
        r.sf[k].template unpack<T>(a);
        r.zf[k].template unpack<T>(b);
#pragma unroll
        for (int j = 0; j < E; ++j) cell[k][j] = sigmoid_f(fmaf(p.alpha, b[j], a[j]));
        __builtin_amdgcn_sched_barrier(0);
        if (kZeroCell || !live[k] || !p.prev_cell) r.pc[k] = C::zero();
        r.pc[k].template unpack<T>(c);
#pragma unroll
        for (int j = 0; j < E; ++j) {
          const float cnew = fmaf(cact[k][j], gi[j], cell[k][j] * c[j]);
          ss = fmaf(cnew, cnew, ss);  // unrounded, as in the reference (:136)
          cell[k][j] = cnew;
        }
      } else {
        r.sf[k].template unpack<T>(a);
        r.zf[k].template unpack<T>(b);
        if (kZeroCell || !live[k] || !p.prev_cell) r.pc[k] = C::zero();
        r.pc[k].template unpack<T>(c);
        if constexpr ((kVariant & kLstmSharedReciprocal) && !kFastGelu) {
          // c_new = (pc (1 + e_i) + cand (1 + e_f)) / ((1 + e_f)(1 + e_i)): one reciprocal for both gates
          float df[E];
#pragma unroll
          for (int j = 0; j < E; ++j) df[j] = sigmoid_den(fmaf(p.alpha, b[j], a[j]));
          r.si[k].template unpack<T>(a);
          r.zi[k].template unpack<T>(b);
#pragma unroll
          for (int j = 0; j < E; ++j) {
            const float di = sigmoid_den(fmaf(p.alpha, b[j], a[j]));
            const float num = fmaf(cact[k][j], df[j], c[j] * di);
            const float cnew = num * __builtin_amdgcn_rcpf(df[j] * di);
            ss = fmaf(cnew, cnew, ss);
            cell[k][j] = cnew;
          }
        } else {
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
        }
      }
      const C packed = C::template pack<T>(cell[k]);
      if (live[k]) packed.store_stream(oc_row + off[k]);
      packed.template unpack<T>(cell[k]);
    }
    float og[K][E];
    if constexpr (kVariant & kLstmEarlyOutputGate) {
#pragma unroll
      for (int k = 0; k < K; ++k) {
        float a[E], g[E];
        r.so[k].template unpack<T>(a);
        r.zo[k].template unpack<T>(g);
#pragma unroll
        for (int j = 0; j < E; ++j) og[k][j] = sigmoid_f(fmaf(p.alpha, g[j], a[j]));
      }
    }
    const float inv_cnew = rsqrtf(block_sum(ss, slots_b) * p.inv_D + p.eps_state);

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
      if constexpr ((kVariant & kLstmSharedReciprocal) && !kFastGelu) {
        // the GELU's reciprocal and the output gate's from one: 1 / (u v), times v, times u
        float a[E], g[E];
        r.so[k].template unpack<T>(a);
        r.zo[k].template unpack<T>(g);
#pragma unroll
        for (int j = 0; j < E; ++j) {
          const float x = fmaf(cell[k][j] * inv_cnew, w[j], b[j]);
          const float u = gelu_erf_den(x), v = sigmoid_den(fmaf(p.alpha, g[j], a[j]));
          const float rcp = __builtin_amdgcn_rcpf(u * v);
          st[j] = gelu_erf_given_t(x, rcp * v) * (rcp * u);
        }
        if (live[k]) C::template pack<T>(st).store_stream(os_row + off[k]);
        continue;
      }
#pragma unroll
      for (int j = 0; j < E; ++j) st[j] = gelu<kFastGelu>(fmaf(cell[k][j] * inv_cnew, w[j], b[j]));
      if constexpr (kVariant & kLstmEarlyOutputGate) {
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
  };

  const int64_t row0 = (int64_t)blockIdx.x * kRows;
  // every row's loads are issued unconditionally (a workgroup past the last row reads that row again and drops
  // it): loads behind a branch would make the waits below count as if they had not been issued
#pragma unroll
  for (int r = 0; r < kRows; ++r) issue_loads(min(row0 + r, p.rows - 1), in[r]);
#pragma unroll
  for (int r = 0; r < kRows; ++r)
    if (r == 0 || row0 + r < p.rows) compute(row0 + r, in[r], slots_cpre[r], slots_cnew[r]);
}

// The speculator's shape (every lane owns one 16-byte chunk of the row, all four scale / shift vectors given) with the
// requests of a row issued in stages.  A CU accepts vector-memory requests only as fast as HBM answers them: a wave
// that asks for its nine chunks at once sits in the ninth request for microseconds, long after the first chunks have
// arrived and with nothing computed, and the younger workgroup of the CU does not get its first request in before
// the older one's last (time stamps of the waves: bench.py --lstm-timeline).  Here a wave requests the first kAhead0
// chunks (order: cell gate z, s; forget gate s, z; previous cell; input gate s, z; output gate s, z), starts on the
// cell gate as soon as that is in, and requests the rest at four later points of its arithmetic: kAhead1 chunks are
// out after the first sum of squares, kAhead2 after the candidate's GELU, kAhead3 after the forget gate's part of
// the cell update, all nine once the new cell is stored.  Waves that are computing leave the request slots to the
// others, so both rows of a CU arrive gate by gate and every stage's arithmetic runs while the next stage is in flight.
// kBarriers: bit k = a workgroup barrier that waits for no memory behind the requests of point k (0: the first
// chunks, 2: after the candidate's GELU, 3: after the forget gate's part; point 1 is followed by the first row sum's
// barrier anyway).  kVectors places the requests for the scale / shift vectors (the same for every row, cache resident): 0: all four
// ahead of the row; 1: the cell norm's pair behind the first sum of squares, the state norm's behind the forget
// gate's part; 2: the cell norm's pair right behind the first kAhead0 chunks, the state norm's behind the candidate's
// GELU.  kStreamOutputs / kStreamCell: non-temporal stores of both outputs / load of the previous cell (a step's
// outputs are read by the next launches of the step, but a launch boundary writes them back anyway, and stores that
// stream leave earlier).
template <int kAhead0_, int kAhead1_, int kAhead2_, int kAhead3_, bool kEarlyGate_, int kVectors_, bool kStreamOutputs_,
          bool kStreamCell_, int kBarriers_ = 0>
struct LstmSchedule {
  static constexpr int kBarriers = kBarriers_;   // bit k: a workgroup barrier (no memory wait) behind the requests of point k
  static constexpr int kAhead0 = kAhead0_, kAhead1 = kAhead1_, kAhead2 = kAhead2_, kAhead3 = kAhead3_;
  static constexpr bool kEarlyGate = kEarlyGate_, kStreamOutputs = kStreamOutputs_, kStreamCell = kStreamCell_;
  static constexpr int kVectors = kVectors_;
  static_assert(kAhead0 >= 2 && kAhead1 >= kAhead0 && kAhead2 >= 5 && kAhead2 >= kAhead1 && kAhead3 >= 7 &&
                    kAhead3 >= kAhead2 && kAhead3 <= 9,
                "a chunk must be requested before the arithmetic that reads it");
};
// measured best of a sweep over the request points (512 rows of 4096): the cell gate first, the forget gate's s
// behind the first sum of squares, the rest of the forget gate, the previous cell and the input gate behind the
// candidate's GELU, with a workgroup barrier (no memory wait) behind them, so that every wave of the row has made
// these requests before any wave makes the next ones; the output gate behind the forget gate's part; the output gate
// is consumed last
using LstmShippedSchedule = LstmSchedule<2, 3, 7, 7, false, 2, true, true, 4>;

// Same arithmetic, operation for operation, as sum_lstm_vec_kernel: results are bit-identical.
// kMaxLanes: 512 for rows of up to 4096 elements, 1024 (half the registers per lane) for rows of up to 8192.
// kRagged: the row's chunks do not fill the last wave; the lanes behind the last chunk run along on that chunk (the
// barriers need every wave), add nothing to the row sums and store nothing.
template <typename T, bool kFastGelu, bool kSharedZ, bool kZeroCell, typename S = LstmShippedSchedule, bool kTrace = false,
          int kMaxLanes = 512, bool kRagged = false>
__global__ __launch_bounds__(kMaxLanes) void sum_lstm_staged_kernel(const LstmParams p) {
  __shared__ float slots_cpre[16];
  __shared__ float slots_cnew[16];
  constexpr int E = 8;
  using C = Chunk<E>;
  using std::integral_constant;
  const int64_t row = blockIdx.x;
  const bool active = !kRagged || (int)threadIdx.x < p.D / E;
  const int64_t off = (int64_t)(kRagged ? min((int)threadIdx.x, p.D / E - 1) : (int)threadIdx.x) * C::kBytes;
  const int64_t gate_bytes = (int64_t)p.D * 2;
  // measurement build: the constant-rate clock (100 MHz) at eight points of a wave's life, written by its first lane
  auto stamp = [&](int k) {
#ifdef ARCTIC_TUNING
    if constexpr (kTrace) {
      __builtin_amdgcn_sched_barrier(0);
      const unsigned long long t = __builtin_amdgcn_s_memrealtime();
      if (p.trace && (threadIdx.x & 63) == 0) p.trace[((size_t)blockIdx.x * 8 + threadIdx.x / 64) * 8 + k] = t;
      __builtin_amdgcn_sched_barrier(0);
    }
#endif
  };
  stamp(0);   // the wave has started
  C wc, bc, ws, bs;
  auto request_vectors = [&](int place) {
    if (place == (S::kVectors == 0 ? 0 : S::kVectors == 1 ? 2 : 1)) {
      wc = C::load(p.w_cell + off);
      bc = C::load(p.b_cell + off);
    }
    if (place == (S::kVectors == 0 ? 0 : S::kVectors == 1 ? 4 : 3)) {
      ws = C::load(p.w_state + off);
      bs = C::load(p.b_state + off);
    }
  };
  request_vectors(0);
  const char *s_row = p.states + row * p.s_stride * 2 + off;
  int64_t zr = row;
  if (kSharedZ && p.z_index) zr = min(max(p.z_index[row], (int64_t)0), p.z_rows - 1);
  const char *z_row = p.z4 + zr * p.z_stride * 2 + off;
  const char *pc_row = kZeroCell ? s_row : p.prev_cell + row * p.pc_stride * 2 + off;
  char *oc_row = p.out_cell + row * p.out_stride * 2 + off;
  char *os_row = p.out_state + row * p.out_stride * 2 + off;

  C in[9];   // zc sc sf zf pc si zi so zo; with kSharedZ the one z chunk stands for all four, with kZeroCell pc is unused
  auto request = [&](auto from, auto to) {
    constexpr int kFrom = decltype(from)::value, kTo = decltype(to)::value;
    __builtin_amdgcn_sched_barrier(0);   // neither hoisted above the arithmetic in front nor sunk below what follows
    if constexpr (kFrom <= 0 && 0 < kTo) in[0] = C::load_stream(z_row + (kSharedZ ? 0 : 3 * gate_bytes));
    if constexpr (kFrom <= 1 && 1 < kTo) in[1] = C::load_stream(s_row + 3 * gate_bytes);
    if constexpr (kFrom <= 2 && 2 < kTo) in[2] = C::load_stream(s_row);
    if constexpr (kFrom <= 3 && 3 < kTo && !kSharedZ) in[3] = C::load_stream(z_row);
    if constexpr (kFrom <= 4 && 4 < kTo && !kZeroCell) in[4] = S::kStreamCell ? C::load_stream(pc_row) : C::load(pc_row);
    if constexpr (kFrom <= 5 && 5 < kTo) in[5] = C::load_stream(s_row + gate_bytes);
    if constexpr (kFrom <= 6 && 6 < kTo && !kSharedZ) in[6] = C::load_stream(z_row + gate_bytes);
    if constexpr (kFrom <= 7 && 7 < kTo) in[7] = C::load_stream(s_row + 2 * gate_bytes);
    if constexpr (kFrom <= 8 && 8 < kTo && !kSharedZ) in[8] = C::load_stream(z_row + 2 * gate_bytes);
    __builtin_amdgcn_sched_barrier(0);
  };
  auto in_step = [&](int point) {
    if ((S::kBarriers >> point) & 1) {
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  request(integral_constant<int, 0>(), integral_constant<int, S::kAhead0>());
  in_step(0);
  request_vectors(1);
  stamp(1);   // the first requests are out

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
  stamp(2);   // the cell gate is in, its squares are summed
  request_vectors(2);
  request(integral_constant<int, S::kAhead0>(), integral_constant<int, S::kAhead1>());
  const float inv_cpre = rsqrtf(block_sum(active ? ss : 0.f, slots_cpre) * p.inv_D + p.eps_cell);
  stamp(3);   // first row sum known
  {
    float w[E], sh[E];
    wc.template unpack<T>(w);
    bc.template unpack<T>(sh);
#pragma unroll
    for (int j = 0; j < E; ++j) cact[j] = gelu<kFastGelu>(fmaf(cact[j] * inv_cpre, w[j], sh[j]));
  }
  request_vectors(3);
  request(integral_constant<int, S::kAhead1>(), integral_constant<int, S::kAhead2>());
  in_step(2);

  // phase 2: cell update; write out_cell (reference :104-140)
  float cell[E];
  in[2].template unpack<T>(a);
  (kSharedZ ? in[0] : in[3]).template unpack<T>(b);
  (kZeroCell ? C::zero() : in[4]).template unpack<T>(c);
#pragma unroll
  for (int j = 0; j < E; ++j) cell[j] = sigmoid_f(fmaf(p.alpha, b[j], a[j])) * c[j];
  request_vectors(4);
  request(integral_constant<int, S::kAhead2>(), integral_constant<int, S::kAhead3>());
  in_step(3);
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
    if (active) {
      if constexpr (S::kStreamOutputs) packed.store_stream(oc_row);
      else packed.store(oc_row);
    }
    packed.template unpack<T>(cell);   // the state phase sees the rounded cell (:163,174)
  }
  stamp(4);   // forget gate, previous cell and input gate are in; the new cell is stored
  request(integral_constant<int, S::kAhead3>(), integral_constant<int, 9>());
  float og[E];
  if constexpr (S::kEarlyGate) {
    in[7].template unpack<T>(a);
    (kSharedZ ? in[0] : in[8]).template unpack<T>(b);
#pragma unroll
    for (int j = 0; j < E; ++j) og[j] = sigmoid_f(fmaf(p.alpha, b[j], a[j]));
    __builtin_amdgcn_sched_barrier(0);
  }
  const float inv_cnew = rsqrtf(block_sum(active ? ss : 0.f, slots_cnew) * p.inv_D + p.eps_state);
  stamp(5);   // second row sum known

  // phase 3: state = gelu(rmsnorm(rounded cell)) * sigmoid(pre_o) (reference :160-190)
  float st[E];
  {
    float w[E], sh[E];
    ws.template unpack<T>(w);
    bs.template unpack<T>(sh);
#pragma unroll
    for (int j = 0; j < E; ++j) st[j] = gelu<kFastGelu>(fmaf(cell[j] * inv_cnew, w[j], sh[j]));
  }
  stamp(6);   // state GELU done (with the late output gate: before the output gate is looked at)
  if constexpr (S::kEarlyGate) {
#pragma unroll
    for (int j = 0; j < E; ++j) st[j] *= og[j];
  } else {
    __builtin_amdgcn_sched_barrier(0);   // the GELU above runs while the output gate is still on its way
    in[7].template unpack<T>(a);
    (kSharedZ ? in[0] : in[8]).template unpack<T>(b);
#pragma unroll
    for (int j = 0; j < E; ++j) st[j] *= sigmoid_f(fmaf(p.alpha, b[j], a[j]));
  }
  if (active) {
    if constexpr (S::kStreamOutputs) C::template pack<T>(st).store_stream(os_row);
    else C::template pack<T>(st).store(os_row);
  }
  stamp(7);   // state stored
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

#ifdef ARCTIC_TUNING
// Measurement build only: ARCTIC_LSTM_VARIANT = variant bits (see sum_lstm_vec_kernel) + 8 for two rows per workgroup
// + 16 for two chunks per lane (256 lanes per 4096-wide row), or + 32 for 8-byte chunks (1024 lanes per 4096-wide
// row); 66 = variant 2 with barriers between the groups of requests.  ARCTIC_LSTM_STAGED selects a schedule of
// sum_lstm_staged_kernel instead.  Read at every call.
static int lstm_tuning_variant() {
  const char *e = getenv("ARCTIC_LSTM_VARIANT");
  return e ? atoi(e) : 0;
}
template <typename T, bool kFastGelu, bool kSharedZ, int kVariant>
static void launch_lstm_tuned(const LstmParams &p, int64_t rows, int shape, int threads, hipStream_t s) {
  const dim3 one((unsigned)rows), two((unsigned)((rows + 1) / 2));
  switch (shape) {
    case 0: hipLaunchKernelGGL((sum_lstm_vec_kernel<T, 8, 1, kFastGelu, 512, kSharedZ, true, 1, kVariant>), one, dim3(threads), 0, s, p); break;
    case 1: hipLaunchKernelGGL((sum_lstm_vec_kernel<T, 8, 1, kFastGelu, 512, kSharedZ, true, 2, kVariant>), two, dim3(threads), 0, s, p); break;
    case 2: hipLaunchKernelGGL((sum_lstm_vec_kernel<T, 8, 2, kFastGelu, 512, kSharedZ, true, 1, kVariant>), one, dim3(threads / 2), 0, s, p); break;
    case 3: hipLaunchKernelGGL((sum_lstm_vec_kernel<T, 8, 2, kFastGelu, 512, kSharedZ, true, 2, kVariant>), two, dim3(threads / 2), 0, s, p); break;
    default: hipLaunchKernelGGL((sum_lstm_vec_kernel<T, 4, 1, kFastGelu, 1024, kSharedZ, true, 1, kVariant>), one, dim3(threads * 2), 0, s, p); break;
  }
}
#endif

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
    const bool all = p.w_cell && p.b_cell && p.w_state && p.b_state && threads * cpt == chunks;
    (void)all;   // (the measurement build's variants below ask for it)
#ifdef ARCTIC_TUNING
    if (cpt == 1 && all && threads % 128 == 0 && p.prev_cell) {
      if (const char *st = getenv("ARCTIC_LSTM_STAGED")) {
        // the staged kernel's schedules that the benchmark times against each other; + 100 for the time stamps
        LstmParams q = p;
        const char *e = getenv("ARCTIC_LSTM_TRACE");   // address of rows x 8 waves x 8 words
        q.trace = e ? (unsigned long long *)strtoull(e, nullptr, 0) : nullptr;
        const int code = atoi(st);
#define ARCTIC_STAGED(CODE, ...)                                                                                     \
  if (code == CODE)                                                                                                  \
    hipLaunchKernelGGL((sum_lstm_staged_kernel<T, kFastGelu, kSharedZ, false, LstmSchedule<__VA_ARGS__>>), grid,     \
                       dim3(threads), 0, s, q);                                                                      \
  if (code == 100 + CODE)                                                                                            \
    hipLaunchKernelGGL((sum_lstm_staged_kernel<T, kFastGelu, kSharedZ, false, LstmSchedule<__VA_ARGS__>, true>),     \
                       grid, dim3(threads), 0, s, q);
        ARCTIC_STAGED(0, 9, 9, 9, 9, true, 0, false, false)    // everything requested at once, as sum_lstm_vec_kernel does
        ARCTIC_STAGED(1, 2, 3, 7, 7, false, 0, false, false)   // staged requests
        ARCTIC_STAGED(2, 2, 3, 7, 7, false, 2, false, false)   // + the vectors requested where they are needed
        ARCTIC_STAGED(3, 2, 3, 7, 7, false, 2, true, false)    // + streaming stores
        ARCTIC_STAGED(4, 2, 3, 7, 7, false, 2, true, true)     // + streaming load of the previous cell
        ARCTIC_STAGED(5, 2, 3, 7, 7, true, 2, true, true)      // the same with the early output gate
        ARCTIC_STAGED(6, 2, 4, 7, 9, false, 2, true, true)     // other request points
        ARCTIC_STAGED(7, 3, 4, 7, 7, false, 2, true, true)
        ARCTIC_STAGED(8, 2, 3, 5, 7, false, 2, true, true)
        ARCTIC_STAGED(9, 5, 7, 9, 9, false, 2, true, true)
        ARCTIC_STAGED(10, 9, 9, 9, 9, true, 0, true, true)     // everything at once with the streaming accesses
        ARCTIC_STAGED(11, 2, 3, 7, 7, false, 2, true, true, 1)    // 4 + a barrier behind the first requests
        ARCTIC_STAGED(12, 2, 3, 7, 7, false, 2, true, true, 4)    // ... behind the requests after the candidate's GELU: as shipped
        ARCTIC_STAGED(13, 2, 3, 7, 7, false, 2, true, true, 8)    // ... behind the output gate's requests
        ARCTIC_STAGED(14, 2, 3, 7, 7, false, 2, true, true, 13)   // ... behind all three
        ARCTIC_STAGED(15, 2, 3, 7, 7, false, 2, true, true, 12)   // ... behind the last two
#undef ARCTIC_STAGED
        return;
      }
      const int v = lstm_tuning_variant();
      const int shape = (v >> 3) & 7;   // 4: 8-byte units, twice the lanes (rows of up to 4096)
      if (v == 66) {   // variant 2 + a barrier between the groups of requests
        launch_lstm_tuned<T, kFastGelu, kSharedZ, kLstmEarlyOutputGate | kLstmLoadGroupBarriers>(p, rows, 0, threads, s);
        return;
      }
      switch (v & 7) {
        case 0: launch_lstm_tuned<T, kFastGelu, kSharedZ, 0>(p, rows, shape, threads, s); break;
        case 1: launch_lstm_tuned<T, kFastGelu, kSharedZ, 1>(p, rows, shape, threads, s); break;
        case 2: launch_lstm_tuned<T, kFastGelu, kSharedZ, 2>(p, rows, shape, threads, s); break;
        case 3: launch_lstm_tuned<T, kFastGelu, kSharedZ, 3>(p, rows, shape, threads, s); break;
        case 4: launch_lstm_tuned<T, kFastGelu, kSharedZ, 4>(p, rows, shape, threads, s); break;
        default: launch_lstm_tuned<T, kFastGelu, kSharedZ, 5>(p, rows, shape, threads, s); break;
      }
      return;
    }
#endif
    constexpr int kShipped = kLstmEarlyOutputGate;   // measured best of the variants that change no result bit
    // All four vectors given and a row of up to 8192 elements: the staged kernel, one chunk per lane (512 rows of
    // 5120 / 6144 / 8192 elements: 12.0 / 13.9 / 17.9 us against 17.6 / 19.9 / 22.5 us with two chunks per lane in the
    // kernel below), with idle lanes in the last wave when the row is no multiple of 512 elements.
    const bool staged = chunks <= 1024 && p.w_cell && p.b_cell && p.w_state && p.b_state;
    const int lanes = (chunks + 63) & ~63;
#define ARCTIC_LSTM_STAGED_LAUNCH(ZERO, MAX_LANES, RAGGED)                                                           \
  hipLaunchKernelGGL((sum_lstm_staged_kernel<T, kFastGelu, kSharedZ, ZERO, LstmShippedSchedule, false, MAX_LANES, RAGGED>), \
                     grid, dim3(lanes), 0, s, p)
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
      hipLaunchKernelGGL((sum_lstm_vec_kernel<T, 8, 1, kFastGelu, 512, kSharedZ, false, 1, kShipped>), grid, dim3(threads), 0, s, p);
    else
      hipLaunchKernelGGL((sum_lstm_vec_kernel<T, 8, 2, kFastGelu, 1024, kSharedZ, false, 1, 0>), grid, dim3(threads), 0, s, p);
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
#ifdef ARCTIC_TUNING
  p.trace = nullptr;
#endif
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
