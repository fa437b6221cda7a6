// Row-wise argmax with clamping, gfx950.
//
// Stands for the token selection at the end of every speculator step,
//   last_tokens = torch.argmax(logits, dim=-1); last_tokens.clamp_(0, vocab_size - 1)
// (arctic_inference/vllm/spec_dec/arctic_speculator.py:846-848, 862), with torch's rules for the winner:
// the largest value, the lowest index among equal values, and a NaN beats every number (the first NaN wins).
//
// One workgroup per row; a lane walks 16-byte chunks of the row with streaming loads and keeps its own
// (value, index) winner; winners are merged inside the wave with lane exchanges and across the waves
// through LDS.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>

#include "common.hpp"

namespace arctic {

// A candidate as one 64-bit key whose unsigned order is torch's order of winners (GreaterOrNan with the index as tie
// break, aten/src/ATen/native/SharedReduceOps.h): the value's bits mapped monotonically to an unsigned number in the
// upper half (-0 counts as +0, every NaN as the largest number of all), the complement of the index in the lower half
// (among equal values the lowest index is the largest key).  0 = nothing seen: no element maps to upper half 0.
// Merging two candidates is then one 64-bit unsigned maximum instead of a cascade of floating-point cases.
__device__ __forceinline__ uint64_t winner_key(float value, int index) {
  if (index < 0) return 0;
  uint32_t b = __float_as_uint(value);
  if (b == 0x80000000u) b = 0;   // -0 -> +0 (on the bits: no arithmetic that a denormal mode could touch)
  uint32_t o = b ^ ((b & 0x80000000u) ? 0xffffffffu : 0x80000000u);
  if (value != value) o = 0xffffffffu;
  return ((uint64_t)o << 32) | (uint32_t)~(uint32_t)index;
}
__device__ __forceinline__ int winner_index(uint64_t key) { return key ? (int)~(uint32_t)key : -1; }

// The wave's winner in every lane.  Inside each row of 16 lanes the candidates meet through DPP lane exchanges
// (vector-ALU moves, no LDS round trip): partners at distance 1 and 2 inside a quad, then the mirrored half and the
// mirrored row, after which all 16 lanes of a row agree; the four row winners are read with v_readlane.
template <int kCtrl>
__device__ __forceinline__ uint64_t meet(uint64_t k) {
  const uint32_t lo = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)(uint32_t)k, kCtrl, 0xf, 0xf, true);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)(uint32_t)(k >> 32), kCtrl, 0xf, 0xf, true);
  const uint64_t other = ((uint64_t)hi << 32) | lo;
  return other > k ? other : k;
}

__device__ __forceinline__ uint64_t wave_winner(uint64_t k) {
  k = meet<0xB1>(k);   // quad_perm [1,0,3,2]
  k = meet<0x4E>(k);   // quad_perm [2,3,0,1]
  k = meet<0x141>(k);  // row_half_mirror
  k = meet<0x140>(k);  // row_mirror
  uint64_t r = 0;
#pragma unroll
  for (int lane = 0; lane < 64; lane += 16) {
    const uint64_t row = ((uint64_t)(uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(k >> 32), lane) << 32) |
                         (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)k, lane);
    r = row > r ? row : r;
  }
  return r;
}

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));

struct F32Elem {
  static constexpr int kPerChunk = 4;
  // NaN exactly when the chunk holds a NaN or infinities of both signs
  __device__ static __forceinline__ float probe(const uint4 &v) {
    return (__uint_as_float(v.x) + __uint_as_float(v.y)) + (__uint_as_float(v.z) + __uint_as_float(v.w));
  }
  __device__ static __forceinline__ void unpack(const uint4 &v, float (&f)[8]) {
    f[0] = __uint_as_float(v.x);
    f[1] = __uint_as_float(v.y);
    f[2] = __uint_as_float(v.z);
    f[3] = __uint_as_float(v.w);
  }
  __device__ static __forceinline__ float one(const void *p, int64_t i) { return ((const float *)p)[i]; }
};
template <typename T>
struct HalfElem {
  static constexpr int kPerChunk = 8;
  // the sum of the chunk's eight values, two per instruction straight from the packed words (v_dot2c_f32_bf16 /
  // v_dot2c_f32_f16 with a vector of ones): NaN exactly when the chunk holds a NaN or infinities of both signs
  __device__ static __forceinline__ float probe(const uint4 &v) {
    float acc = 0.f;
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      if constexpr (T::kCode == ARCTIC_DTYPE_BF16) {
        const bf16x2_t ones = {(__bf16)1.0f, (__bf16)1.0f};
        acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, w[k]), ones, acc, false);
      } else {
        const f16x2_t ones = {(_Float16)1.0f, (_Float16)1.0f};
        acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, w[k]), ones, acc, false);
      }
    }
    return acc;
  }
  __device__ static __forceinline__ void unpack(const uint4 &v, float (&f)[8]) { unpack8<T>(v, f); }
  __device__ static __forceinline__ float one(const void *p, int64_t i) {
    return T::lo((uint32_t)((const uint16_t *)p)[i]);
  }
};

// kVec: the body of a row, from its first 16-byte boundary on, is read in 16-byte chunks; the elements in front of
// that boundary (a row pitch that is no multiple of 16 bytes puts every row somewhere else), those behind the last
// whole chunk, and everything when !kVec (a pointer that is not even element-aligned) are read one by one.
// kUnroll chunks per lane form a batch;
// kLockstep: a workgroup barrier (no memory wait) behind every batch's requests, so that every wave of the row has
// asked for batch k before any wave asks for batch k + 1 (a CU serves its oldest wave first: without the barrier the
// oldest wave runs through all its batches before the youngest gets its first one in).
// kHead: rows may start between two 16-byte boundaries (without it the host has checked that none does).
template <typename Elem, bool kVec, int kUnroll = 4, bool kLockstep = false, bool kHead = false>
__global__ __launch_bounds__(1024) void row_argmax_kernel(int64_t *__restrict__ out, const char *__restrict__ in,
                                                          int64_t row_stride_bytes, int cols, int64_t max_index) {
  __shared__ uint64_t wave_key[16];
  const char *row = in + (int64_t)blockIdx.x * row_stride_bytes;
  // Per lane: the largest number seen, the chunk it was first seen in and that chunk's words (a strict ">" keeps the
  // earlier of equal values, the lane's chunk indices only grow); which of the chunk's elements it was is worked out
  // once, after the loop.  Apart from that the first NaN: a chunk's sum is NaN only if the chunk holds a NaN (or
  // infinities of both signs), so the per-element NaN test runs almost never.
  constexpr int P = Elem::kPerChunk;
  const int head = kVec && kHead ? min(cols, (int)((0 - (uintptr_t)row) & 15) / (16 / P)) : 0;   // elements in front of the body
  const int chunks = kVec ? (cols - head) / P : 0;
  const char *body = row + (int64_t)head * (16 / P);
  float best = -__builtin_inff();
  int best_at = -1;
  int nan_at = 0x7fffffff;
  auto number = [&](float v, int i) {
    if (v > best) {
      best = v;
      best_at = i;
    }
  };
  // a lane's candidates come in the order of their indices (head, chunks, tail), so that ">" keeps the first of equals
  if ((int)threadIdx.x < head) {
    const float v = Elem::one(row, threadIdx.x);
    best_at = threadIdx.x;   // stands for the lane even when it is -inf: a row of -inf must answer 0
    best = v == v ? v : best;
    if (v != v) nan_at = threadIdx.x;
  }
  int done = 0;
  if (kVec) {
    int best_chunk = -1;
    uint4 best_words = make_uint4(0, 0, 0, 0);
    const int stride = kUnroll * blockDim.x;
    auto request = [&](int c0, uint4 (&raw)[kUnroll]) {
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        const int c = c0 + u * blockDim.x;
        if (c < chunks) raw[u] = load16_stream(body + (int64_t)c * 16);
      }
    };
    auto look_at_chunk = [&](int c, const uint4 &words) {
      float f[8];
      Elem::unpack(words, f);
      float top = best;   // fmaxf drops NaNs: they are found through the sum below
#pragma unroll
      for (int j = 0; j < P; j += 2) top = fmaxf(fmaxf(top, f[j]), f[j + 1]);
      if (top > best) {
        best_chunk = c;
        best_words = words;
      }
      best = top;
      const float sum = Elem::probe(words);
      if (sum != sum) {
#pragma unroll
        for (int j = 0; j < P; ++j)
          if (f[j] != f[j]) nan_at = min(nan_at, head + c * P + j);
      }
    };
    auto look_at = [&](int c0, const uint4 (&raw)[kUnroll]) {
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        const int c = c0 + u * blockDim.x;
        if (c < chunks) look_at_chunk(c, raw[u]);
      }
    };
    if constexpr (kLockstep) {
      const int batches = (chunks + stride - 1) / stride;   // the same for every wave, as the barrier needs it
      int c0 = threadIdx.x;
      for (int b = 0; b < batches; ++b, c0 += stride) {
        uint4 raw[kUnroll];
        request(c0, raw);
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        look_at(c0, raw);
      }
    } else {
      int c0 = threadIdx.x;
      for (; c0 < chunks; c0 += stride) {
        uint4 raw[kUnroll];
        request(c0, raw);
        look_at(c0, raw);
      }
    }
    done = head + chunks * P;
    if (best_chunk >= 0) {
      // the first element of that chunk that equals the lane's maximum
      float f[8];
      Elem::unpack(best_words, f);
      int j = P - 1;
#pragma unroll
      for (int k = P - 2; k >= 0; --k)
        if (f[k] == best) j = k;
      best_at = head + best_chunk * P + j;
    } else if (best_at < 0 && (int)threadIdx.x < chunks) {
      best_at = head + (int)threadIdx.x * P;   // nothing above -inf here: the lane's first element stands for its chunks
    }
  }
  // (a lane without chunks takes its first tail element, if it has one, the same way: a row of -inf must answer 0)
  if (best_at < 0 && done + (int)threadIdx.x < cols) best_at = done + (int)threadIdx.x;
  for (int i = done + threadIdx.x; i < cols; i += blockDim.x) {
    const float v = Elem::one(row, i);
    number(v, i);
    if (v != v) nan_at = min(nan_at, i);
  }
  uint64_t w = nan_at != 0x7fffffff ? winner_key(__builtin_nanf(""), nan_at) : winner_key(best, best_at);

  w = wave_winner(w);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (lane == 0) wave_key[wave] = w;
  __syncthreads();
  if (wave == 0) {
    const int waves = blockDim.x >> 6;
    uint64_t x = lane < waves ? wave_key[lane] : 0;
    x = wave_winner(x);
    if (lane == 0) {
      const int found = winner_index(x);
      int64_t idx = found < 0 ? 0 : found;
      out[blockIdx.x] = idx > max_index ? max_index : idx;
    }
  }
}

}  // namespace arctic

using namespace arctic;

extern "C" int arctic_argmax_clamp(int64_t *out, const void *logits, int64_t rows, int cols, int64_t row_stride,
                                   int64_t max_index, int dtype, void *stream) {
  const char *fn = "argmax_clamp";
  if (dtype != ARCTIC_DTYPE_F32 && dtype != ARCTIC_DTYPE_F16 && dtype != ARCTIC_DTYPE_BF16)
    return fail(ARCTIC_ERR_UNSUPPORTED, "%s: logits must be fp32, fp16 or bf16", fn);
  if (rows < 0 || rows > 0x7fffffffLL || cols <= 0 || max_index < 0 || row_stride < 0)
    return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: rows >= 0, cols > 0, max_index >= 0 and a non-negative pitch are required",
                fn);
  if (rows == 0) return ARCTIC_OK;
  if (!out || !logits) return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: null tensor pointer", fn);
  const int es = dtype == ARCTIC_DTYPE_F32 ? 4 : 2;
  if (cols > (1 << 30) || !pitch_ok(row_stride, rows, es))
    return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: more than 2^30 columns, or a row pitch out of range", fn);
  const int64_t stride_bytes = row_stride * es;
  const bool vec = (uintptr_t)logits % es == 0;   // rows may start anywhere between two 16-byte boundaries
  const bool aligned_rows = (uintptr_t)logits % 16 == 0 && (stride_bytes % 16 == 0 || rows == 1);
  const int per_chunk = 16 / es;
  int threads = (int)std::min<int64_t>(1024, std::max<int64_t>(64, ((cols / per_chunk / 4 + 63) / 64) * 64));
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)rows), block((unsigned)threads);
  // Launches of about one and a half to three workgroups per CU (the 256 CUs of this GPU; a decode batch of a few
  // hundred rows) keep their waves in step, a chunk at a time: the two workgroups of a CU then finish together with
  // little left to do, 5 % faster at 384 and 512 rows.  With fewer rows a wave needs four chunks in flight to cover
  // the latency, with more the generations of workgroups overlap by themselves (measured 16 to 4096 rows).
  const bool lockstep = rows > 256 && rows <= 768;
#define ARCTIC_ARGMAX_VEC(ELEM)                                                                                   \
  do {                                                                                                            \
    if (!aligned_rows && lockstep)                                                                                \
      hipLaunchKernelGGL((row_argmax_kernel<ELEM, true, 1, true, true>), grid, block, 0, s, out,    \
                         (const char *)logits, stride_bytes, cols, max_index);                                    \
    else if (!aligned_rows)                                                                                       \
      hipLaunchKernelGGL((row_argmax_kernel<ELEM, true, 4, false, true>), grid, block, 0, s, out,   \
                         (const char *)logits, stride_bytes, cols, max_index);                                    \
    else if (lockstep)                                                                                            \
      hipLaunchKernelGGL((row_argmax_kernel<ELEM, true, 1, true>), grid, block, 0, s, out,          \
                         (const char *)logits, stride_bytes, cols, max_index);                                    \
    else                                                                                                          \
      hipLaunchKernelGGL((row_argmax_kernel<ELEM, true>), grid, block, 0, s, out, (const char *)logits,           \
                         stride_bytes, cols, max_index);                                                          \
  } while (0)
#define ARCTIC_ARGMAX_LAUNCH(ELEM)                                                                          \
  do {                                                                                                      \
    if (vec)                                                                                                \
      ARCTIC_ARGMAX_VEC(ELEM);                                                                              \
    else                                                                                                    \
      hipLaunchKernelGGL((row_argmax_kernel<ELEM, false>), grid, block, 0, s, out, (const char *)logits,    \
                         stride_bytes, cols, max_index);                                                    \
  } while (0)
  if (dtype == ARCTIC_DTYPE_F32) ARCTIC_ARGMAX_LAUNCH(F32Elem);
  else if (dtype == ARCTIC_DTYPE_BF16) ARCTIC_ARGMAX_LAUNCH(HalfElem<BF16>);
  else ARCTIC_ARGMAX_LAUNCH(HalfElem<F16>);
#undef ARCTIC_ARGMAX_LAUNCH
#undef ARCTIC_ARGMAX_VEC
  return check_launch(fn);
}
