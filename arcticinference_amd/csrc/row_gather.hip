// Row gather / scatter over several tensors in one launch, gfx950.
//
// Stands for the index_select calls of LlamaSwiftKVModel.swiftkv_select
// (arctic_inference/vllm/swiftkv/llama_swiftkv.py:663-679: hidden_states,
// residual, positions, k_states and v_states gathered by logits_indices into the
// decode runner's buffers) and for the write-back
// `orig_hidden_states[logits_indices] = hidden_states[:batch_size]` (:733-742).
//
// Every tensor is a matrix of rows; row r of the result is row indices[r] of the
// source (gather) or row r of the source goes to row indices[r] of the
// destination (scatter).  The rows of all tensors of a call are laid end to end
// into one run of units (16 bytes where sizes, pitches and addresses allow it,
// else the largest power of two that does), and a workgroup moves 1024
// consecutive units of one row: loads first, then stores.  An index outside
// [0, num_indexed_rows) moves nothing.
#include <hip/hip_runtime.h>

#include <algorithm>

#include "common.hpp"

namespace arctic {

constexpr int kMaxGatherTensors = 8;
// Lanes per workgroup.  Measured on swiftkv_select's five tensors (208 KiB per row): 512 rows 39.0 / 38.7 / 38.5 /
// 39.6 / 42.1 us with 64 / 128 / 256 / 512 / 1024 lanes, 2048 rows 140.2 / 140.5 / 140.5 / 139.3 / 153.2 us.
constexpr int kGatherLanes = 256;
constexpr int kGatherUnroll = 4;

struct GatherTable {
  const char *src[kMaxGatherTensors];
  char *dst[kMaxGatherTensors];
  int64_t src_stride[kMaxGatherTensors];   // bytes between rows
  int64_t dst_stride[kMaxGatherTensors];
  // Position of the tensor's first unit in the run and one past its last.  A tensor starts at a multiple of 8 units,
  // so that workgroup boundaries inside wide rows fall on 128-byte lines of the row (a one-unit tensor such as the
  // positions would otherwise shift every boundary behind it into the middle of a line).
  int64_t first_unit[kMaxGatherTensors];
  int64_t end_unit[kMaxGatherTensors];
  int unit_shift[kMaxGatherTensors];           // log2 of the unit size in bytes
  int count;
};

template <int kBytes>
struct Unit;
template <>
struct Unit<16> { typedef unsigned type __attribute__((ext_vector_type(4))); };
template <>
struct Unit<8> { typedef unsigned type __attribute__((ext_vector_type(2))); };
template <>
struct Unit<4> { typedef unsigned type; };
template <>
struct Unit<2> { typedef unsigned short type; };
template <>
struct Unit<1> { typedef unsigned char type; };

template <int kBytes>
__device__ __forceinline__ void move_units(const char *src, char *dst, int64_t first, int64_t end) {
  typedef typename Unit<kBytes>::type U;
  typedef const U ARCTIC_GLOBAL *SrcPtr;
  typedef U ARCTIC_GLOBAL *DstPtr;
  U v[kGatherUnroll];
#pragma unroll
  for (int k = 0; k < kGatherUnroll; ++k) {
    const int64_t u = first + (int64_t)k * kGatherLanes;
    if (u < end) v[k] = __builtin_nontemporal_load((SrcPtr)(src + u * kBytes));
  }
#pragma unroll
  for (int k = 0; k < kGatherUnroll; ++k) {
    const int64_t u = first + (int64_t)k * kGatherLanes;
    if (u < end) __builtin_nontemporal_store(v[k], (DstPtr)(dst + u * kBytes));
  }
}

template <typename Index>
__global__ __launch_bounds__(kGatherLanes) void row_gather_kernel(GatherTable tab, const Index *__restrict__ indices,
                                                                    int64_t num_indices, int64_t num_indexed_rows,
                                                                    int scatter) {
  // the 1024 units of this workgroup may straddle tensors; each tensor's share is moved in turn
  const int64_t begin = (int64_t)blockIdx.x * (kGatherLanes * kGatherUnroll);
  const int64_t end = begin + kGatherLanes * kGatherUnroll;
  // the grid's second dimension holds at most 65535 rows; beyond that a workgroup takes several
  for (int64_t row = blockIdx.y; row < num_indices; row += gridDim.y) {
    const int64_t idx = (int64_t)indices[row];
    if (idx < 0 || idx >= num_indexed_rows) continue;   // uniform over the workgroup
    const int64_t src_row = scatter ? row : idx;
    const int64_t dst_row = scatter ? idx : row;
    for (int t = 0; t < tab.count; ++t) {
      const int64_t lo = std::max(begin, tab.first_unit[t]);
      const int64_t hi = std::min(end, tab.end_unit[t]);
      if (lo >= hi) continue;
      const char *src = tab.src[t] + src_row * tab.src_stride[t];
      char *dst = tab.dst[t] + dst_row * tab.dst_stride[t];
      const int64_t first = lo - tab.first_unit[t] + threadIdx.x;
      const int64_t last = hi - tab.first_unit[t];
      switch (tab.unit_shift[t]) {
        case 4: move_units<16>(src, dst, first, last); break;
        case 3: move_units<8>(src, dst, first, last); break;
        case 2: move_units<4>(src, dst, first, last); break;
        case 1: move_units<2>(src, dst, first, last); break;
        default: move_units<1>(src, dst, first, last); break;
      }
    }
  }
}

static inline int alignment_shift(uint64_t v) {
  // log2 of the largest power of two (at most 16) that divides v; 16 for v == 0
  return v == 0 ? 4 : std::min(4, __builtin_ctzll(v));
}

}  // namespace arctic

using namespace arctic;

extern "C" int arctic_gather_rows(int num_tensors, const void *const *src, void *const *dst,
                                  const int64_t *row_bytes, const int64_t *src_row_stride_bytes,
                                  const int64_t *dst_row_stride_bytes, const void *indices, int index_bytes,
                                  int64_t num_indices, int64_t num_indexed_rows, int scatter, void *stream) {
  const char *fn = scatter ? "scatter_rows" : "gather_rows";
  if (num_tensors < 0 || num_tensors > kMaxGatherTensors)
    return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: between 0 and %d tensors per call, got %d", fn, kMaxGatherTensors,
                num_tensors);
  if (index_bytes != 4 && index_bytes != 8)
    return fail(ARCTIC_ERR_UNSUPPORTED, "%s: indices must be int32 or int64", fn);
  if (num_indices < 0) return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: negative number of indices", fn);
  if (num_indexed_rows < 0) return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: negative row count", fn);
  if (num_tensors == 0 || num_indices == 0) return ARCTIC_OK;
  if (!src || !dst || !row_bytes || !src_row_stride_bytes || !dst_row_stride_bytes || !indices)
    return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: null argument", fn);

  GatherTable tab = {};
  int64_t units = 0;
  for (int t = 0; t < num_tensors; ++t) {
    if (row_bytes[t] < 0 || src_row_stride_bytes[t] < 0 || dst_row_stride_bytes[t] < 0)
      return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: tensor %d: negative size or pitch", fn, t);
    if (row_bytes[t] == 0) continue;
    const int64_t most_rows = std::max(num_indices, num_indexed_rows);
    if (row_bytes[t] > ((int64_t)1 << 40) || !pitch_ok(src_row_stride_bytes[t], most_rows, 1) ||
        !pitch_ok(dst_row_stride_bytes[t], most_rows, 1))
      return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: tensor %d: row size or pitch out of range", fn, t);
    if (!src[t] || !dst[t]) return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: tensor %d: null pointer", fn, t);
    const int c = tab.count++;
    tab.src[c] = (const char *)src[t];
    tab.dst[c] = (char *)dst[t];
    tab.src_stride[c] = src_row_stride_bytes[t];
    tab.dst_stride[c] = dst_row_stride_bytes[t];
    int shift = alignment_shift((uint64_t)row_bytes[t]);
    shift = std::min(shift, alignment_shift((uint64_t)(uintptr_t)src[t]));
    shift = std::min(shift, alignment_shift((uint64_t)(uintptr_t)dst[t]));
    shift = std::min(shift, alignment_shift((uint64_t)src_row_stride_bytes[t]));
    shift = std::min(shift, alignment_shift((uint64_t)dst_row_stride_bytes[t]));
    tab.unit_shift[c] = shift;
    units = (units + 7) & ~(int64_t)7;
    tab.first_unit[c] = units;
    units += row_bytes[t] >> shift;
    tab.end_unit[c] = units;
  }
  if (units == 0) return ARCTIC_OK;
  const int64_t per_group = (int64_t)kGatherLanes * kGatherUnroll;
  const int64_t groups = (units + per_group - 1) / per_group;
  if (groups > 0x7fffffffLL) return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: rows too long", fn);

  const dim3 grid((unsigned)groups, (unsigned)std::min<int64_t>(num_indices, 65535));
  hipStream_t s = (hipStream_t)stream;
  if (index_bytes == 8)
    hipLaunchKernelGGL((row_gather_kernel<int64_t>), grid, dim3(kGatherLanes), 0, s, tab,
                       (const int64_t *)indices, num_indices, num_indexed_rows, scatter);
  else
    hipLaunchKernelGGL((row_gather_kernel<int32_t>), grid, dim3(kGatherLanes), 0, s, tab,
                       (const int32_t *)indices, num_indices, num_indexed_rows, scatter);
  return check_launch(fn);
}
