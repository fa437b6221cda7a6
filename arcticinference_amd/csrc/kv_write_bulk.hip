// SwiftKV bulk KV-cache write for gfx950.
//
// Replaces reshape_and_cache_flash_bulk (host launcher and kernel,
// csrc/custom_ops/reshape_and_cache_flash_bulk.cu:12-144 in the reference).
//
// Work decomposition
// ------------------
// One workgroup owns one token and a run of consecutive layers.  The token's
// slot is looked up once; a prologue turns (slot, layer, K|V) into a table of
// row descriptors in LDS - destination address of the token's row in that
// layer's cache and the fp64 reciprocal of that layer's scale - with one lane per
// row, so the per-layer pointer and scale reads are issued together instead of
// one dependent pair per layer.  The main loop then streams the token's source
// rows: every lane moves 16 bytes per access (8 bf16/fp16 or 4 fp32 elements),
// consecutive lanes cover consecutive addresses along head_size, and the cache
// row is written with 16-byte (copy) or 8-byte (fp8, 8 codes) stores.  Source
// and destination are each touched exactly once, so both use streaming
// (non-temporal) accesses.
//
// The four per-layer pointer tables travel in the kernel-argument segment, so a
// call uploads nothing and can be recorded into a HIP graph.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>
#include <mutex>
#include <type_traits>

#include "common.hpp"
#include "fp8_convert.hpp"

namespace arctic {

constexpr int kScalarThreads = 256;
constexpr int kLayersPerLaunch = 64;  // 4 tables x 64 pointers = 2 KiB of kernel arguments

struct LayerTables {
  const void *key_cache[kLayersPerLaunch];
  const void *value_cache[kLayersPerLaunch];
  const float *k_scale[kLayersPerLaunch];
  const float *v_scale[kLayersPerLaunch];
};

struct BulkParams {
  const char *keys;    // already offset to the first layer of this launch
  const char *values;
  const int64_t *slot_mapping;
  int64_t key_stride_bytes;
  int64_t value_stride_bytes;
  int64_t block_stride;  // elements
  int64_t num_slots;     // slots at or beyond this move nothing
  int num_layers;        // layers in this launch
  int layers_per_group;  // consecutive layers owned by one workgroup
  int groups_per_token;
  int n;                 // num_heads * head_size
  int block_size;
  int chunks_per_row;    // 16-byte source chunks per (token, layer) row
  int chunk_shift;       // log2(chunks_per_row) or -1
  // select variants: token t's source rows are also copied, unconverted, to the rows j of keys_out / values_out with
  // indices[j] == t.  With a row map (kSelectByRowMap) that is row row_map[t] of keys_out /
  // values_out (already offset to the first layer of this launch); a negative row or one >= num_out_rows = none
  const int64_t *row_map;
  char *keys_out;
  char *values_out;
  int64_t out_key_stride_bytes;
  int64_t out_value_stride_bytes;
  int64_t num_out_rows;
  // The first index_blocks workgroups serve the index list itself, one output row per lane: output row j whose
  // index the row map does not credit to j (a repeated index, or a source row at or beyond num_tokens) is copied
  // straight from source row indices[j], so the output equals index_select for every index in [0, num_src_rows).
  // A handful of workgroups, first in the grid so that their two dependent lookups overlap the token workgroups'
  // streaming instead of trailing it.  indices == nullptr: no such workgroups are launched.
  const void *indices;
  int64_t num_tokens;
  int64_t num_src_rows;
  unsigned index_blocks;
  int index_is_64;
  int select_mode;   // kSelectNone / kSelectByRowMap / kSelectByScan (the vector kernels take it as a template argument)
};

// How a launch finds the output rows of a token: not at all, through the inverse of the index list that the caller
// built beforehand, or by scanning the index list itself (short lists: one or a few loads per lane, no launch and
// no workspace for the inverse).
enum : int { kSelectNone = 0, kSelectByRowMap = 1, kSelectByScan = 2 };

struct __align__(16) RowDesc {
  char *dst;    // first byte of this token's row in the layer's K or V cache
  double inv;   // RN64(1 / scale); unused by the copy path
};

// ---- element-type plumbing ---------------------------------------------------
struct SrcBF16 {
  static constexpr int kElemsPerChunk = 8;
  static constexpr int kBytes = 2;
  __device__ static __forceinline__ void to_float(const uint4 &v, float (&f)[8]) { unpack8<BF16>(v, f); }
};
struct SrcF16 {
  static constexpr int kElemsPerChunk = 8;
  static constexpr int kBytes = 2;
  __device__ static __forceinline__ void to_float(const uint4 &v, float (&f)[8]) { unpack8<F16>(v, f); }
};
struct SrcF32 {
  static constexpr int kElemsPerChunk = 4;
  static constexpr int kBytes = 4;
};

struct Copy {};  // ARCTIC_KV_AUTO

template <typename F8>
__device__ __forceinline__ void quantize_store(char *dst, const float (&f)[8], double inv) {
  uint2 out;
  out.x = encode4<F8>(div_by_scale(f[0], inv), div_by_scale(f[1], inv),
                      div_by_scale(f[2], inv), div_by_scale(f[3], inv));
  out.y = encode4<F8>(div_by_scale(f[4], inv), div_by_scale(f[5], inv),
                      div_by_scale(f[6], inv), div_by_scale(f[7], inv));
  store8_stream(dst, out);
}

// One 16-byte source chunk -> cache.  `col` is the chunk's index inside its row.
template <typename Src, typename Dst>
__device__ __forceinline__ void emit_chunk(const uint4 &v, const RowDesc &d, int col) {
  if constexpr (std::is_same<Dst, Copy>::value) {
    store16_stream(d.dst + (int64_t)col * 16, v);
  } else if constexpr (Src::kElemsPerChunk == 8) {
    float f[8];
    Src::to_float(v, f);
    quantize_store<Dst>(d.dst + (int64_t)col * 8, f, d.inv);
  } else {
    const uint32_t w = encode4<Dst>(div_by_scale(__uint_as_float(v.x), d.inv),
                                    div_by_scale(__uint_as_float(v.y), d.inv),
                                    div_by_scale(__uint_as_float(v.z), d.inv),
                                    div_by_scale(__uint_as_float(v.w), d.inv));
    store4_stream(d.dst + (int64_t)col * 4, w);
  }
}

// Which source row output row j wants, or -1 when the token workgroups already copy it or the index lies outside
// the source.  By row map: the token's workgroup serves the one output row the map credits the token with.  By scan:
// it serves every output row that names the token, so only source rows beyond the slot mapping are left.
template <int kSelect>
__device__ __forceinline__ int64_t leftover_source_row(const BulkParams &p, int64_t j) {
  const int64_t t = p.index_is_64 ? ((const int64_t *)p.indices)[j] : (int64_t)((const int32_t *)p.indices)[j];
  if (t < 0 || t >= p.num_src_rows) return -1;
  if (t < p.num_tokens && (kSelect == kSelectByScan || p.row_map[t] == j)) return -1;
  return t;
}

// Index workgroup `b`: its lanes look at output rows b * kThreads ... (one each); almost always none of them is
// left over (SwiftKV selects each token once) and the workgroup is done after two dependent lookups.  The rows that
// are left over are listed in LDS and copied by the whole workgroup, all layers of the launch, one row after the other.
template <int kThreads, int kSelect>
__device__ __forceinline__ int list_leftover_rows(const BulkParams &p, unsigned b, int64_t (&todo_j)[kThreads],
                                                  int64_t (&todo_t)[kThreads], int &count) {
  if (threadIdx.x == 0) count = 0;
  __syncthreads();
  const int64_t j = (int64_t)b * kThreads + threadIdx.x;
  if (j < p.num_out_rows) {
    const int64_t t = leftover_source_row<kSelect>(p, j);
    if (t >= 0) {
      const int k = atomicAdd(&count, 1);
      todo_j[k] = j;
      todo_t[k] = t;
    }
  }
  __syncthreads();
  return count;
}

template <typename Src, bool kPow2, int kBulkThreads, int kSelect>
__device__ __forceinline__ void select_leftover_rows(const BulkParams &p, unsigned b) {
  __shared__ int64_t todo_j[kBulkThreads], todo_t[kBulkThreads];
  __shared__ int count;
  const int n = list_leftover_rows<kBulkThreads, kSelect>(p, b, todo_j, todo_t, count);
  const int cpr = p.chunks_per_row;
  const int total = 2 * p.num_layers * cpr;
  for (int e = 0; e < n; ++e) {
    const int64_t j = todo_j[e], t = todo_t[e];
    const char *ksrc = p.keys + t * p.key_stride_bytes, *vsrc = p.values + t * p.value_stride_bytes;
    char *kout = p.keys_out + j * p.out_key_stride_bytes, *vout = p.values_out + j * p.out_value_stride_bytes;
    for (int c = threadIdx.x; c < total; c += kBulkThreads) {
      int r, col;
      if constexpr (kPow2) {
        r = c >> p.chunk_shift;
        col = c & (cpr - 1);
      } else {
        r = c / cpr;
        col = c - r * cpr;
      }
      const int64_t off = ((int64_t)(r >> 1) * cpr + col) * 16;
      store16_stream(((r & 1) ? vout : kout) + off, load16_stream(((r & 1) ? vsrc : ksrc) + off));
    }
  }
}

// kBulkThreads x kUnroll 16-byte chunks form one batch of a workgroup.  Three shapes are built, all with batches
// of 1024 chunks: 1024 x 1 (launches of more than 8192 tokens: a workgroup moves up to five batches), 512 x 2 (the
// same launches when rows are selected as well) and 256 x 4 (everything smaller: one or two batches per workgroup).
template <typename Src, typename Dst, bool kPow2, int kBulkThreads, int kUnroll, int kSelect>
__device__ __forceinline__ void bulk_item(const BulkParams &p, const LayerTables &tab, unsigned block) {
  constexpr bool kCopy = std::is_same<Dst, Copy>::value;
  constexpr int kDstElemBytes = kCopy ? Src::kBytes : 1;

  __shared__ RowDesc rows[2 * kLayersPerLaunch];

  if constexpr (kSelect) {
    if (block < p.index_blocks) {  // uniform over the workgroup, before any barrier
      select_leftover_rows<Src, kPow2, kBulkThreads, kSelect>(p, block);
      return;
    }
    block -= p.index_blocks;
  }
  const int64_t token = block / (unsigned)p.groups_per_token;
  const int group = block - (unsigned)token * (unsigned)p.groups_per_token;
  const int layer0 = group * p.layers_per_group;
  const int nlayers = min(p.layers_per_group, p.num_layers - layer0);

  const char *ksrc = p.keys + token * p.key_stride_bytes + (int64_t)layer0 * p.n * Src::kBytes;
  const char *vsrc = p.values + token * p.value_stride_bytes + (int64_t)layer0 * p.n * Src::kBytes;
  const int cpr = p.chunks_per_row;
  const int total = 2 * nlayers * cpr;  // chunks this workgroup moves

  auto locate = [&](int c, int &r, int &col) {
    if constexpr (kPow2) {
      r = c >> p.chunk_shift;
      col = c & (cpr - 1);
    } else {
      r = c / cpr;
      col = c - r * cpr;
    }
  };
  // kUnroll independent 16-byte loads per lane; lanes past the end load nothing
  auto load_batch = [&](int c, uint4 (&v)[kUnroll]) {
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int cu = c + u * kBulkThreads;
      if (cu < total) {
        int r, col;
        locate(cu, r, col);
        const char *base = (r & 1) ? vsrc : ksrc;
        v[u] = load16_stream(base + ((int64_t)(r >> 1) * cpr + col) * 16);
      }
    }
  };

  // The slot lookup and the first batch of source loads are issued together:
  // source addresses do not depend on the slot, so HBM is already streaming
  // while the row descriptors below are being built.  (A padding token throws
  // its first batch away.)
  const int64_t slot = p.slot_mapping[token];
  int64_t out_row = -1;
  if constexpr (kSelect == kSelectByRowMap) out_row = p.row_map[token];
  // by scan: every lane requests its share of the index list ahead of the source rows, like the slot, and compares
  // it with the token once the first batch is on its way; the output rows that name this token end up in `hits`
  constexpr int kIndicesPerLane = ARCTIC_SELECT_SCAN_MAX_INDICES / kBulkThreads;
  __shared__ int hits[kSelect == kSelectByScan ? ARCTIC_SELECT_SCAN_MAX_INDICES : 1];
  __shared__ int num_hits;
  int64_t mine[kIndicesPerLane];
  if constexpr (kSelect == kSelectByScan) {
#pragma unroll
    for (int k = 0; k < kIndicesPerLane; ++k) {
      const int j = threadIdx.x + k * kBulkThreads;
      mine[k] = -1;   // no token
      if (j < (int)p.num_out_rows)
        mine[k] = p.index_is_64 ? ((const int64_t *)p.indices)[j] : (int64_t)((const int32_t *)p.indices)[j];
    }
    if (threadIdx.x == 0) num_hits = 0;
  }
  int c = threadIdx.x;
  uint4 cur[kUnroll];
  load_batch(c, cur);
  int nhits = 0;
  if constexpr (kSelect == kSelectByScan) {
    __syncthreads();
#pragma unroll
    for (int k = 0; k < kIndicesPerLane; ++k)
      if (mine[k] == token) hits[atomicAdd(&num_hits, 1)] = threadIdx.x + k * kBulkThreads;
    __syncthreads();
    nhits = num_hits;
  }
  // padding (or a slot outside the cache) writes no cache row; both tests are uniform over the workgroup
  const bool to_cache = slot >= 0 && slot < p.num_slots;
  const bool to_out = kSelect == kSelectByScan ? nhits > 0
                                               : (kSelect == kSelectByRowMap && out_row >= 0 && out_row < p.num_out_rows);
  if (!to_cache && !to_out) return;  // uniform, and behind the scan's barriers

  if (to_cache) {
    int64_t blk, off;
    if (slot < 0x7fffffffLL) {
      const uint32_t s32 = (uint32_t)slot, bs = (uint32_t)p.block_size;
      blk = s32 / bs;
      off = s32 - (uint32_t)blk * bs;
    } else {
      blk = slot / p.block_size;
      off = slot - blk * p.block_size;
    }
    const int64_t row_elem = blk * p.block_stride + off * (int64_t)p.n;

    // one lane per (layer, K|V) row of this token
    for (int r = threadIdx.x; r < 2 * nlayers; r += kBulkThreads) {
      const int layer = layer0 + (r >> 1);
      const bool is_v = r & 1;
      const void *base = is_v ? tab.value_cache[layer] : tab.key_cache[layer];
      RowDesc d;
      d.dst = (char *)base + row_elem * kDstElemBytes;
      d.inv = 0.0;
      if constexpr (!kCopy) {
        const float *sp = is_v ? tab.v_scale[layer] : tab.k_scale[layer];
        d.inv = 1.0 / (double)(*sp);
      }
      rows[r] = d;
    }
    __syncthreads();
  }
  char *kout = nullptr, *vout = nullptr;
  if constexpr (kSelect == kSelectByRowMap) {
    if (to_out) {
      kout = p.keys_out + out_row * p.out_key_stride_bytes + (int64_t)layer0 * p.n * Src::kBytes;
      vout = p.values_out + out_row * p.out_value_stride_bytes + (int64_t)layer0 * p.n * Src::kBytes;
    }
  }
  if constexpr (kSelect == kSelectByScan) {   // the columns of this workgroup's layers; the row is added per hit
    kout = p.keys_out + (int64_t)layer0 * p.n * Src::kBytes;
    vout = p.values_out + (int64_t)layer0 * p.n * Src::kBytes;
  }

  // Main loop: a batch is converted and stored, then the next one is requested.  (Requesting the next batch first,
  // so that it is in flight during the conversion, measures the same within half a per cent at every size and
  // placement: the other workgroups of the CU cover a workgroup's wait either way.)
  while (c < total) {
    const int cn = c + kUnroll * kBulkThreads;
    uint4 nxt[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int cu = c + u * kBulkThreads;
      if (cu < total) {
        int r, col;
        locate(cu, r, col);
        if (!kSelect || to_cache) emit_chunk<Src, Dst>(cur[u], rows[r], col);
        if constexpr (kSelect == kSelectByRowMap) {
          if (to_out) store16_stream(((r & 1) ? vout : kout) + ((int64_t)(r >> 1) * cpr + col) * 16, cur[u]);
        }
        if constexpr (kSelect == kSelectByScan) {
          const int64_t off = ((int64_t)(r >> 1) * cpr + col) * 16;
          for (int h = 0; h < nhits; ++h) {   // one hit unless the list names the token more than once
            const int64_t j = hits[h];
            store16_stream((r & 1) ? vout + j * p.out_value_stride_bytes + off : kout + j * p.out_key_stride_bytes + off,
                           cur[u]);
          }
        }
      }
    }
    load_batch(cn, nxt);
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) cur[u] = nxt[u];
    c = cn;
  }
}

template <typename Src, typename Dst, bool kPow2, int kBulkThreads, int kUnroll, int kSelect>
__global__ __launch_bounds__(kBulkThreads) void kv_write_bulk_kernel(
    const BulkParams p, const LayerTables tab) {
  bulk_item<Src, Dst, kPow2, kBulkThreads, kUnroll, kSelect>(p, tab, blockIdx.x);
}



// Fallback for shapes or addresses that do not allow 16-byte accesses: one
// element per lane per step, any alignment.  Same arithmetic, no vector access.
template <typename SrcElem, typename Dst>
__global__ __launch_bounds__(kScalarThreads) void kv_write_bulk_scalar_kernel(
    const BulkParams p, const LayerTables tab, const int src_dtype) {
  constexpr bool kCopy = std::is_same<Dst, Copy>::value;
  if (blockIdx.x < p.index_blocks) {  // the index list's own workgroups (select variant only)
    __shared__ int64_t todo_j[kScalarThreads], todo_t[kScalarThreads];
    __shared__ int count;
    const int n = p.select_mode == kSelectByScan
                      ? list_leftover_rows<kScalarThreads, kSelectByScan>(p, blockIdx.x, todo_j, todo_t, count)
                      : list_leftover_rows<kScalarThreads, kSelectByRowMap>(p, blockIdx.x, todo_j, todo_t, count);
    for (int e = 0; e < n; ++e) {
      const int64_t j = todo_j[e], t = todo_t[e];
      const SrcElem *ks = reinterpret_cast<const SrcElem *>(p.keys + t * p.key_stride_bytes);
      const SrcElem *vs = reinterpret_cast<const SrcElem *>(p.values + t * p.value_stride_bytes);
      SrcElem *ko = reinterpret_cast<SrcElem *>(p.keys_out + j * p.out_key_stride_bytes);
      SrcElem *vo = reinterpret_cast<SrcElem *>(p.values_out + j * p.out_value_stride_bytes);
      for (int64_t i = threadIdx.x; i < (int64_t)p.num_layers * p.n; i += kScalarThreads) {
        ko[i] = ks[i];
        vo[i] = vs[i];
      }
    }
    return;
  }
  const unsigned block = blockIdx.x - p.index_blocks;
  const int64_t token = block / (unsigned)p.groups_per_token;
  const int group = block - (unsigned)token * (unsigned)p.groups_per_token;
  const int layer0 = group * p.layers_per_group;
  const int nlayers = min(p.layers_per_group, p.num_layers - layer0);
  const int64_t slot = p.slot_mapping[token];
  // output rows of this token: the one the row map names, or all that a scan of the index list finds
  __shared__ int hits[ARCTIC_SELECT_SCAN_MAX_INDICES];
  __shared__ int num_hits;
  int nhits = 0;
  if (p.select_mode == kSelectByScan) {   // uniform
    if (threadIdx.x == 0) num_hits = 0;
    __syncthreads();
    for (int j = threadIdx.x; j < (int)p.num_out_rows; j += kScalarThreads) {
      const int64_t t = p.index_is_64 ? ((const int64_t *)p.indices)[j] : (int64_t)((const int32_t *)p.indices)[j];
      if (t == token) hits[atomicAdd(&num_hits, 1)] = j;
    }
    __syncthreads();
    nhits = num_hits;
  } else if (p.select_mode == kSelectByRowMap) {
    const int64_t out_row = p.row_map[token];
    if (out_row >= 0 && out_row < p.num_out_rows) {
      if (threadIdx.x == 0) hits[0] = (int)out_row;
      nhits = 1;
    }
    __syncthreads();
  }
  const bool to_cache = slot >= 0 && slot < p.num_slots;
  if (!to_cache && nhits == 0) return;
  const SrcElem *ks = reinterpret_cast<const SrcElem *>(p.keys + token * p.key_stride_bytes);
  const SrcElem *vs = reinterpret_cast<const SrcElem *>(p.values + token * p.value_stride_bytes);
  for (int h = 0; h < nhits; ++h) {
    const int64_t out_row = hits[h];
    SrcElem *ko = reinterpret_cast<SrcElem *>(p.keys_out + out_row * p.out_key_stride_bytes);
    SrcElem *vo = reinterpret_cast<SrcElem *>(p.values_out + out_row * p.out_value_stride_bytes);
    for (int64_t i = (int64_t)layer0 * p.n + threadIdx.x; i < (int64_t)(layer0 + nlayers) * p.n; i += kScalarThreads) {
      ko[i] = ks[i];
      vo[i] = vs[i];
    }
  }
  if (!to_cache) return;
  const int64_t blk = slot / p.block_size;
  const int64_t off = slot - blk * p.block_size;
  const int64_t row_elem = blk * p.block_stride + off * (int64_t)p.n;

  for (int l = layer0; l < layer0 + nlayers; ++l) {
    double kinv = 0.0, vinv = 0.0;
    if constexpr (!kCopy) {
      kinv = 1.0 / (double)(*tab.k_scale[l]);
      vinv = 1.0 / (double)(*tab.v_scale[l]);
    }
    for (int i = threadIdx.x; i < p.n; i += kScalarThreads) {
      const SrcElem k = ks[(int64_t)l * p.n + i];
      const SrcElem v = vs[(int64_t)l * p.n + i];
      if constexpr (kCopy) {
        ((SrcElem *)tab.key_cache[l])[row_elem + i] = k;
        ((SrcElem *)tab.value_cache[l])[row_elem + i] = v;
      } else {
        float kf, vf;
        if constexpr (sizeof(SrcElem) == 4) {
          kf = __uint_as_float((uint32_t)k);
          vf = __uint_as_float((uint32_t)v);
        } else if (src_dtype == ARCTIC_DTYPE_BF16) {
          kf = BF16::lo((uint32_t)k);
          vf = BF16::lo((uint32_t)v);
        } else {
          kf = F16::lo((uint32_t)k);
          vf = F16::lo((uint32_t)v);
        }
        const uint32_t wk = encode4<Dst>(div_by_scale(kf, kinv), 0.f, 0.f, 0.f);
        const uint32_t wv = encode4<Dst>(div_by_scale(vf, vinv), 0.f, 0.f, 0.f);
        ((uint8_t *)tab.key_cache[l])[row_elem + i] = (uint8_t)(wk & 0xffu);
        ((uint8_t *)tab.value_cache[l])[row_elem + i] = (uint8_t)(wv & 0xffu);
      }
    }
  }
}

template <typename Src, typename Dst, int kSelect>
static void launch_vec_shape(const BulkParams &p, const LayerTables &tab, int64_t grid, bool wide, hipStream_t s) {
  const dim3 g((unsigned)grid);
  if (p.chunk_shift >= 0) {
    if (wide && kSelect == kSelectNone)   // the same batch of 1024 chunks by 1024 lanes: 0.5-2 % faster than 512 x 2
      hipLaunchKernelGGL((kv_write_bulk_kernel<Src, Dst, true, 1024, 1, kSelectNone>), g, dim3(1024), 0, s, p, tab);
    else if (wide)
      hipLaunchKernelGGL((kv_write_bulk_kernel<Src, Dst, true, 512, 2, kSelect>), g, dim3(512), 0, s, p, tab);
    else
      hipLaunchKernelGGL((kv_write_bulk_kernel<Src, Dst, true, 256, 4, kSelect>), g, dim3(256), 0, s, p, tab);
  } else {
    hipLaunchKernelGGL((kv_write_bulk_kernel<Src, Dst, false, 256, 4, kSelect>), g, dim3(256), 0, s, p, tab);
  }
}
template <typename Src, typename Dst>
static void launch_vec(const BulkParams &p, const LayerTables &tab, int64_t grid, bool wide, hipStream_t s) {
  switch (p.select_mode) {
    case kSelectByScan: launch_vec_shape<Src, Dst, kSelectByScan>(p, tab, grid, wide, s); break;
    case kSelectByRowMap: launch_vec_shape<Src, Dst, kSelectByRowMap>(p, tab, grid, wide, s); break;
    default: launch_vec_shape<Src, Dst, kSelectNone>(p, tab, grid, wide, s); break;
  }
}
template <typename SrcElem, typename Dst>
static void launch_scalar(const BulkParams &p, const LayerTables &tab, int64_t grid, int src_dtype,
                          hipStream_t s) {
  hipLaunchKernelGGL((kv_write_bulk_scalar_kernel<SrcElem, Dst>), dim3((unsigned)grid),
                     dim3(kScalarThreads), 0, s, p, tab, src_dtype);
}

template <typename Dst>
static void dispatch_src(bool vec, bool wide, int src_dtype, const BulkParams &p, const LayerTables &tab,
                         int64_t grid, hipStream_t s) {
  if (vec) {
    switch (src_dtype) {
      case ARCTIC_DTYPE_BF16: launch_vec<SrcBF16, Dst>(p, tab, grid, wide, s); break;
      case ARCTIC_DTYPE_F16: launch_vec<SrcF16, Dst>(p, tab, grid, wide, s); break;
      default: launch_vec<SrcF32, Dst>(p, tab, grid, wide, s); break;
    }
  } else {
    if (src_dtype == ARCTIC_DTYPE_F32)
      launch_scalar<uint32_t, Dst>(p, tab, grid, src_dtype, s);
    else
      launch_scalar<uint16_t, Dst>(p, tab, grid, src_dtype, s);
  }
}

// row_map[t] = j where indices[j] == t, -1 where no j is: one workgroup, so that the fill is complete
// (barrier) before the rows are entered.  Tens of thousands of tokens at most: a few microseconds.
template <typename Index>
__global__ __launch_bounds__(1024) void build_row_map_kernel(int64_t *__restrict__ row_map, int64_t num_tokens,
                                                             const Index *__restrict__ indices, int64_t num_indices) {
  for (int64_t t = threadIdx.x; t < num_tokens; t += blockDim.x) row_map[t] = -1;
  __syncthreads();
  for (int64_t j = threadIdx.x; j < num_indices; j += blockDim.x) {
    const int64_t t = (int64_t)indices[j];
    if (t >= 0 && t < num_tokens) row_map[t] = j;
  }
}

static inline bool aligned(const void *p, uintptr_t a) { return ((uintptr_t)p % a) == 0; }

}  // namespace arctic

using namespace arctic;

// The rows a launch may also copy out (the select variant); row_map == nullptr: none.
struct SelectArgs {
  int mode;                  // kSelectNone / kSelectByRowMap / kSelectByScan
  const int64_t *row_map;    // kSelectByRowMap only
  void *keys_out;
  void *values_out;
  int64_t out_key_stride;    // elements
  int64_t out_value_stride;
  int64_t num_out_rows;
  const void *indices;       // the index list (num_out_rows entries); with a row map it may be nullptr
  int index_bytes;
  int64_t num_src_rows;      // rows of keys / values an index may name
};

static int bulk_entry(const char *fn, const void *keys, const void *values, int64_t key_stride, int64_t value_stride,
                      const void *const *key_cache_ptrs, const void *const *value_cache_ptrs,
                      const float *const *k_scale_ptrs, const float *const *v_scale_ptrs,
                      const int64_t *slot_mapping, int64_t num_tokens, int num_layers, int num_heads, int head_size,
                      int block_size, int64_t block_stride, int64_t num_blocks, int src_dtype, int kv_cache_dtype,
                      const SelectArgs &sel_in, void *stream, bool check_only = false) {
  if (num_layers == 0 || num_tokens == 0) return ARCTIC_OK;  // reference :87-89
  if (num_layers < 0 || num_layers > ARCTIC_MAX_LAYERS)
    return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: num_layers=%d outside [0, %d]", fn, num_layers,
                ARCTIC_MAX_LAYERS);
  if (num_tokens < 0 || num_tokens > 0x7fffffffLL)
    return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: num_tokens=%lld outside [0, 2^31)", fn, (long long)num_tokens);
  if (num_heads <= 0 || head_size <= 0 || block_size <= 0)
    return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: num_heads, head_size and block_size must be positive", fn);
  if (num_blocks < 0) return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: negative num_blocks", fn);
  if (src_dtype != ARCTIC_DTYPE_F32 && src_dtype != ARCTIC_DTYPE_F16 && src_dtype != ARCTIC_DTYPE_BF16)
    return fail(ARCTIC_ERR_UNSUPPORTED, "%s: Unsupported input type of kv cache: %d", fn, src_dtype);
  if (kv_cache_dtype != ARCTIC_KV_AUTO && kv_cache_dtype != ARCTIC_KV_FP8_E4M3 &&
      kv_cache_dtype != ARCTIC_KV_FP8_E5M2)
    return fail(ARCTIC_ERR_UNSUPPORTED, "%s: Unsupported data type of kv cache: %d", fn, kv_cache_dtype);
  if (!keys || !values || !slot_mapping || !key_cache_ptrs || !value_cache_ptrs)
    return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: null tensor pointer", fn);
  if (block_size > (1 << 20) || num_blocks > ((int64_t)1 << 40))
    return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: block_size beyond 2^20 or num_blocks beyond 2^40", fn);
  {
    const int src_bytes = src_dtype == ARCTIC_DTYPE_F32 ? 4 : 2;
    const int64_t src_rows = sel_in.mode != kSelectNone && sel_in.indices ? std::max(num_tokens, sel_in.num_src_rows) : num_tokens;
    if (!pitch_ok(key_stride, src_rows, src_bytes) || !pitch_ok(value_stride, src_rows, src_bytes) ||
        !pitch_ok(block_stride, num_blocks, kv_cache_dtype == ARCTIC_KV_AUTO ? src_bytes : 1))
      return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: row or block pitch out of range", fn);
    if (sel_in.mode != kSelectNone && (!pitch_ok(sel_in.out_key_stride, sel_in.num_out_rows, src_bytes) ||
                                       !pitch_ok(sel_in.out_value_stride, sel_in.num_out_rows, src_bytes)))
      return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: negative number of output rows or row pitch out of range", fn);
  }
  SelectArgs sel = sel_in;
  if (sel.mode != kSelectNone) {
    if (sel.num_out_rows < 0 || sel.num_out_rows > 0x7fffffffLL || sel.out_key_stride < 0 || sel.out_value_stride < 0)
      return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: negative number of output rows or row pitch, or 2^31 output rows or more", fn);
    if (sel.num_out_rows == 0) sel.mode = kSelectNone;   // no row to copy to: the plain write
  }
  if (sel.mode != kSelectNone) {
    if (!sel.keys_out || !sel.values_out) return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: null keys_out or values_out", fn);
    if (sel.mode == kSelectByRowMap && !sel.row_map) return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: null row map", fn);
    if (sel.mode == kSelectByScan && (!sel.indices || sel.num_out_rows > ARCTIC_SELECT_SCAN_MAX_INDICES))
      return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: the index list is missing or longer than %d entries and there is no row map",
                  fn, ARCTIC_SELECT_SCAN_MAX_INDICES);
    if (sel.indices) {
      if (sel.index_bytes != 4 && sel.index_bytes != 8)
        return fail(ARCTIC_ERR_UNSUPPORTED, "%s: indices must be int32 or int64", fn);
      if (sel.num_src_rows < num_tokens)
        return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: keys / values have fewer rows (%lld) than slot_mapping (%lld)", fn,
                    (long long)sel.num_src_rows, (long long)num_tokens);
    }
  }
  const bool quant = kv_cache_dtype != ARCTIC_KV_AUTO;
  if (quant && (!k_scale_ptrs || !v_scale_ptrs))
    return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: fp8 cache needs k_scales and v_scales", fn);
  const int64_t n64 = (int64_t)num_heads * head_size;
  if (n64 > (1 << 24)) return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: num_heads*head_size too large", fn);
  const int n = (int)n64;
  for (int l = 0; l < num_layers; ++l) {
    if (!key_cache_ptrs[l] || !value_cache_ptrs[l])
      return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: null cache pointer for layer %d", fn, l);
    if (quant && (!k_scale_ptrs[l] || !v_scale_ptrs[l]))
      return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: null scale pointer for layer %d", fn, l);
  }

  const int es = src_dtype == ARCTIC_DTYPE_F32 ? 4 : 2;
  const int des = quant ? 1 : es;
  const int epc = 16 / es;  // elements per 16-byte chunk
  // 16-byte loads need aligned rows; stores are 16 B (copy), 8 B (fp8 from 16-bit) or 4 B (fp8 from fp32)
  const int store_bytes = quant ? epc : 16;
  // (a single source row needs no pitch; with an index list the index workgroups read rows up to num_src_rows)
  const bool one_source_row =
      (sel.mode != kSelectNone && sel.indices ? std::max(num_tokens, sel.num_src_rows) : num_tokens) == 1;
  bool vec = (n % epc == 0) && aligned(keys, 16) && aligned(values, 16) &&
             ((key_stride * es) % 16 == 0 || one_source_row) &&
             ((value_stride * es) % 16 == 0 || one_source_row) && ((block_stride * des) % store_bytes == 0);
  for (int l = 0; vec && l < num_layers; ++l)
    vec = aligned(key_cache_ptrs[l], store_bytes) && aligned(value_cache_ptrs[l], store_bytes);
  if (vec && sel.mode != kSelectNone)
    vec = aligned(sel.keys_out, 16) && aligned(sel.values_out, 16) &&
          ((sel.out_key_stride * es) % 16 == 0 || sel.num_out_rows <= 1) &&
          ((sel.out_value_stride * es) % 16 == 0 || sel.num_out_rows <= 1);

  hipStream_t s = (hipStream_t)stream;
  // More than kLayersPerLaunch layers take several launches.  Pass 0 plans every launch and checks its grid, so that
  // a call that is refused has launched nothing; pass 1 launches (a single launch is checked just before it is made).
  for (int pass = (check_only || num_layers > kLayersPerLaunch) ? 0 : 1; pass < (check_only ? 1 : 2); ++pass) {
    for (int first = 0; first < num_layers; first += kLayersPerLaunch) {
      const int count = std::min(kLayersPerLaunch, num_layers - first);
      LayerTables tab;
      for (int l = 0; l < kLayersPerLaunch; ++l) {
        const bool in = l < count;
        tab.key_cache[l] = in ? key_cache_ptrs[first + l] : nullptr;
        tab.value_cache[l] = in ? value_cache_ptrs[first + l] : nullptr;
        tab.k_scale[l] = (in && quant) ? k_scale_ptrs[first + l] : nullptr;
        tab.v_scale[l] = (in && quant) ? v_scale_ptrs[first + l] : nullptr;
      }
      BulkParams p;
      p.keys = (const char *)keys + (int64_t)first * n * es;
      p.values = (const char *)values + (int64_t)first * n * es;
      p.slot_mapping = slot_mapping;
      const bool select = sel.mode != kSelectNone;
      p.select_mode = sel.mode;
      p.row_map = sel.mode == kSelectByRowMap ? sel.row_map : nullptr;
      p.keys_out = select ? (char *)sel.keys_out + (int64_t)first * n * es : nullptr;
      p.values_out = select ? (char *)sel.values_out + (int64_t)first * n * es : nullptr;
      p.out_key_stride_bytes = sel.out_key_stride * es;
      p.out_value_stride_bytes = sel.out_value_stride * es;
      p.num_out_rows = select ? sel.num_out_rows : 0;
      p.indices = select ? sel.indices : nullptr;
      p.index_is_64 = sel.index_bytes == 8;
      p.num_tokens = num_tokens;
      p.num_src_rows = sel.num_src_rows;
      p.key_stride_bytes = key_stride * es;
      p.value_stride_bytes = value_stride * es;
      p.block_stride = block_stride;
      p.num_slots = num_blocks > 0 ? num_blocks * (int64_t)block_size : INT64_MAX;
      p.num_layers = count;
      p.n = n;
      p.block_size = block_size;
      p.chunks_per_row = vec ? n / epc : 0;
      p.chunk_shift = -1;
      if (vec && (p.chunks_per_row & (p.chunks_per_row - 1)) == 0) p.chunk_shift = __builtin_ctz(p.chunks_per_row);

      // A token's layers are split over `groups` workgroups.  Measured best on gfx950 (sweeps over the group count and
      // both shapes at 64 to 16384 tokens, 16 and 40 layers):
      //  - above 8192 tokens, the wide shape (batches of 1024 chunks by 1024 lanes, by 512 lanes when rows are
      //    selected as well) with up to five batches per workgroup (20 layers of 8 x 128 bf16) and at least about
      //    1024 workgroups; a workgroup that would get less than two batches takes the 256-lane shape instead;
      //  - below that, the 256-lane shape with about two batches of 1024 chunks per workgroup (8 such layers), more
      //    and smaller workgroups when fewer than about 2048 would exist otherwise, but never less than one batch each.
      int groups = 1;
      bool wide = false;
      if (vec) {
        const int64_t chunks_per_layer = 2LL * p.chunks_per_row;
        const int min_layers = (int)std::max<int64_t>(1, (1024 + chunks_per_layer - 1) / chunks_per_layer);
        if (num_tokens > 8192) {
          int64_t g = std::max<int64_t>((1024 + num_tokens - 1) / num_tokens, (chunks_per_layer * count + 5119) / 5120);
          g = std::max<int64_t>(1, std::min<int64_t>(g, count));
          const int64_t layers_per_group = (count + g - 1) / g;
          if (layers_per_group * chunks_per_layer >= 2048) {
            wide = true;
            groups = (int)g;
          } else {
            const int64_t want = (2048 + num_tokens - 1) / num_tokens;
            groups = (int)std::max<int64_t>(1, std::min<int64_t>(want, count / min_layers));
          }
        } else {
          const int64_t two_batches = std::max<int64_t>(1, (2048 + chunks_per_layer - 1) / chunks_per_layer);   // layers
          const int64_t want =
              std::max<int64_t>((count + two_batches - 1) / two_batches, (2048 + num_tokens - 1) / num_tokens);
          groups = (int)std::max<int64_t>(1, std::min<int64_t>(want, count / min_layers));
        }
      } else {
        groups = (int)std::max<int64_t>(1, std::min<int64_t>(count, (2048 + num_tokens - 1) / num_tokens));
      }
      p.layers_per_group = (count + groups - 1) / groups;
      p.groups_per_token = (count + p.layers_per_group - 1) / p.layers_per_group;
      // lanes of the shape launched below when rows are selected (the only case with index workgroups)
      const int lanes = !vec ? kScalarThreads : (wide && p.chunk_shift >= 0) ? 512 : 256;
      const int64_t index_blocks = p.indices ? (p.num_out_rows + lanes - 1) / lanes : 0;
      const int64_t grid = num_tokens * p.groups_per_token + index_blocks;
      p.index_blocks = (unsigned)index_blocks;
      if (grid > 0x7fffffffLL)
        return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: too many tokens (%lld)", fn, (long long)num_tokens);
      if (pass == 0) continue;

      switch (kv_cache_dtype) {
        case ARCTIC_KV_AUTO: dispatch_src<Copy>(vec, wide, src_dtype, p, tab, grid, s); break;
        case ARCTIC_KV_FP8_E4M3: dispatch_src<E4M3>(vec, wide, src_dtype, p, tab, grid, s); break;
        default: dispatch_src<E5M2>(vec, wide, src_dtype, p, tab, grid, s); break;
      }
      const int rc = check_launch(fn);
      if (rc) return rc;
    }
  }
  return ARCTIC_OK;
}

extern "C" int arctic_reshape_and_cache_flash_bulk(
    const void *keys, const void *values, int64_t key_stride, int64_t value_stride,
    const void *const *key_cache_ptrs, const void *const *value_cache_ptrs,
    const float *const *k_scale_ptrs, const float *const *v_scale_ptrs,
    const int64_t *slot_mapping, int64_t num_tokens, int num_layers, int num_heads,
    int head_size, int block_size, int64_t block_stride, int64_t num_blocks, int src_dtype,
    int kv_cache_dtype, void *stream) {
  const SelectArgs none = {kSelectNone, nullptr, nullptr, nullptr, 0, 0, 0, nullptr, 0, 0};
  return bulk_entry("reshape_and_cache_flash_bulk", keys, values, key_stride, value_stride, key_cache_ptrs,
                    value_cache_ptrs, k_scale_ptrs, v_scale_ptrs, slot_mapping, num_tokens, num_layers, num_heads,
                    head_size, block_size, block_stride, num_blocks, src_dtype, kv_cache_dtype, none, stream);
}

extern "C" int arctic_reshape_and_cache_flash_bulk_select(
    const void *keys, const void *values, int64_t key_stride, int64_t value_stride,
    const void *const *key_cache_ptrs, const void *const *value_cache_ptrs,
    const float *const *k_scale_ptrs, const float *const *v_scale_ptrs,
    const int64_t *slot_mapping, int64_t num_tokens, int num_layers, int num_heads,
    int head_size, int block_size, int64_t block_stride, int64_t num_blocks, int src_dtype,
    int kv_cache_dtype, const int64_t *row_map, const void *indices, int index_bytes, int64_t num_indices,
    int64_t num_src_rows, void *keys_out, void *values_out, int64_t out_key_stride, int64_t out_value_stride,
    void *stream) {
  const char *fn = "reshape_and_cache_flash_bulk_select";
  // a row map is used when one is given; without one the token workgroups scan the index list themselves
  const SelectArgs sel = {row_map ? kSelectByRowMap : kSelectByScan, row_map, keys_out, values_out, out_key_stride,
                          out_value_stride, num_indices, indices, index_bytes, num_src_rows};
  return bulk_entry(fn, keys, values, key_stride, value_stride, key_cache_ptrs, value_cache_ptrs, k_scale_ptrs,
                    v_scale_ptrs, slot_mapping, num_tokens, num_layers, num_heads, head_size, block_size, block_stride,
                    num_blocks, src_dtype, kv_cache_dtype, sel, stream);
}

static int build_row_map(const char *fn, int64_t *row_map, int64_t num_tokens, const void *indices, int index_bytes,
                         int64_t num_indices, void *stream) {
  if (index_bytes != 4 && index_bytes != 8) return fail(ARCTIC_ERR_UNSUPPORTED, "%s: indices must be int32 or int64", fn);
  if (num_tokens < 0 || num_indices < 0) return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: negative size", fn);
  if (num_tokens == 0) return ARCTIC_OK;
  if (!row_map || (num_indices > 0 && !indices)) return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: null pointer", fn);
  hipStream_t s = (hipStream_t)stream;
  if (index_bytes == 8)
    hipLaunchKernelGGL(build_row_map_kernel<int64_t>, dim3(1), dim3(1024), 0, s, row_map, num_tokens,
                       (const int64_t *)indices, num_indices);
  else
    hipLaunchKernelGGL(build_row_map_kernel<int32_t>, dim3(1), dim3(1024), 0, s, row_map, num_tokens,
                       (const int32_t *)indices, num_indices);
  return check_launch(fn);
}

extern "C" int arctic_build_row_map(int64_t *row_map, int64_t num_tokens, const void *indices, int index_bytes,
                                    int64_t num_indices, void *stream) {
  return build_row_map("build_row_map", row_map, num_tokens, indices, index_bytes, num_indices, stream);
}

// ---- the select variant that allocates nothing ---------------------------------------------------------------
// The row map of arctic_reshape_and_cache_flash_bulk_select_static lives in this array instead of a workspace
// the caller brings in: 8 bytes per token, 2 MiB, held by every GPU the library has run on until the process
// ends.  In host code `scratch` is only a handle for the symbol; the array's address on a device comes from
// hipGetSymbolAddress with that device current, is looked up once per device and is what the kernels receive.
static __device__ __align__(256) int64_t scratch[ARCTIC_SELECT_STATIC_MAX_TOKENS];

namespace {
constexpr int kMaxDevices = 64;
// Per device: its copy of `scratch` (nullptr until first asked for), and what orders the calls that use it.  The
// array is shared by every call on the GPU, so a call on another stream than the last one first makes its stream
// wait for `last_use`, an event recorded behind the last call's kernels: calls on different streams then use the
// array one after the other instead of racing on it.  Under stream capture nothing of this is recorded.
struct DeviceScratch {
  int64_t *ptr = nullptr;
  hipEvent_t last_use = nullptr;
  hipStream_t last_stream = nullptr;
  bool used = false;
};
std::mutex g_scratch_mutex;
DeviceScratch g_scratch[kMaxDevices];
}  // namespace

static int scratch_on_current_device(const char *fn, DeviceScratch **out) {
  int dev = -1;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return fail(ARCTIC_ERR_LAUNCH, "%s: hipGetDevice failed: %s", fn, hipGetErrorString(err));
  if (dev < 0 || dev >= kMaxDevices) return fail(ARCTIC_ERR_UNSUPPORTED, "%s: device index %d not supported", fn, dev);
  DeviceScratch &d = g_scratch[dev];
  if (!d.ptr) {
    void *ptr = nullptr;
    err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (err != hipSuccess || !ptr)
      return fail(ARCTIC_ERR_LAUNCH, "%s: hipGetSymbolAddress failed on device %d: %s", fn, dev, hipGetErrorString(err));
    err = hipEventCreateWithFlags(&d.last_use, hipEventDisableTiming);
    if (err != hipSuccess)
      return fail(ARCTIC_ERR_LAUNCH, "%s: hipEventCreateWithFlags failed on device %d: %s", fn, dev, hipGetErrorString(err));
    d.ptr = (int64_t *)ptr;
  }
  *out = &d;
  return ARCTIC_OK;
}

extern "C" int arctic_reshape_and_cache_flash_bulk_select_static(
    const void *keys, const void *values, int64_t key_stride, int64_t value_stride,
    const void *const *key_cache_ptrs, const void *const *value_cache_ptrs,
    const float *const *k_scale_ptrs, const float *const *v_scale_ptrs,
    const int64_t *slot_mapping, int64_t num_tokens, int num_layers, int num_heads,
    int head_size, int block_size, int64_t block_stride, int64_t num_blocks, int src_dtype,
    int kv_cache_dtype, const void *indices, int index_bytes, int64_t num_indices, int64_t num_src_rows,
    void *keys_out, void *values_out, int64_t out_key_stride, int64_t out_value_stride, void *stream) {
  const char *fn = "reshape_and_cache_flash_bulk_select_static";
  if (num_tokens > ARCTIC_SELECT_STATIC_MAX_TOKENS)
    return fail(ARCTIC_ERR_INVALID_ARGUMENT,
                "%s: num_tokens=%lld exceeds the %d tokens the static row map holds; use "
                "arctic_reshape_and_cache_flash_bulk_select with a row map of the caller's",
                fn, (long long)num_tokens, ARCTIC_SELECT_STATIC_MAX_TOKENS);
  if (num_indices < 0) return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: negative number of indices", fn);
  if (num_indices > 0 && !indices) return fail(ARCTIC_ERR_INVALID_ARGUMENT, "%s: null indices", fn);
  // short index lists are scanned by the token workgroups and need no row map; longer ones get theirs in `scratch`
  if (num_layers == 0 || num_tokens <= 0 || num_indices <= ARCTIC_SELECT_SCAN_MAX_INDICES) {
    const SelectArgs sel = {kSelectByScan, nullptr, keys_out, values_out, out_key_stride, out_value_stride, num_indices,
                            indices, index_bytes, num_src_rows};
    return bulk_entry(fn, keys, values, key_stride, value_stride, key_cache_ptrs, value_cache_ptrs, k_scale_ptrs,
                      v_scale_ptrs, slot_mapping, num_tokens, num_layers, num_heads, head_size, block_size,
                      block_stride, num_blocks, src_dtype, kv_cache_dtype, sel, stream);
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);   // one call at a time plans its use of the array
  DeviceScratch *d = nullptr;
  int rc = scratch_on_current_device(fn, &d);
  if (rc) return rc;
  const SelectArgs sel = {kSelectByRowMap, d->ptr, keys_out, values_out, out_key_stride, out_value_stride, num_indices,
                          indices, index_bytes, num_src_rows};
  // every argument is checked before the first kernel is enqueued: a call that is refused has launched nothing
  rc = bulk_entry(fn, keys, values, key_stride, value_stride, key_cache_ptrs, value_cache_ptrs, k_scale_ptrs,
                  v_scale_ptrs, slot_mapping, num_tokens, num_layers, num_heads, head_size, block_size, block_stride,
                  num_blocks, src_dtype, kv_cache_dtype, sel, stream, /*check_only=*/true);
  if (rc) return rc;
  hipStream_t s = (hipStream_t)stream;
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(s, &capture) != hipSuccess) capture = hipStreamCaptureStatusNone;
  const bool eager = capture == hipStreamCaptureStatusNone;
  if (eager && d->used && d->last_stream != s) {
    const hipError_t err = hipStreamWaitEvent(s, d->last_use, 0);
    if (err != hipSuccess) return fail(ARCTIC_ERR_LAUNCH, "%s: hipStreamWaitEvent failed: %s", fn, hipGetErrorString(err));
  }
  // every entry below num_tokens is rewritten, so nothing of an earlier call is seen
  rc = build_row_map(fn, d->ptr, num_tokens, indices, index_bytes, num_indices, stream);
  if (rc) return rc;
  rc = bulk_entry(fn, keys, values, key_stride, value_stride, key_cache_ptrs, value_cache_ptrs, k_scale_ptrs,
                  v_scale_ptrs, slot_mapping, num_tokens, num_layers, num_heads, head_size, block_size, block_stride,
                  num_blocks, src_dtype, kv_cache_dtype, sel, stream);
  if (eager) {
    const hipError_t err = hipEventRecord(d->last_use, s);
    if (err != hipSuccess && rc == ARCTIC_OK)
      rc = fail(ARCTIC_ERR_LAUNCH, "%s: hipEventRecord failed: %s", fn, hipGetErrorString(err));
    d->last_stream = s;
    d->used = true;
  }
  return rc;
}
