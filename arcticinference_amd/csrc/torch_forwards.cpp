// Host side of the operators in C++ (torch_host.hpp), and on top of it the four functions that ArcticInference's
// csrc/custom_ops/custom_ops.h declares.  Compiled together with the reference's own
// csrc/custom_ops/torch_bindings.cpp (unchanged: its TORCH_LIBRARY block binds exactly these four symbols,
// torch_bindings.cpp:6-51) this gives the reference's native extension for PyTorch-ROCm without any of its CUDA
// sources; compiled together with host_ext.cpp it is the Python package's own host layer.  Host code only: any
// C++17 compiler, the torch headers and -larctic_mi355x.
//
// Each function repeats the argument checks of the launcher it stands for
//   reshape_and_cache_flash_bulk   csrc/custom_ops/reshape_and_cache_flash_bulk.cu:77-144
//   reshape_and_cache_flash_fp4    csrc/custom_ops/reshape_and_cache_flash_fp4.cu:256-337
//   speculator_ln_cuda             csrc/custom_ops/speculator_ln.cu:152-252
//   sum_lstm_cuda                  csrc/custom_ops/sum_lstm.cu:293-473
// allocates outputs as it does, and hands pointers, sizes and strides to the library on torch's current stream.
// Checks that the reference leaves out (it would read or write out of bounds instead) are marked as such.
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/all.h>

#include <string>
#include <tuple>
#include <vector>

#include "../../include/arctic_mi355x.h"
#include "torch_host.hpp"

namespace arctic_host {
namespace {

using DeviceGuard = c10::hip::OptionalHIPGuardMasqueradingAsCUDA;

void *current_stream() { return (void *)c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream(); }

const void *optional_ptr(const OptTensor &t) { return t.has_value() && t->defined() ? t->data_ptr() : nullptr; }

bool given(const OptTensor &t) { return t.has_value() && t->defined(); }

bool is_half(const at::Tensor &t) { return t.scalar_type() == at::kHalf || t.scalar_type() == at::kBFloat16; }

int half_code(const at::Tensor &t) { return t.scalar_type() == at::kHalf ? ARCTIC_DTYPE_F16 : ARCTIC_DTYPE_BF16; }

// t.view(-1, cols); a tensor that is 2-D already is passed through.  A single row still goes through view(), which
// sets its row stride to `cols` as the reference's view() does.
at::Tensor rows_of(const at::Tensor &t, int64_t cols) {
  return t.dim() == 2 && t.size(0) != 1 ? t : t.view({-1, cols});
}

// Whether every row t[i] is dense (what t[0].is_contiguous() says, without making the view).
bool rows_dense(const at::Tensor &t) {
  int64_t expected = 1;
  for (int64_t d = t.dim() - 1; d >= 1; --d) {
    if (t.size(d) == 0) return true;
    if (t.size(d) != 1 && t.stride(d) != expected) return false;
    expected *= t.size(d);
  }
  return true;
}

void check_rc(int rc) { TORCH_CHECK(rc == 0, arctic_last_error()); }

// A size on its way into an `int` parameter of the C ABI: out of range is an error here, not a wrapped value there.
int to_int(int64_t v, const char *what) {
  TORCH_CHECK(v >= 0 && v <= 0x7fffffffLL, what, " = ", v, " is outside [0, 2^31)");
  return (int)v;
}

}  // namespace

CheckedLayers check_layers(const LayerLists &layers) {
  CheckedLayers c;
  const int64_t num_layers = layers.count[0];
  c.num_layers = num_layers;
  if (num_layers == 0) return c;
  TORCH_CHECK(num_layers == layers.count[1], "Expected num_layers == value_caches.size() to be true");
  TORCH_CHECK(num_layers == layers.count[2], "Expected num_layers == k_scales.size() to be true");
  TORCH_CHECK(num_layers == layers.count[3], "Expected num_layers == v_scales.size() to be true");
  const at::Tensor &first = layers(0, 0), &first_v = layers(1, 0);
  c.block_size = first.size(1);
  c.block_stride = first.stride(0);
  TORCH_CHECK(c.block_stride == first_v.stride(0), "Expected block_stride == value_caches[0].stride(0) to be true");
  // From here on: not checked by the reference (it reinterprets the pointers); a mismatch there corrupts memory,
  // here it is an error.  Every layer's K and V view must look like layer 0's: the kernel takes one block stride,
  // block size and number of blocks for all of them.
  c.num_blocks = first.size(0);
  c.cache_element_size = first.element_size();
  c.device = first.device();
  const auto dtype0 = first.scalar_type();
  c.key_caches.resize(num_layers);
  c.value_caches.resize(num_layers);
  c.k_scales.assign(num_layers, nullptr);
  c.v_scales.assign(num_layers, nullptr);
  for (int64_t l = 0; l < num_layers; ++l) {
    const at::Tensor &k = layers(0, l), &v = layers(1, l);
    TORCH_CHECK(k.scalar_type() == dtype0 && v.scalar_type() == dtype0 && k.stride(0) == c.block_stride &&
                    v.stride(0) == c.block_stride && k.size(0) == c.num_blocks && v.size(0) == c.num_blocks &&
                    k.size(1) == c.block_size && v.size(1) == c.block_size && k.device() == c.device &&
                    v.device() == c.device,
                "reshape_and_cache_flash_bulk: key and value caches of all layers must share dtype, block stride, "
                "number of blocks, block size and device");
    c.key_caches[l] = k.data_ptr();
    c.value_caches[l] = v.data_ptr();
  }
  // the scales matter to an fp8 write only, so what is wrong with them is kept until one is asked for
  for (int64_t l = 0; l < num_layers && !c.scales_problem; ++l) {
    const at::Tensor &k = layers(2, l), &v = layers(3, l);
    if (k.scalar_type() != at::kFloat || v.scalar_type() != at::kFloat)
      c.scales_problem = "reshape_and_cache_flash_bulk: k_scales / v_scales must be float32";
    else if (k.device() != c.device || v.device() != c.device)
      c.scales_problem = "reshape_and_cache_flash_bulk: all tensors must be on the same device";
    c.k_scales[l] = (const float *)k.data_ptr();
    c.v_scales[l] = (const float *)v.data_ptr();
  }
  return c;
}

void bulk_write(const at::Tensor &keys, const at::Tensor &values, const CheckedLayers &layers,
                const at::Tensor &slot_mapping, const std::string &kv_cache_dtype, int64_t num_heads,
                int64_t head_size, const SelectRows *select) {
  const int64_t num_layers = layers.num_layers;
  int64_t n_sel = 0;
  if (select) {
    const char *fn = "reshape_and_cache_flash_bulk_select";
    const at::Tensor &idx = select->logits_indices;
    TORCH_CHECK(idx.is_cuda() && idx.dim() == 1 && (idx.scalar_type() == at::kInt || idx.scalar_type() == at::kLong), fn,
                ": logits_indices must be a 1-D int32 or int64 CUDA tensor");
    n_sel = idx.numel();
    const char *names[2] = {"k_out", "v_out"};
    const at::Tensor *srcs[2] = {&keys, &values}, *outs[2] = {&select->k_out, &select->v_out};
    for (int i = 0; i < 2; ++i) {
      const at::Tensor &out = *outs[i], &src = *srcs[i];
      TORCH_CHECK(out.is_cuda() && out.device() == src.device() && out.scalar_type() == src.scalar_type(), fn, ": ",
                  names[i], " must be on the device of keys / values and of their type");
      TORCH_CHECK(out.dim() == 2 && out.size(0) >= n_sel, fn, ": ", names[i], " must be 2-D with at least ", n_sel,
                  " rows");
      TORCH_CHECK(out.stride(1) == 1, fn, ": rows of ", names[i], " must be contiguous");
    }
  }
  if (num_layers == 0) return;   // reference :87-89; no layer, so no column to write or to select either
  TORCH_CHECK(num_heads >= 1 && head_size >= 1 && num_heads <= (1 << 24) && head_size <= (1 << 24) &&
                  num_heads * head_size <= (1 << 24),
              "reshape_and_cache_flash_bulk: num_heads and head_size must be positive and num_heads * head_size at most 2^24");
  const int64_t width = num_layers * num_heads * head_size;
  const int64_t num_tokens = slot_mapping.size(0);
  at::Tensor idx;
  if (select) {
    const char *fn = "reshape_and_cache_flash_bulk_select";
    TORCH_CHECK(select->k_out.size(1) == width && select->v_out.size(1) == width && keys.size(1) >= width &&
                    values.size(1) >= width,
                fn, ": k_out and v_out must have ", width, " columns (layers x heads x head_size)");
    TORCH_CHECK(keys.size(0) == values.size(0), fn, ": keys and values differ in their number of rows");
    idx = select->logits_indices.is_contiguous() ? select->logits_indices : select->logits_indices.contiguous();
    if (num_tokens == 0) {
      // nothing is written to a cache, but the selected rows (of the first `width` columns) are still wanted
      if (n_sel) {
        const at::Tensor src[2] = {keys.narrow(1, 0, width), values.narrow(1, 0, width)};
        const at::Tensor *dst[2] = {&select->k_out, &select->v_out};
        const TensorList sources = {
            2, [](const void *c, int64_t i) -> const at::Tensor & { return ((const at::Tensor *)c)[i]; }, src};
        const TensorList outs = {
            2, [](const void *c, int64_t i) -> const at::Tensor & { return *((const at::Tensor *const *)c)[i]; }, dst};
        move_rows("gather_rows", sources, idx, outs, false);
      }
      return;
    }
  }

  // DISPATCH_BY_KV_CACHE_DTYPE, csrc/custom_ops/quant_utils.cuh:532-567
  int kv = -1;
  if (kv_cache_dtype == "auto") kv = ARCTIC_KV_AUTO;
  else if (kv_cache_dtype == "fp8" || kv_cache_dtype == "fp8_e4m3") kv = ARCTIC_KV_FP8_E4M3;
  else if (kv_cache_dtype == "fp8_e5m2") kv = ARCTIC_KV_FP8_E5M2;
  TORCH_CHECK(kv >= 0, "Unsupported data type of kv cache: ", kv_cache_dtype);
  int src = -1;
  switch (keys.scalar_type()) {
    case at::kFloat: src = ARCTIC_DTYPE_F32; break;
    case at::kHalf: src = ARCTIC_DTYPE_F16; break;
    case at::kBFloat16: src = ARCTIC_DTYPE_BF16; break;
    default: break;
  }
  TORCH_CHECK(src >= 0, "Unsupported input type of kv cache: ", keys.scalar_type());
  TORCH_CHECK(slot_mapping.scalar_type() == at::kLong, "expected scalar type Long but found ", slot_mapping.scalar_type());
  // not checked by the reference either
  TORCH_CHECK(values.scalar_type() == keys.scalar_type(), "reshape_and_cache_flash_bulk: keys and values dtype differ");
  TORCH_CHECK(keys.stride(-1) == 1 && values.stride(-1) == 1,
              "reshape_and_cache_flash_bulk: last dimension of keys/values must be contiguous");
  TORCH_CHECK(slot_mapping.dim() == 1 && (num_tokens <= 1 || slot_mapping.stride(0) == 1),
              "reshape_and_cache_flash_bulk: slot_mapping must be 1-D and contiguous");
  const int64_t want_elem = kv == ARCTIC_KV_AUTO ? keys.element_size() : 1;
  TORCH_CHECK(layers.cache_element_size == want_elem, "reshape_and_cache_flash_bulk: cache element size ",
              layers.cache_element_size, " does not match kv_cache_dtype '", kv_cache_dtype, "' (expected ", want_elem, ")");
  TORCH_CHECK(layers.device == keys.device() && values.device() == keys.device() && slot_mapping.device() == keys.device(),
              "reshape_and_cache_flash_bulk: all tensors must be on the same device");
  TORCH_CHECK(keys.is_cuda(), "reshape_and_cache_flash_bulk: the tensors must be CUDA tensors");
  // Row t is read at t * stride(0), `width` elements long.  The reference looks at stride(0) only, and its own unit
  // test (tests/unit_tests/test_custom_ops.py:79-80) passes keys of shape [L * T, H * D]; rows narrower than `width`
  // are therefore accepted as long as the last row read still ends inside the tensor's storage.
  auto covers = [&](const at::Tensor &t) {
    if (t.dim() != 2 || t.size(0) < num_tokens) return false;
    if (t.size(1) >= width || num_tokens == 0) return true;
    const int64_t have = (int64_t)(t.storage().nbytes() / t.element_size()) - t.storage_offset();
    return (num_tokens - 1) * t.stride(0) + width <= have;
  };
  TORCH_CHECK(covers(keys) && covers(values), "reshape_and_cache_flash_bulk: keys and values must be 2-D with at least ",
              num_tokens, " rows (one per slot) and ", width, " columns (layers x heads x head_size)");
  if (kv != ARCTIC_KV_AUTO) TORCH_CHECK(!layers.scales_problem, layers.scales_problem);

  const int layer_count = to_int(num_layers, "num_layers"), heads = to_int(num_heads, "num_heads");
  const int head = to_int(head_size, "head_size"), block = to_int(layers.block_size, "block_size");
  const DeviceGuard guard(keys.device());
  void *stream = current_stream();
  if (!select) {
    check_rc(arctic_reshape_and_cache_flash_bulk(
        keys.data_ptr(), values.data_ptr(), keys.stride(0), values.stride(0), layers.key_caches.data(),
        layers.value_caches.data(), layers.k_scales.data(), layers.v_scales.data(),
        (const int64_t *)slot_mapping.data_ptr(), num_tokens, layer_count, heads, head, block, layers.block_stride,
        layers.num_blocks, src, kv, stream));
    return;
  }
  // A long list: the inverse of logits_indices (which output row, if any, a token goes to) is built first; up to
  // ARCTIC_SELECT_SCAN_MAX_INDICES entries every token's workgroup scans the list itself and nothing is allocated.
  at::Tensor row_map;
  if (n_sel > ARCTIC_SELECT_SCAN_MAX_INDICES) {
    row_map = at::empty({num_tokens}, keys.options().dtype(at::kLong));
    check_rc(arctic_build_row_map((int64_t *)row_map.data_ptr(), num_tokens, idx.data_ptr(), (int)idx.element_size(), n_sel,
                                  stream));
  }
  check_rc(arctic_reshape_and_cache_flash_bulk_select(
      keys.data_ptr(), values.data_ptr(), keys.stride(0), values.stride(0), layers.key_caches.data(),
      layers.value_caches.data(), layers.k_scales.data(), layers.v_scales.data(),
      (const int64_t *)slot_mapping.data_ptr(), num_tokens, layer_count, heads, head, block, layers.block_stride,
      layers.num_blocks, src, kv, row_map.defined() ? (const int64_t *)row_map.data_ptr() : nullptr, idx.data_ptr(),
      (int)idx.element_size(), n_sel, keys.size(0), select->k_out.data_ptr(), select->v_out.data_ptr(),
      select->k_out.stride(0), select->v_out.stride(0), stream));
}

void bulk_write(const at::Tensor &keys, const at::Tensor &values, const LayerLists &layers,
                const at::Tensor &slot_mapping, const std::string &kv_cache_dtype, int64_t num_heads,
                int64_t head_size, const SelectRows *select) {
  // (looked at on every call: an address does not identify a tensor's shape)
  bulk_write(keys, values, check_layers(layers), slot_mapping, kv_cache_dtype, num_heads, head_size, select);
}

void cache_write_fp4(const at::Tensor &key, const at::Tensor &value, const at::Tensor &key_cache,
                     const at::Tensor &value_cache, const at::Tensor &slot_mapping, const at::Tensor &key_scale_cache,
                     const at::Tensor &value_scale_cache) {
  TORCH_CHECK(is_half(key), "Unsupported input dtype for reshape_and_cache_fp4. Must be half or bfloat16.");
  TORCH_CHECK(key.dim() == 3 && value.dim() == 3, "reshape_and_cache_flash_fp4: key/value must be [tokens, heads, head_size]");
  TORCH_CHECK(key_cache.dim() == 4 && value_cache.dim() == 4, "KV cache must be rank-4");
  const int64_t num_heads = key.size(1), head_size = key.size(2);
  const bool nhd = key_cache.size(2) == num_heads;   // [blocks, block, heads, head_size / 2], else heads first
  const int64_t block_stride = key_cache.stride(0);
  const int64_t page_stride = nhd ? key_cache.stride(1) : key_cache.stride(2);
  const int64_t head_stride = nhd ? key_cache.stride(2) : key_cache.stride(1);
  const int64_t block_size = nhd ? key_cache.size(1) : key_cache.size(2);
  TORCH_CHECK(value_cache.stride(0) == block_stride, "block_stride mismatch");
  TORCH_CHECK((nhd ? value_cache.stride(1) : value_cache.stride(2)) == page_stride, "page_stride mismatch");
  TORCH_CHECK((nhd ? value_cache.stride(2) : value_cache.stride(1)) == head_stride, "head_stride mismatch");
  TORCH_CHECK((nhd ? value_cache.size(1) : value_cache.size(2)) == block_size,
              "block_size mismatch between key_cache and value_cache");
  // assumed, not checked, by the reference (it would write out of bounds instead)
  TORCH_CHECK(value.scalar_type() == key.scalar_type() && value.sizes() == key.sizes(),
              "reshape_and_cache_flash_fp4: key/value mismatch");
  TORCH_CHECK(key.stride(2) == 1 && key.stride(1) == head_size && value.stride(2) == 1 && value.stride(1) == head_size,
              "reshape_and_cache_flash_fp4: heads of a token must be dense");
  TORCH_CHECK(slot_mapping.scalar_type() == at::kLong, "expected scalar type Long but found ", slot_mapping.scalar_type());
  TORCH_CHECK(key_cache.element_size() == 1 && value_cache.element_size() == 1 && key_scale_cache.element_size() == 1 &&
                  value_scale_cache.element_size() == 1,
              "reshape_and_cache_flash_fp4: caches and scale caches must be byte tensors");
  TORCH_CHECK(key_cache.size(3) * 2 == head_size && key_cache.stride(3) == 1,
              "reshape_and_cache_flash_fp4: cache last dim must be head_size / 2 packed bytes");
  TORCH_CHECK(key_scale_cache.numel() * 8 >= key_cache.numel() && value_scale_cache.numel() * 8 >= value_cache.numel(),
              "reshape_and_cache_flash_fp4: scale cache too small (one byte per 16 elements)");
  for (const at::Tensor *t : {&value, &key_cache, &value_cache, &slot_mapping, &key_scale_cache, &value_scale_cache})
    TORCH_CHECK(key.is_cuda() && t->device() == key.device(),
                "reshape_and_cache_flash_fp4: all tensors must be on one CUDA device");
  TORCH_CHECK(slot_mapping.dim() == 1 && (slot_mapping.size(0) <= 1 || slot_mapping.stride(0) == 1) &&
                  key.size(0) >= slot_mapping.size(0),
              "reshape_and_cache_flash_fp4: slot_mapping must be 1-D, contiguous and no longer than key has tokens");
  const DeviceGuard guard(key.device());
  check_rc(arctic_reshape_and_cache_flash_fp4(
      key.data_ptr(), value.data_ptr(), key.stride(0), value.stride(0), key_cache.data_ptr(), value_cache.data_ptr(),
      key_scale_cache.data_ptr(), value_scale_cache.data_ptr(), (const int64_t *)slot_mapping.data_ptr(),
      slot_mapping.size(0), to_int(num_heads, "num_heads"), to_int(head_size, "head_size"),
      to_int(block_size, "block_size"), block_stride, page_stride, head_stride, key_cache.size(0), half_code(key),
      current_stream()));
}

namespace {

// An embedding table [V, width] in the activations' type and one int64 token id per row.
void check_embedding(const char *fn, const at::Tensor &table, const at::Tensor &token_ids, const at::Tensor &like,
                     int64_t width, int64_t rows) {
  TORCH_CHECK(table.is_cuda() && token_ids.is_cuda() && table.device() == like.device() &&
                  token_ids.device() == like.device(),
              fn, ": embedding table and token ids must be on the input's device");
  TORCH_CHECK(table.scalar_type() == like.scalar_type(), fn, ": embedding table dtype must match input dtype");
  TORCH_CHECK(table.dim() == 2 && table.size(1) == width && table.stride(1) == 1, fn,
              ": embedding table must be [num_embeddings, ", width, "] with contiguous rows");
  TORCH_CHECK(table.size(0) > 0, fn, ": the embedding table has no rows");
  TORCH_CHECK(token_ids.scalar_type() == at::kLong, fn, ": token ids must be int64");
  TORCH_CHECK(token_ids.numel() == rows && token_ids.is_contiguous(), fn, ": one contiguous token id per row is needed (",
              token_ids.numel(), " ids, ", rows, " rows)");
}

}  // namespace

at::Tensor add_ln_act(const char *fn, const at::Tensor &input, const OptTensor &z, const OptTensor &token_ids,
                      const OptTensor &weight, const OptTensor &bias, double alpha, double eps,
                      const std::string &activation, double out_scale) {
  // the checks of csrc/custom_ops/speculator_ln.cu:152-201
  TORCH_CHECK(is_half(input), fn, ": only fp16 and bf16 are supported.");
  TORCH_CHECK(input.is_cuda(), fn, ": input must be CUDA");
  const auto dtype = input.scalar_type();
  const int64_t hidden = input.size(-1);
  TORCH_CHECK(hidden > 0, fn, ": hidden size must be > 0");
  TORCH_CHECK(input.stride(-1) == 1, fn, ": last dimension must be contiguous (stride -1 == 1)");
  if (given(weight)) {
    TORCH_CHECK(weight->is_cuda() && weight->device() == input.device(), "weight must be CUDA");
    TORCH_CHECK(weight->scalar_type() == dtype, "weight dtype must match input dtype");
    TORCH_CHECK(weight->dim() == 1 && weight->numel() == hidden, "weight must be 1D of size hidden");
    TORCH_CHECK(weight->is_contiguous(), "weight must be contiguous");
  }
  if (given(bias)) {
    TORCH_CHECK(bias->is_cuda() && bias->device() == input.device(), "bias must be CUDA");
    TORCH_CHECK(bias->scalar_type() == dtype, "bias dtype must match input dtype");
    TORCH_CHECK(bias->dim() == 1 && bias->numel() == hidden, "bias must be 1D of size hidden");
    TORCH_CHECK(bias->is_contiguous(), "bias must be contiguous");
  }
  int act = -1;
  if (activation == "none") act = ARCTIC_ACT_NONE;
  else if (activation == "gelu") act = ARCTIC_ACT_GELU;
  else if (activation == "gelu_tanh") act = ARCTIC_ACT_GELU_TANH;
  TORCH_CHECK(act >= 0, fn, ": activation must be one of ['gelu', 'gelu_tanh', 'none']");

  const at::Tensor in_2d = rows_of(input, hidden);
  const int64_t rows = in_2d.size(0);
  at::Tensor z_2d;
  if (given(token_ids)) {
    TORCH_CHECK(given(z), fn, ": token ids without an embedding table");
    check_embedding(fn, *z, *token_ids, input, hidden, rows);
  } else if (given(z)) {
    TORCH_CHECK(z->is_cuda() && z->device() == input.device(), "z must be CUDA, on the input's device");
    TORCH_CHECK(z->scalar_type() == dtype, "z dtype must match input dtype");
    TORCH_CHECK(z->sizes() == input.sizes(), "z must have the input's shape");
    TORCH_CHECK(z->stride(-1) == 1, fn, ": last dimension of z must be contiguous");
    z_2d = rows_of(*z, hidden);
  }
  at::Tensor out = at::empty_like(input);
  if (rows == 0) return out;
  const at::Tensor out_2d = rows_of(out, hidden);   // rows are written dense, `hidden` apart
  TORCH_CHECK(out_2d.stride(0) == hidden || rows == 1, fn, ": internal - output rows must be dense");
  const DeviceGuard guard(input.device());
  const int code = half_code(input);
  if (given(token_ids)) {
    check_rc(arctic_speculator_embed_add_ln_act(
        out_2d.data_ptr(), in_2d.data_ptr(), z->data_ptr(), (const int64_t *)token_ids->data_ptr(), optional_ptr(weight),
        optional_ptr(bias), rows, to_int(hidden, "hidden"), in_2d.stride(0), z->stride(0), z->size(0), (float)alpha,
        (float)eps, act, (float)out_scale, code, current_stream()));
  } else if (!z_2d.defined() && act == ARCTIC_ACT_NONE && out_scale == 1.0) {
    check_rc(arctic_speculator_ln(out_2d.data_ptr(), in_2d.data_ptr(), optional_ptr(weight), optional_ptr(bias), rows,
                                  to_int(hidden, "hidden"), in_2d.stride(0), (float)eps, code, current_stream()));
  } else {
    check_rc(arctic_speculator_add_ln_act(out_2d.data_ptr(), in_2d.data_ptr(), z_2d.defined() ? z_2d.data_ptr() : nullptr,
                                          optional_ptr(weight), optional_ptr(bias), rows, to_int(hidden, "hidden"),
                                          in_2d.stride(0), z_2d.defined() ? z_2d.stride(0) : 0, (float)alpha, (float)eps,
                                          act, (float)out_scale, code, current_stream()));
  }
  return out;
}

std::tuple<at::Tensor, at::Tensor> sum_lstm(const at::Tensor &states_4d, const at::Tensor &z, const OptTensor &token_ids,
                                            const OptTensor &prev_cell_d, const OptTensor &w_cell,
                                            const OptTensor &b_cell, const OptTensor &w_state,
                                            const OptTensor &b_state, double alpha, double eps_cell, double eps_state,
                                            bool use_fast_gelu, bool shared_z) {
  const auto dtype = states_4d.scalar_type();
  TORCH_CHECK(is_half(states_4d), "sum_lstm: only fp16 and bf16 are supported.");
  // not in the reference's schema: no prev_cell = the cell of zeros a proposal round starts from
  const bool zero_cell = !given(prev_cell_d);
  TORCH_CHECK(states_4d.is_cuda() && z.is_cuda() && (zero_cell || prev_cell_d->is_cuda()),
              "sum_lstm: inputs must be CUDA tensors");
  TORCH_CHECK(z.device() == states_4d.device() && (zero_cell || prev_cell_d->device() == states_4d.device()),
              "sum_lstm: inputs must be on one device");
  TORCH_CHECK(z.scalar_type() == dtype && (zero_cell || prev_cell_d->scalar_type() == dtype),
              "sum_lstm: all input dtypes must match");
  const int64_t hidden4 = states_4d.size(-1);
  TORCH_CHECK(hidden4 > 0 && hidden4 % 4 == 0, "sum_lstm: last dim of states must be 4*D_gate");
  const int64_t d_gate = hidden4 / 4;
  if (shared_z) {
    TORCH_CHECK(z.size(-1) == d_gate, "sum_lstm_shared_z: z must have last dim D_gate");
  } else {
    TORCH_CHECK(z.size(-1) == hidden4, "sum_lstm: z4 must have last dim 4*D_gate");
  }
  const int64_t d_cell = zero_cell ? d_gate : prev_cell_d->size(-1);
  TORCH_CHECK(d_cell == d_gate, "sum_lstm: prev_cell last dim must equal D_gate. Got ", d_cell, " vs expected ", d_gate, ".");
  TORCH_CHECK(states_4d.stride(-1) == 1 && z.stride(-1) == 1 && (zero_cell || prev_cell_d->stride(-1) == 1),
              "sum_lstm: last dimension must be contiguous (stride -1 == 1)");
  const char *names[4] = {"w_cell", "b_cell", "w_state", "b_state"};
  const OptTensor *vecs[4] = {&w_cell, &b_cell, &w_state, &b_state};
  for (int i = 0; i < 4; ++i) {
    if (!given(*vecs[i])) continue;
    const at::Tensor &t = **vecs[i];
    TORCH_CHECK(t.is_cuda() && t.device() == states_4d.device(), "sum_lstm: ", names[i], " must be CUDA");
    TORCH_CHECK(t.scalar_type() == dtype, "sum_lstm: ", names[i], " dtype mismatch");
    TORCH_CHECK(t.numel() >= d_gate, "sum_lstm: ", names[i], " must have length >= D_eff");
    TORCH_CHECK(t.is_contiguous(), "sum_lstm: ", names[i], " must be contiguous");
  }
  const at::Tensor s2 = rows_of(states_4d, hidden4);
  const int64_t rows = s2.size(0);
  at::Tensor z2, p2;
  if (!zero_cell) p2 = rows_of(*prev_cell_d, d_cell);
  if (given(token_ids)) {
    TORCH_CHECK(zero_cell || p2.size(0) == rows, "sum_lstm: row counts of the inputs differ");
    check_embedding("sum_lstm_embedded", z, *token_ids, states_4d, d_gate, rows);
  } else {
    z2 = rows_of(z, shared_z ? d_gate : hidden4);
    TORCH_CHECK(z2.size(0) == rows && (zero_cell || p2.size(0) == rows), "sum_lstm: row counts of the inputs differ");
  }
  at::Tensor out_cell, out_state, cell_shaped, state_shaped;
  if (zero_cell) {
    // dense outputs shaped like states_4d with its last dimension cut to D_gate
    out_cell = at::empty({rows, d_gate}, states_4d.options());
    out_state = at::empty({rows, d_gate}, states_4d.options());
    if (states_4d.dim() == 2) {
      cell_shaped = out_cell;
      state_shaped = out_state;
    } else {
      std::vector<int64_t> shape(states_4d.sizes().begin(), states_4d.sizes().end());
      shape.back() = d_gate;
      cell_shaped = out_cell.view(shape);
      state_shaped = out_state.view(shape);
    }
  } else {
    // outputs inherit prev_cell's row pitch (reference :356-365)
    out_cell = at::empty_strided(p2.sizes(), p2.strides(), p2.options());
    out_state = at::empty_strided(p2.sizes(), p2.strides(), p2.options());
    TORCH_CHECK(out_cell.stride(0) == out_state.stride(0), "sum_lstm: internal - output strides mismatch");
    const bool flat = prev_cell_d->dim() == 2;
    cell_shaped = flat ? out_cell : out_cell.view(prev_cell_d->sizes());
    state_shaped = flat ? out_state : out_state.view(prev_cell_d->sizes());
  }
  if (rows == 0) return std::make_tuple(state_shaped, cell_shaped);

  const void *pc = zero_cell ? nullptr : p2.data_ptr();
  const int64_t pc_stride = zero_cell ? 0 : p2.stride(0);
  const DeviceGuard guard(states_4d.device());
  const int code = half_code(states_4d);
  if (given(token_ids)) {
    check_rc(arctic_sum_lstm_embedded(
        out_state.data_ptr(), out_cell.data_ptr(), s2.data_ptr(), z.data_ptr(), (const int64_t *)token_ids->data_ptr(), pc,
        optional_ptr(w_cell), optional_ptr(b_cell), optional_ptr(w_state), optional_ptr(b_state), rows,
        to_int(d_gate, "d_gate"), s2.stride(0), z.stride(0), pc_stride, out_cell.stride(0), z.size(0), (float)alpha,
        (float)eps_cell, (float)eps_state, use_fast_gelu ? 1 : 0, code, current_stream()));
  } else {
    const auto entry = shared_z ? arctic_sum_lstm_shared_z : arctic_sum_lstm;
    check_rc(entry(out_state.data_ptr(), out_cell.data_ptr(), s2.data_ptr(), z2.data_ptr(), pc, optional_ptr(w_cell),
                   optional_ptr(b_cell), optional_ptr(w_state), optional_ptr(b_state), rows, to_int(d_gate, "d_gate"),
                   s2.stride(0), z2.stride(0), pc_stride, out_cell.stride(0), (float)alpha, (float)eps_cell,
                   (float)eps_state, use_fast_gelu ? 1 : 0, code, current_stream()));
  }
  return std::make_tuple(state_shaped, cell_shaped);
}

void move_rows(const char *fn, const TensorList &sources, const at::Tensor &indices, const TensorList &outs,
               bool scatter) {
  TORCH_CHECK(sources.count == outs.count, fn, ": ", sources.count, " sources but ", outs.count, " outputs");
  TORCH_CHECK(indices.is_cuda() && indices.dim() == 1 && indices.is_contiguous(), fn,
              ": indices must be a contiguous 1-D CUDA tensor");
  TORCH_CHECK(indices.scalar_type() == at::kInt || indices.scalar_type() == at::kLong, fn,
              ": indices must be int32 or int64");
  const int64_t n = indices.numel();
  const int64_t count = sources.count;
  if (n == 0 || count == 0) return;
  int64_t indexed_rows = -1;
  std::vector<const void *> src_ptr(count);
  std::vector<void *> dst_ptr(count);
  std::vector<int64_t> row_bytes(count), src_stride(count), dst_stride(count);
  for (int64_t k = 0; k < count; ++k) {
    const at::Tensor &src = sources[k], &dst = outs[k];
    TORCH_CHECK(src.is_cuda() && dst.is_cuda() && src.device() == indices.device() && dst.device() == indices.device(), fn,
                ": tensor ", k, ": sources, outputs and indices must be on one CUDA device");
    TORCH_CHECK(src.scalar_type() == dst.scalar_type(), fn, ": tensor ", k, ": source and output dtypes differ");
    TORCH_CHECK(src.dim() >= 1 && dst.dim() >= 1 && src.sizes().slice(1) == dst.sizes().slice(1), fn, ": tensor ", k,
                ": row shapes differ");
    TORCH_CHECK(src.size(0) == 0 || rows_dense(src), fn, ": tensor ", k, ": source rows must be contiguous");
    TORCH_CHECK(dst.size(0) == 0 || rows_dense(dst), fn, ": tensor ", k, ": output rows must be contiguous");
    const at::Tensor &indexed = scatter ? dst : src, &linear = scatter ? src : dst;
    TORCH_CHECK(linear.size(0) >= n, fn, ": tensor ", k, ": ", n, " indices but only ", linear.size(0), " rows");
    TORCH_CHECK(indexed_rows < 0 || indexed_rows == indexed.size(0), fn, ": indexed tensors differ in their number of rows");
    indexed_rows = indexed.size(0);
    const int64_t es = src.element_size();
    int64_t row = 1;
    for (int64_t d = 1; d < src.dim(); ++d) row *= src.size(d);
    row_bytes[k] = row * es;
    src_stride[k] = src.stride(0) * es;
    dst_stride[k] = dst.stride(0) * es;
    src_ptr[k] = src.data_ptr();
    dst_ptr[k] = dst.data_ptr();
  }
  const DeviceGuard guard(indices.device());
  check_rc(arctic_gather_rows(to_int(count, "count"), src_ptr.data(), dst_ptr.data(), row_bytes.data(),
                              src_stride.data(), dst_stride.data(), indices.data_ptr(), (int)indices.element_size(), n,
                              indexed_rows, scatter ? 1 : 0, current_stream()));
}

at::Tensor argmax_clamp(const at::Tensor &logits, int64_t max_index) {
  TORCH_CHECK(logits.is_cuda(), "speculator_argmax: logits must be CUDA");
  int code = -1;
  switch (logits.scalar_type()) {
    case at::kFloat: code = ARCTIC_DTYPE_F32; break;
    case at::kHalf: code = ARCTIC_DTYPE_F16; break;
    case at::kBFloat16: code = ARCTIC_DTYPE_BF16; break;
    default: break;
  }
  TORCH_CHECK(code >= 0, "speculator_argmax: logits must be fp32, fp16 or bf16");
  TORCH_CHECK(logits.dim() >= 1 && logits.size(-1) > 0, "speculator_argmax: logits need a non-empty last dimension");
  TORCH_CHECK(logits.stride(-1) == 1, "speculator_argmax: last dimension must be contiguous");
  TORCH_CHECK(max_index >= 0, "speculator_argmax: max_index must not be negative");
  const int64_t cols = logits.size(-1);
  const at::Tensor in_2d = rows_of(logits, cols);
  const int64_t rows = in_2d.size(0);
  at::Tensor out = at::empty(logits.sizes().slice(0, logits.dim() - 1), logits.options().dtype(at::kLong));
  if (rows == 0) return out;
  const DeviceGuard guard(logits.device());
  check_rc(arctic_argmax_clamp((int64_t *)out.data_ptr(), in_2d.data_ptr(), rows, to_int(cols, "cols"), in_2d.stride(0), max_index,
                               code, current_stream()));
  return out;
}

}  // namespace arctic_host

// ---- the four functions of the reference's custom_ops.h ------------------------------------------------------
namespace {

struct VectorLists {
  const std::vector<torch::Tensor> *list[4];
};
const at::Tensor &vector_lists_get(const void *ctx, int list, int64_t l) {
  return (*((const VectorLists *)ctx)->list[list])[(size_t)l];
}

}  // namespace

void reshape_and_cache_flash_bulk(torch::Tensor &keys, torch::Tensor &values,
                                  std::vector<torch::Tensor> const &key_caches,
                                  std::vector<torch::Tensor> const &value_caches, torch::Tensor &slot_mapping,
                                  const std::string &kv_cache_dtype, std::vector<torch::Tensor> const &k_scales,
                                  std::vector<torch::Tensor> const &v_scales, int64_t num_heads, int64_t head_size) {
  const VectorLists lists = {{&key_caches, &value_caches, &k_scales, &v_scales}};
  const arctic_host::LayerLists layers = {
      {(int64_t)key_caches.size(), (int64_t)value_caches.size(), (int64_t)k_scales.size(), (int64_t)v_scales.size()},
      vector_lists_get, &lists};
  arctic_host::bulk_write(keys, values, layers, slot_mapping, kv_cache_dtype, num_heads, head_size, nullptr);
}

void reshape_and_cache_flash_fp4(torch::Tensor &key, torch::Tensor &value, torch::Tensor &key_cache,
                                 torch::Tensor &value_cache, torch::Tensor &slot_mapping,
                                 const std::string &kv_cache_dtype, torch::Tensor &k_scale, torch::Tensor &v_scale,
                                 torch::Tensor &key_scale_cache, torch::Tensor &value_scale_cache) {
  (void)kv_cache_dtype, (void)k_scale, (void)v_scale;   // accepted and unused, as in the reference
  arctic_host::cache_write_fp4(key, value, key_cache, value_cache, slot_mapping, key_scale_cache, value_scale_cache);
}

torch::Tensor speculator_ln_cuda(const torch::Tensor &input, const c10::optional<torch::Tensor> &weight,
                                 const c10::optional<torch::Tensor> &bias, double eps) {
  return arctic_host::add_ln_act("speculator_ln", input, c10::nullopt, c10::nullopt, weight, bias, 0.0, eps, "none", 1.0);
}

std::tuple<torch::Tensor, torch::Tensor> sum_lstm_cuda(
    const torch::Tensor &states_4d, const torch::Tensor &z4_4d, const torch::Tensor &prev_cell_d,
    const c10::optional<torch::Tensor> &w_cell, const c10::optional<torch::Tensor> &b_cell,
    const c10::optional<torch::Tensor> &w_state, const c10::optional<torch::Tensor> &b_state, double alpha,
    double eps_cell, double eps_state, bool use_fast_gelu) {
  TORCH_CHECK(prev_cell_d.defined(), "sum_lstm: prev_cell_d is required");
  return arctic_host::sum_lstm(states_4d, z4_4d, c10::nullopt, prev_cell_d, w_cell, b_cell, w_state, b_state, alpha,
                               eps_cell, eps_state, use_fast_gelu, false);
}
