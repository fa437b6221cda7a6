// The four functions that ArcticInference's csrc/custom_ops/custom_ops.h declares, as thin forwards to the C ABI
// of libarctic_mi355x.so.  Compiled together with the reference's own csrc/custom_ops/torch_bindings.cpp (unchanged:
// its TORCH_LIBRARY block binds exactly these four symbols, torch_bindings.cpp:6-51) this gives the reference's
// native extension for PyTorch-ROCm without any of its CUDA sources.  Host code only: any C++17 compiler, the torch
// headers and -larctic_mi355x.
//
// Each function repeats the argument checks of the launcher it stands for
//   reshape_and_cache_flash_bulk   csrc/custom_ops/reshape_and_cache_flash_bulk.cu:77-144
//   reshape_and_cache_flash_fp4    csrc/custom_ops/reshape_and_cache_flash_fp4.cu:256-337
//   speculator_ln_cuda             csrc/custom_ops/speculator_ln.cu:152-252
//   sum_lstm_cuda                  csrc/custom_ops/sum_lstm.cu:293-473
// allocates outputs as it does, and hands pointers, sizes and strides to the library on torch's current stream.
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/all.h>

#include <optional>
#include <string>
#include <tuple>
#include <vector>

#include "../../include/arctic_mi355x.h"

namespace {

using DeviceGuard = c10::hip::OptionalHIPGuardMasqueradingAsCUDA;

void *current_stream() { return (void *)c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream(); }

int half_dtype(const torch::Tensor &t, const char *message) {
  TORCH_CHECK(t.scalar_type() == at::kHalf || t.scalar_type() == at::kBFloat16, message);
  return t.scalar_type() == at::kHalf ? ARCTIC_DTYPE_F16 : ARCTIC_DTYPE_BF16;
}

const void *optional_ptr(const c10::optional<torch::Tensor> &t) {
  return t.has_value() && t->defined() ? t->data_ptr() : nullptr;
}

}  // namespace

void reshape_and_cache_flash_bulk(torch::Tensor &keys, torch::Tensor &values,
                                  std::vector<torch::Tensor> const &key_caches,
                                  std::vector<torch::Tensor> const &value_caches, torch::Tensor &slot_mapping,
                                  const std::string &kv_cache_dtype, std::vector<torch::Tensor> const &k_scales,
                                  std::vector<torch::Tensor> const &v_scales, int64_t num_heads, int64_t head_size) {
  const int64_t num_layers = (int64_t)key_caches.size();
  if (num_layers == 0) return;
  TORCH_CHECK(num_layers == (int64_t)value_caches.size());
  TORCH_CHECK(num_layers == (int64_t)k_scales.size());
  TORCH_CHECK(num_layers == (int64_t)v_scales.size());
  int kv;
  if (kv_cache_dtype == "auto") kv = ARCTIC_KV_AUTO;
  else if (kv_cache_dtype == "fp8" || kv_cache_dtype == "fp8_e4m3") kv = ARCTIC_KV_FP8_E4M3;
  else if (kv_cache_dtype == "fp8_e5m2") kv = ARCTIC_KV_FP8_E5M2;
  else TORCH_CHECK(false, "Unsupported data type of kv cache: ", kv_cache_dtype);
  int src;
  switch (keys.scalar_type()) {
    case at::kFloat: src = ARCTIC_DTYPE_F32; break;
    case at::kHalf: src = ARCTIC_DTYPE_F16; break;
    case at::kBFloat16: src = ARCTIC_DTYPE_BF16; break;
    default: TORCH_CHECK(false, "Unsupported input type of kv cache: ", keys.scalar_type());
  }
  TORCH_CHECK(values.scalar_type() == keys.scalar_type(), "reshape_and_cache_flash_bulk: keys and values dtype differ");
  TORCH_CHECK(slot_mapping.scalar_type() == at::kLong, "expected scalar type Long but found ", slot_mapping.scalar_type());
  TORCH_CHECK(keys.stride(-1) == 1 && values.stride(-1) == 1,
              "reshape_and_cache_flash_bulk: last dimension of keys/values must be contiguous");
  const int64_t block_stride = key_caches[0].stride(0);
  TORCH_CHECK(block_stride == value_caches[0].stride(0));
  const int64_t want_elem = kv == ARCTIC_KV_AUTO ? keys.element_size() : 1;
  std::vector<const void *> kc(num_layers), vc(num_layers);
  std::vector<const float *> ks(num_layers, nullptr), vs(num_layers, nullptr);
  for (int64_t l = 0; l < num_layers; ++l) {
    TORCH_CHECK(key_caches[l].element_size() == want_elem && value_caches[l].element_size() == want_elem,
                "reshape_and_cache_flash_bulk: cache element size does not match kv_cache_dtype '", kv_cache_dtype, "'");
    TORCH_CHECK(key_caches[l].stride(0) == block_stride && value_caches[l].stride(0) == block_stride &&
                    key_caches[l].size(0) == key_caches[0].size(0) && key_caches[l].size(1) == key_caches[0].size(1),
                "reshape_and_cache_flash_bulk: the caches of all layers must share block stride, blocks and block size");
    kc[l] = key_caches[l].data_ptr();
    vc[l] = value_caches[l].data_ptr();
    if (kv != ARCTIC_KV_AUTO) {
      TORCH_CHECK(k_scales[l].scalar_type() == at::kFloat && v_scales[l].scalar_type() == at::kFloat &&
                      k_scales[l].is_cuda() && v_scales[l].is_cuda(),
                  "reshape_and_cache_flash_bulk: k_scales / v_scales must be float32 device tensors");
      ks[l] = (const float *)k_scales[l].data_ptr();
      vs[l] = (const float *)v_scales[l].data_ptr();
    }
  }
  const DeviceGuard guard(keys.device());
  const int rc = arctic_reshape_and_cache_flash_bulk(
      keys.data_ptr(), values.data_ptr(), keys.stride(0), values.stride(0), kc.data(), vc.data(), ks.data(), vs.data(),
      (const int64_t *)slot_mapping.data_ptr(), slot_mapping.size(0), (int)num_layers, (int)num_heads, (int)head_size,
      (int)key_caches[0].size(1), block_stride, key_caches[0].size(0), src, kv, current_stream());
  TORCH_CHECK(rc == 0, arctic_last_error());
}

void reshape_and_cache_flash_fp4(torch::Tensor &key, torch::Tensor &value, torch::Tensor &key_cache,
                                 torch::Tensor &value_cache, torch::Tensor &slot_mapping,
                                 const std::string &kv_cache_dtype, torch::Tensor &k_scale, torch::Tensor &v_scale,
                                 torch::Tensor &key_scale_cache, torch::Tensor &value_scale_cache) {
  (void)kv_cache_dtype, (void)k_scale, (void)v_scale;   // accepted and unused, as in the reference
  const int dtype = half_dtype(key, "Unsupported input dtype for reshape_and_cache_fp4. Must be half or bfloat16.");
  TORCH_CHECK(key.dim() == 3 && value.dim() == 3, "reshape_and_cache_flash_fp4: key/value must be [tokens, heads, head_size]");
  TORCH_CHECK(key_cache.dim() == 4 && value_cache.dim() == 4, "KV cache must be rank-4");
  const int64_t num_heads = key.size(1), head_size = key.size(2);
  const bool nhd = key_cache.size(2) == num_heads;       // [blocks, block, heads, head_size / 2], else heads first
  const int64_t block_stride = key_cache.stride(0);
  const int64_t page_stride = nhd ? key_cache.stride(1) : key_cache.stride(2);
  const int64_t head_stride = nhd ? key_cache.stride(2) : key_cache.stride(1);
  const int64_t block_size = nhd ? key_cache.size(1) : key_cache.size(2);
  TORCH_CHECK(value_cache.stride(0) == block_stride, "block_stride mismatch");
  TORCH_CHECK((nhd ? value_cache.stride(1) : value_cache.stride(2)) == page_stride, "page_stride mismatch");
  TORCH_CHECK((nhd ? value_cache.stride(2) : value_cache.stride(1)) == head_stride, "head_stride mismatch");
  TORCH_CHECK(value.scalar_type() == key.scalar_type() && value.sizes() == key.sizes(),
              "reshape_and_cache_flash_fp4: key/value mismatch");
  TORCH_CHECK(key.stride(2) == 1 && key.stride(1) == head_size && value.stride(2) == 1 && value.stride(1) == head_size,
              "reshape_and_cache_flash_fp4: heads of a token must be dense");
  TORCH_CHECK(slot_mapping.scalar_type() == at::kLong, "expected scalar type Long but found ", slot_mapping.scalar_type());
  TORCH_CHECK(key_cache.size(3) * 2 == head_size && key_cache.stride(3) == 1,
              "reshape_and_cache_flash_fp4: cache last dim must be head_size / 2 packed bytes");
  const DeviceGuard guard(key.device());
  const int rc = arctic_reshape_and_cache_flash_fp4(
      key.data_ptr(), value.data_ptr(), key.stride(0), value.stride(0), key_cache.data_ptr(), value_cache.data_ptr(),
      key_scale_cache.data_ptr(), value_scale_cache.data_ptr(), (const int64_t *)slot_mapping.data_ptr(),
      slot_mapping.size(0), (int)num_heads, (int)head_size, (int)block_size, block_stride, page_stride, head_stride,
      key_cache.size(0), dtype, current_stream());
  TORCH_CHECK(rc == 0, arctic_last_error());
}

torch::Tensor speculator_ln_cuda(const torch::Tensor &input, const c10::optional<torch::Tensor> &weight,
                                 const c10::optional<torch::Tensor> &bias, double eps) {
  TORCH_CHECK(input.is_cuda(), "speculator_ln: input must be a CUDA tensor");
  const int dtype = half_dtype(input, "speculator_ln: only fp16 and bf16 are supported.");
  const int64_t hidden = input.size(-1);
  TORCH_CHECK(hidden > 0, "speculator_ln: hidden size must be > 0");
  TORCH_CHECK(input.stride(-1) == 1, "speculator_ln: last dimension must be contiguous (stride -1 == 1)");
  for (const auto *v : {&weight, &bias}) {
    if (!v->has_value()) continue;
    const torch::Tensor &t = **v;
    TORCH_CHECK(t.is_cuda(), "weight must be CUDA");
    TORCH_CHECK(t.scalar_type() == input.scalar_type(), "weight dtype must match input dtype");
    TORCH_CHECK(t.dim() == 1 && t.numel() == hidden, "weight must be 1D of size hidden");
    TORCH_CHECK(t.is_contiguous(), "weight must be contiguous");
  }
  const torch::Tensor in_2d = input.view({-1, hidden});
  torch::Tensor out = torch::empty_like(input);
  const int64_t rows = in_2d.size(0);
  if (rows == 0) return out;
  torch::Tensor out_2d = out.view({-1, hidden});      // the kernel writes rows `hidden` apart
  TORCH_CHECK(rows == 1 || out_2d.stride(0) == hidden, "speculator_ln: internal - output rows must be dense");
  const DeviceGuard guard(input.device());
  const int rc = arctic_speculator_ln(out_2d.data_ptr(), in_2d.data_ptr(), optional_ptr(weight), optional_ptr(bias), rows,
                                      (int)hidden, in_2d.stride(0), (float)eps, dtype, current_stream());
  TORCH_CHECK(rc == 0, arctic_last_error());
  return out;
}

std::tuple<torch::Tensor, torch::Tensor> sum_lstm_cuda(
    const torch::Tensor &states_4d, const torch::Tensor &z4_4d, const torch::Tensor &prev_cell_d,
    const c10::optional<torch::Tensor> &w_cell, const c10::optional<torch::Tensor> &b_cell,
    const c10::optional<torch::Tensor> &w_state, const c10::optional<torch::Tensor> &b_state, double alpha,
    double eps_cell, double eps_state, bool use_fast_gelu) {
  const int dtype = half_dtype(states_4d, "sum_lstm: only fp16 and bf16 are supported.");
  TORCH_CHECK(states_4d.is_cuda() && z4_4d.is_cuda() && prev_cell_d.is_cuda(), "sum_lstm: inputs must be CUDA tensors");
  TORCH_CHECK(z4_4d.scalar_type() == states_4d.scalar_type() && prev_cell_d.scalar_type() == states_4d.scalar_type(),
              "sum_lstm: all input dtypes must match");
  const int64_t hidden4 = states_4d.size(-1);
  TORCH_CHECK(hidden4 > 0 && hidden4 % 4 == 0, "sum_lstm: last dim of states must be 4*D_gate");
  const int64_t d_gate = hidden4 / 4;
  TORCH_CHECK(z4_4d.size(-1) == hidden4, "sum_lstm: z4 must have last dim 4*D_gate");
  TORCH_CHECK(prev_cell_d.size(-1) == d_gate, "sum_lstm: prev_cell last dim must equal D_gate. Got ", prev_cell_d.size(-1),
              " vs expected ", d_gate, ".");
  TORCH_CHECK(states_4d.stride(-1) == 1 && z4_4d.stride(-1) == 1 && prev_cell_d.stride(-1) == 1,
              "sum_lstm: last dimension must be contiguous (stride -1 == 1)");
  const char *names[4] = {"w_cell", "b_cell", "w_state", "b_state"};
  const c10::optional<torch::Tensor> *vecs[4] = {&w_cell, &b_cell, &w_state, &b_state};
  for (int i = 0; i < 4; ++i) {
    if (!vecs[i]->has_value()) continue;
    const torch::Tensor &t = **vecs[i];
    TORCH_CHECK(t.is_cuda(), "sum_lstm: ", names[i], " must be CUDA");
    TORCH_CHECK(t.scalar_type() == states_4d.scalar_type(), "sum_lstm: ", names[i], " dtype mismatch");
    TORCH_CHECK(t.numel() >= d_gate, "sum_lstm: ", names[i], " must have length >= D_eff");
    TORCH_CHECK(t.is_contiguous(), "sum_lstm: ", names[i], " must be contiguous");
  }
  const torch::Tensor s2 = states_4d.view({-1, hidden4}), z2 = z4_4d.view({-1, hidden4});
  const torch::Tensor p2 = prev_cell_d.view({-1, d_gate});
  const int64_t rows = s2.size(0);
  TORCH_CHECK(z2.size(0) == rows && p2.size(0) == rows, "sum_lstm: row counts of the inputs differ");
  // outputs inherit prev_cell's row pitch (sum_lstm.cu:356-365)
  torch::Tensor out_cell = torch::empty_strided(p2.sizes(), p2.strides(), p2.options());
  torch::Tensor out_state = torch::empty_strided(p2.sizes(), p2.strides(), p2.options());
  if (rows > 0) {
    const DeviceGuard guard(states_4d.device());
    const int rc = arctic_sum_lstm(out_state.data_ptr(), out_cell.data_ptr(), s2.data_ptr(), z2.data_ptr(), p2.data_ptr(),
                                   optional_ptr(w_cell), optional_ptr(b_cell), optional_ptr(w_state), optional_ptr(b_state),
                                   rows, (int)d_gate, s2.stride(0), z2.stride(0), p2.stride(0), out_cell.stride(0),
                                   (float)alpha, (float)eps_cell, (float)eps_state, use_fast_gelu ? 1 : 0, dtype,
                                   current_stream());
    TORCH_CHECK(rc == 0, arctic_last_error());
  }
  return std::make_tuple(out_state.view(prev_cell_d.sizes()), out_cell.view(prev_cell_d.sizes()));
}
