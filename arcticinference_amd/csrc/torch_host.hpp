// Host side of the operators above the C ABI of libarctic_mi355x.so, in C++ on torch tensors: the argument checks
// of the reference's launchers, the allocation of outputs the way they allocate them, and the hand-over of
// pointers, sizes and strides to the library on torch's current stream.  Defined in torch_forwards.cpp; used by the
// four functions of the reference's custom_ops.h (same file) and by the Python extension module in host_ext.cpp.
#pragma once

#include <torch/all.h>

#include <string>
#include <tuple>
#include <vector>

namespace arctic_host {

using OptTensor = c10::optional<at::Tensor>;

// The four per-layer tensor lists of a bulk write, however the caller holds them (a std::vector, a Python list):
// get(ctx, list, l) returns tensor l of list 0 (key caches), 1 (value caches), 2 (k scales) or 3 (v scales).
struct LayerLists {
  int64_t count[4];
  const at::Tensor &(*get)(const void *ctx, int list, int64_t l);
  const void *ctx;
  const at::Tensor &operator()(int list, int64_t l) const { return get(ctx, list, l); }
};

// The rows a bulk write also copies out: k_out[j] = keys[logits_indices[j]], v_out likewise.
struct SelectRows {
  const at::Tensor &logits_indices;
  const at::Tensor &k_out;
  const at::Tensor &v_out;
};

// What a bulk write needs to know of its layers, after every layer has been compared with layer 0: the four pointer
// tables of the C ABI and the geometry all layers share.  Holds addresses, not tensors: whoever keeps one beyond the
// call that made it must keep the tensors alive and unchanged as well (PreparedLayers of host_ext.cpp does).
struct CheckedLayers {
  int64_t num_layers = 0, block_size = 0, block_stride = 0, num_blocks = 0, cache_element_size = 0;
  c10::Device device = c10::Device(c10::kCPU);
  const char *scales_problem = nullptr;   // why the scales cannot serve an fp8 write, or nullptr
  std::vector<const void *> key_caches, value_caches;
  std::vector<const float *> k_scales, v_scales;
};
CheckedLayers check_layers(const LayerLists &layers);

// reshape_and_cache_flash_bulk (csrc/custom_ops/reshape_and_cache_flash_bulk.cu:77-144) and, with `select`, the
// variant that also gathers the selected rows (llama_swiftkv.py:663-679).  The first form checks the layers itself.
void bulk_write(const at::Tensor &keys, const at::Tensor &values, const LayerLists &layers,
                const at::Tensor &slot_mapping, const std::string &kv_cache_dtype, int64_t num_heads,
                int64_t head_size, const SelectRows *select);
void bulk_write(const at::Tensor &keys, const at::Tensor &values, const CheckedLayers &layers,
                const at::Tensor &slot_mapping, const std::string &kv_cache_dtype, int64_t num_heads,
                int64_t head_size, const SelectRows *select);

// reshape_and_cache_flash_fp4 (csrc/custom_ops/reshape_and_cache_flash_fp4.cu:256-337)
void cache_write_fp4(const at::Tensor &key, const at::Tensor &value, const at::Tensor &key_cache,
                     const at::Tensor &value_cache, const at::Tensor &slot_mapping, const at::Tensor &key_scale_cache,
                     const at::Tensor &value_scale_cache);

// speculator_ln_cuda (csrc/custom_ops/speculator_ln.cu:152-252) and the forms with the speculator's element-wise
// steps around the norm: z (or, with token_ids, an embedding table that z is looked up in), an activation
// ("none", "gelu", "gelu_tanh") and a scaling of the output.  `fn` names the operator in error messages.
at::Tensor add_ln_act(const char *fn, const at::Tensor &input, const OptTensor &z, const OptTensor &token_ids,
                      const OptTensor &weight, const OptTensor &bias, double alpha, double eps,
                      const std::string &activation, double out_scale);

// sum_lstm_cuda (csrc/custom_ops/sum_lstm.cu:293-473).  shared_z: `z` is the un-repeated [..., D] row; with
// token_ids it is an embedding table [V, D]; no prev_cell: the cell of zeros.  Returns (state, cell).
std::tuple<at::Tensor, at::Tensor> sum_lstm(const at::Tensor &states_4d, const at::Tensor &z, const OptTensor &token_ids,
                                            const OptTensor &prev_cell_d, const OptTensor &w_cell,
                                            const OptTensor &b_cell, const OptTensor &w_state,
                                            const OptTensor &b_state, double alpha, double eps_cell, double eps_state,
                                            bool use_fast_gelu, bool shared_z);

// A list of tensors, however the caller holds it.
struct TensorList {
  int64_t count;
  const at::Tensor &(*get)(const void *ctx, int64_t i);
  const void *ctx;
  const at::Tensor &operator[](int64_t i) const { return get(ctx, i); }
};

// gather_rows / scatter_rows: the index_select calls and the write-back of swiftkv_select
// (llama_swiftkv.py:663-679, 733-742) in one launch.
void move_rows(const char *fn, const TensorList &sources, const at::Tensor &indices, const TensorList &outs,
               bool scatter);

// torch.argmax(logits, -1).clamp_(0, max_index) (arctic_speculator.py:846-848, 862)
at::Tensor argmax_clamp(const at::Tensor &logits, int64_t max_index);

}  // namespace arctic_host
