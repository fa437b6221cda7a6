// Python extension module arcticinference_amd._host_ext: the host layer of torch_forwards.cpp as plain functions,
// one per operator schema of py_custom_ops.py, which binds them to the CUDA dispatch key and calls them directly
// for eager GPU calls.  The per-layer tensor lists of the bulk write are read in place from the Python list
// (borrowed references, no copy into a vector): at 40 layers that is 160 tensors per call, and what a serving
// process pays on every engine step.  A failed check raises RuntimeError, as TORCH_CHECK does in the reference.
#include <torch/csrc/autograd/python_variable.h>
#include <torch/extension.h>

#include <string>
#include <tuple>
#include <vector>

#include "torch_host.hpp"

namespace {

namespace py = pybind11;
using arctic_host::OptTensor;

// A Python list or tuple of tensors, read in place.
class TensorSequence {
 public:
  TensorSequence(const py::handle &obj, const char *what) {
    fast_ = py::reinterpret_steal<py::object>(PySequence_Fast(obj.ptr(), what));
    if (!fast_) throw py::error_already_set();
    count_ = PySequence_Fast_GET_SIZE(fast_.ptr());
    items_ = PySequence_Fast_ITEMS(fast_.ptr());
    for (Py_ssize_t i = 0; i < count_; ++i)
      TORCH_CHECK(THPVariable_Check(items_[i]), what, ": element ", (int64_t)i, " is not a Tensor");
  }
  int64_t size() const { return (int64_t)count_; }
  const at::Tensor &operator[](int64_t i) const { return THPVariable_Unpack(items_[i]); }

 private:
  py::object fast_;
  PyObject **items_ = nullptr;
  Py_ssize_t count_ = 0;
};

struct PyLayerLists {
  const TensorSequence *list[4];
};
const at::Tensor &py_layer_get(const void *ctx, int list, int64_t l) { return (*((const PyLayerLists *)ctx)->list[list])[l]; }
const at::Tensor &py_list_get(const void *ctx, int64_t i) { return (*(const TensorSequence *)ctx)[i]; }

void bulk(const at::Tensor &keys, const at::Tensor &values, const py::handle &key_caches, const py::handle &value_caches,
          const at::Tensor &slot_mapping, const std::string &kv_cache_dtype, const py::handle &k_scales,
          const py::handle &v_scales, int64_t num_heads, int64_t head_size, const arctic_host::SelectRows *select) {
  const TensorSequence kc(key_caches, "key_caches must be a list of Tensors"),
      vc(value_caches, "value_caches must be a list of Tensors"), ks(k_scales, "k_scales must be a list of Tensors"),
      vs(v_scales, "v_scales must be a list of Tensors");
  const PyLayerLists lists = {{&kc, &vc, &ks, &vs}};
  const arctic_host::LayerLists layers = {{kc.size(), vc.size(), ks.size(), vs.size()}, py_layer_get, &lists};
  arctic_host::bulk_write(keys, values, layers, slot_mapping, kv_cache_dtype, num_heads, head_size, select);
}

void reshape_and_cache_flash_bulk(const at::Tensor &keys, const at::Tensor &values, const py::handle &key_caches,
                                  const py::handle &value_caches, const at::Tensor &slot_mapping,
                                  const std::string &kv_cache_dtype, const py::handle &k_scales,
                                  const py::handle &v_scales, int64_t num_heads, int64_t head_size) {
  bulk(keys, values, key_caches, value_caches, slot_mapping, kv_cache_dtype, k_scales, v_scales, num_heads, head_size,
       nullptr);
}

void reshape_and_cache_flash_bulk_select(const at::Tensor &keys, const at::Tensor &values, const py::handle &key_caches,
                                         const py::handle &value_caches, const at::Tensor &slot_mapping,
                                         const std::string &kv_cache_dtype, const py::handle &k_scales,
                                         const py::handle &v_scales, int64_t num_heads, int64_t head_size,
                                         const at::Tensor &logits_indices, const at::Tensor &k_out,
                                         const at::Tensor &v_out) {
  const arctic_host::SelectRows select = {logits_indices, k_out, v_out};
  bulk(keys, values, key_caches, value_caches, slot_mapping, kv_cache_dtype, k_scales, v_scales, num_heads, head_size,
       &select);
}

// The per-layer tensors of a bulk write, checked once and held, for a caller that writes the same layers on every
// step (SwiftKV's caller rebuilds its four lists of views on every engine step, llama_swiftkv.py:594-615, which costs
// it more host time than the write).  The object keeps an alias of every tensor, so the addresses in its tables stay
// allocated and the geometry it checked cannot change under it; it must be rebuilt when the pool is (the caller
// knows: its kv_cache objects are new ones then).
class PreparedLayers {
 public:
  PreparedLayers(const py::handle &key_caches, const py::handle &value_caches, const py::handle &k_scales,
                 const py::handle &v_scales) {
    const TensorSequence kc(key_caches, "key_caches must be a list of Tensors"),
        vc(value_caches, "value_caches must be a list of Tensors"), ks(k_scales, "k_scales must be a list of Tensors"),
        vs(v_scales, "v_scales must be a list of Tensors");
    const TensorSequence *lists[4] = {&kc, &vc, &ks, &vs};
    for (const TensorSequence *list : lists)
      for (int64_t i = 0; i < list->size(); ++i) held_.push_back((*list)[i].alias());
    // the tables are made from the held aliases, not from the caller's objects
    offsets_[0] = 0;
    for (int k = 0; k < 4; ++k) offsets_[k + 1] = offsets_[k] + lists[k]->size();
    const arctic_host::LayerLists layers = {
        {kc.size(), vc.size(), ks.size(), vs.size()},
        [](const void *ctx, int list, int64_t l) -> const at::Tensor & {
          const PreparedLayers *self = (const PreparedLayers *)ctx;
          return self->held_[(size_t)(self->offsets_[list] + l)];
        },
        this};
    checked_ = arctic_host::check_layers(layers);
  }
  int64_t num_layers() const { return checked_.num_layers; }
  void write(const at::Tensor &keys, const at::Tensor &values, const at::Tensor &slot_mapping,
             const std::string &kv_cache_dtype, int64_t num_heads, int64_t head_size) const {
    arctic_host::bulk_write(keys, values, checked_, slot_mapping, kv_cache_dtype, num_heads, head_size, nullptr);
  }
  void write_select(const at::Tensor &keys, const at::Tensor &values, const at::Tensor &slot_mapping,
                    const std::string &kv_cache_dtype, int64_t num_heads, int64_t head_size,
                    const at::Tensor &logits_indices, const at::Tensor &k_out, const at::Tensor &v_out) const {
    const arctic_host::SelectRows select = {logits_indices, k_out, v_out};
    arctic_host::bulk_write(keys, values, checked_, slot_mapping, kv_cache_dtype, num_heads, head_size, &select);
  }

 private:
  std::vector<at::Tensor> held_;
  int64_t offsets_[5];
  arctic_host::CheckedLayers checked_;
};

void reshape_and_cache_flash_fp4(const at::Tensor &key, const at::Tensor &value, const at::Tensor &key_cache,
                                 const at::Tensor &value_cache, const at::Tensor &slot_mapping,
                                 const std::string &kv_cache_dtype, const at::Tensor &k_scale, const at::Tensor &v_scale,
                                 const at::Tensor &key_scale_cache, const at::Tensor &value_scale_cache) {
  (void)kv_cache_dtype, (void)k_scale, (void)v_scale;   // accepted and unused, as in the reference
  arctic_host::cache_write_fp4(key, value, key_cache, value_cache, slot_mapping, key_scale_cache, value_scale_cache);
}

at::Tensor speculator_ln_cuda(const at::Tensor &input, const OptTensor &weight, const OptTensor &bias, double eps) {
  return arctic_host::add_ln_act("speculator_ln", input, c10::nullopt, c10::nullopt, weight, bias, 0.0, eps, "none", 1.0);
}

at::Tensor speculator_add_ln_act_cuda(const at::Tensor &input, const OptTensor &z, const OptTensor &weight,
                                      const OptTensor &bias, double alpha, double eps, const std::string &activation,
                                      double out_scale) {
  return arctic_host::add_ln_act("speculator_add_ln_act", input, z, c10::nullopt, weight, bias, alpha, eps, activation,
                                 out_scale);
}

at::Tensor speculator_embed_add_ln_act_cuda(const at::Tensor &input, const at::Tensor &emb_weight,
                                            const at::Tensor &token_ids, const OptTensor &weight, const OptTensor &bias,
                                            double alpha, double eps, const std::string &activation, double out_scale) {
  return arctic_host::add_ln_act("speculator_embed_add_ln_act", input, emb_weight, token_ids, weight, bias, alpha, eps,
                                 activation, out_scale);
}

using TwoTensors = std::tuple<at::Tensor, at::Tensor>;

TwoTensors sum_lstm_cuda(const at::Tensor &states_4d, const at::Tensor &z4_4d, const OptTensor &prev_cell_d,
                         const OptTensor &w_cell, const OptTensor &b_cell, const OptTensor &w_state,
                         const OptTensor &b_state, double alpha, double eps_cell, double eps_state, bool use_fast_gelu) {
  return arctic_host::sum_lstm(states_4d, z4_4d, c10::nullopt, prev_cell_d, w_cell, b_cell, w_state, b_state, alpha,
                               eps_cell, eps_state, use_fast_gelu, false);
}

TwoTensors sum_lstm_zero_cell_cuda(const at::Tensor &states_4d, const at::Tensor &z4_4d, const OptTensor &w_cell,
                                   const OptTensor &b_cell, const OptTensor &w_state, const OptTensor &b_state,
                                   double alpha, double eps_cell, double eps_state, bool use_fast_gelu) {
  return arctic_host::sum_lstm(states_4d, z4_4d, c10::nullopt, c10::nullopt, w_cell, b_cell, w_state, b_state, alpha,
                               eps_cell, eps_state, use_fast_gelu, false);
}

TwoTensors sum_lstm_shared_z_cuda(const at::Tensor &states_4d, const at::Tensor &z_d, const OptTensor &prev_cell_d,
                                  const OptTensor &w_cell, const OptTensor &b_cell, const OptTensor &w_state,
                                  const OptTensor &b_state, double alpha, double eps_cell, double eps_state,
                                  bool use_fast_gelu) {
  return arctic_host::sum_lstm(states_4d, z_d, c10::nullopt, prev_cell_d, w_cell, b_cell, w_state, b_state, alpha,
                               eps_cell, eps_state, use_fast_gelu, true);
}

TwoTensors sum_lstm_embedded_cuda(const at::Tensor &states_4d, const at::Tensor &emb_weight, const at::Tensor &token_ids,
                                  const OptTensor &prev_cell_d, const OptTensor &w_cell, const OptTensor &b_cell,
                                  const OptTensor &w_state, const OptTensor &b_state, double alpha, double eps_cell,
                                  double eps_state, bool use_fast_gelu) {
  return arctic_host::sum_lstm(states_4d, emb_weight, token_ids, prev_cell_d, w_cell, b_cell, w_state, b_state, alpha,
                               eps_cell, eps_state, use_fast_gelu, true);
}

void move(const char *fn, const py::handle &sources, const at::Tensor &indices, const py::handle &outs, bool scatter) {
  const TensorSequence src(sources, "sources must be a list of Tensors"), dst(outs, "outs must be a list of Tensors");
  const arctic_host::TensorList s = {src.size(), py_list_get, &src}, d = {dst.size(), py_list_get, &dst};
  arctic_host::move_rows(fn, s, indices, d, scatter);
}
void gather_rows(const py::handle &sources, const at::Tensor &indices, const py::handle &outs) {
  move("gather_rows", sources, indices, outs, false);
}
void scatter_rows(const py::handle &sources, const at::Tensor &indices, const py::handle &outs) {
  move("scatter_rows", sources, indices, outs, true);
}

at::Tensor speculator_argmax_cuda(const at::Tensor &logits, int64_t max_index) {
  return arctic_host::argmax_clamp(logits, max_index);
}

}  // namespace

PYBIND11_MODULE(_host_ext, m) {
  m.doc() = "C++ host layer of the arctic_inference operators over libarctic_mi355x.so";
  m.def("reshape_and_cache_flash_bulk", &reshape_and_cache_flash_bulk);
  m.def("reshape_and_cache_flash_bulk_select", &reshape_and_cache_flash_bulk_select);
  m.def("reshape_and_cache_flash_fp4", &reshape_and_cache_flash_fp4);
  m.def("speculator_ln_cuda", &speculator_ln_cuda);
  m.def("speculator_add_ln_act_cuda", &speculator_add_ln_act_cuda);
  m.def("speculator_embed_add_ln_act_cuda", &speculator_embed_add_ln_act_cuda);
  m.def("sum_lstm_cuda", &sum_lstm_cuda);
  m.def("sum_lstm_zero_cell_cuda", &sum_lstm_zero_cell_cuda);
  m.def("sum_lstm_shared_z_cuda", &sum_lstm_shared_z_cuda);
  m.def("sum_lstm_embedded_cuda", &sum_lstm_embedded_cuda);
  m.def("gather_rows", &gather_rows);
  m.def("scatter_rows", &scatter_rows);
  m.def("speculator_argmax_cuda", &speculator_argmax_cuda);
  py::class_<PreparedLayers>(m, "BulkKVLayers")
      .def(py::init<const py::handle &, const py::handle &, const py::handle &, const py::handle &>(),
           py::arg("key_caches"), py::arg("value_caches"), py::arg("k_scales"), py::arg("v_scales"))
      .def_property_readonly("num_layers", &PreparedLayers::num_layers)
      .def("write", &PreparedLayers::write)
      .def("write_select", &PreparedLayers::write_select);
}
