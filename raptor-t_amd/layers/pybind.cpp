// pybind11 module `raptor_t`: the class surface of the reference's python/pybind.cpp:11-80
// (BertAttention, BertIntermediate, BertOutput, TensorSet, MetaData) over the MI355X
// layer functors.  Extra, optional constructor arguments carry what the reference
// hard-codes (LayerNorm eps); `set_plan` selects the random-block plan generator.
#include <pybind11/stl.h>
#include <torch/extension.h>

#include "bert_attention.h"
#include "bert_intermediate.h"
#include "bert_output.h"
#include "metadata.h"

namespace py = pybind11;
using namespace sparse_transformers;

PYBIND11_MODULE(raptor_t, m) {
  m.def("timing_begin", &layers::kernels::timing_begin, py::arg("only") = std::vector<std::string>(),
        "Start bracketing kernel launchers with HIP events (no synchronisation): every launcher, or only the "
        "named ones (each pair of events costs a few microseconds between kernels).");
  m.def("set_gemm_epilogue_fusion", &layers::kernels::set_gemm_epilogue_fusion,
        "BertIntermediate with kernel_fusion runs bias + GELU in the GEMM's epilogue (True, the default) or as the "
        "separate add_bias_act kernel (False).");
  m.def("gemm_epilogue_fusion", &layers::kernels::gemm_epilogue_fusion);
  m.def("tune_layer_gemms",
        [](const std::vector<int64_t>& token_counts, int64_t hidden, int64_t ffn, py::object dtype) {
          return layers::kernels::tune_layer_gemms(token_counts, hidden, ffn,
                                                   torch::python::detail::py_object_to_dtype(dtype));
        },
        py::arg("token_counts"), py::arg("hidden"), py::arg("ffn"), py::arg("dtype"),
        "Run the four GEMMs of an encoder layer once for every token count (start-up tuning of a server: the first "
        "call with a new token count times a few candidate kernels); returns the seconds spent.");
  m.def("set_attention_host_plan", &layers::kernels::set_attention_host_plan,
        "balanced=True launches walk the host's LPT partition like the reference (True) or let the persistent kernel "
        "balance itself with its own XCD-aware schedule, which is faster (False, the default).");
  m.def("attention_host_plan", &layers::kernels::attention_host_plan);
  m.def("set_attention_q_from_rows", &layers::kernels::set_attention_q_from_rows,
        "With kernel_fusion the attention kernel reads its queries from the QKV projection's output and the split "
        "kernel writes only K and V (True, the default), or the split kernel also writes Q (False).  Set it "
        "between layer calls, not during one.");
  m.def("attention_q_from_rows", &layers::kernels::attention_q_from_rows);
  m.def("timing_collect", &layers::kernels::timing_collect,
        "Synchronise and return {launcher: (total microseconds, launches)} since timing_begin().");
  py::class_<layers::BertAttention>(m, "BertAttention")
      .def(py::init([](torch::Tensor& qkv_weight, torch::Tensor& qkv_bias, torch::Tensor& dense_weight,
                       torch::Tensor& dense_bias, torch::Tensor& layer_norm_weight, torch::Tensor& layer_norm_bias,
                       int64_t num_attention_heads, int layer_idx, bool async, double layer_norm_eps) {
             return new layers::BertAttention(std::move(qkv_weight), std::move(qkv_bias), std::move(dense_weight),
                                              std::move(dense_bias), std::move(layer_norm_weight),
                                              std::move(layer_norm_bias), num_attention_heads, layer_idx, async,
                                              layer_norm_eps);
           }),
           py::arg("qkv_weight"), py::arg("qkv_bias"), py::arg("dense_weight"), py::arg("dense_bias"),
           py::arg("layer_norm_weight"), py::arg("layer_norm_bias"), py::arg("num_attention_heads"),
           py::arg("layer_idx"), py::arg("async_") = true, py::arg("layer_norm_eps") = 1e-5)
      .def("__call__", &layers::BertAttention::operator(), py::arg("input_tensor"), py::arg("attention_mask"),
           py::arg("output"), py::arg("seq_position_info"), py::arg("seq_len_info_tensor"),
           py::arg("partition_part_index_tensor"), py::arg("partition_part_tensor"), py::arg("block_limit"),
           py::arg("info"), py::arg("kernel_fusion") = true, py::arg("balanced") = true)
      .def("generate_sparse_block_index", &layers::BertAttention::GenerateSparseBlockIndex);

  py::class_<layers::BertIntermediate>(m, "BertIntermediate")
      .def(py::init([](torch::Tensor& dense_weight, torch::Tensor& dense_bias) {
        return new layers::BertIntermediate(std::move(dense_weight), std::move(dense_bias));
      }))
      .def("__call__", &layers::BertIntermediate::operator(), py::arg("input_tensor"), py::arg("output"),
           py::arg("info"), py::arg("kernel_fusion") = true);

  py::class_<layers::BertOutput>(m, "BertOutput")
      .def(py::init([](torch::Tensor& dense_weight, torch::Tensor& dense_bias, torch::Tensor& layer_norm_weight,
                       torch::Tensor& layer_norm_bias, double layer_norm_eps) {
             return new layers::BertOutput(std::move(dense_weight), std::move(dense_bias), std::move(layer_norm_weight),
                                           std::move(layer_norm_bias), layer_norm_eps);
           }),
           py::arg("dense_weight"), py::arg("dense_bias"), py::arg("layer_norm_weight"), py::arg("layer_norm_bias"),
           py::arg("layer_norm_eps") = 1e-5)
      .def("__call__", &layers::BertOutput::operator(), py::arg("hidden_states"), py::arg("input_tensor"),
           py::arg("output"), py::arg("info"), py::arg("kernel_fusion") = true);

  py::class_<layers::TensorSet, std::shared_ptr<layers::TensorSet>>(m, "TensorSet")
      .def(py::init([](int64_t total_seq_len, int64_t to_select_index_len, int64_t to_select_index_position_len) {
        return std::make_shared<layers::TensorSet>(total_seq_len, to_select_index_len, to_select_index_position_len);
      }))
      .def("update_tensor_set", &layers::TensorSet::update_tensor_set)
      .def("get_tensor", &layers::TensorSet::get_tensor)
      .def_static("get_instance", &layers::TensorSet::get_instance);

  py::class_<layers::MetaData>(m, "MetaData")
      .def(py::init([]() { return new layers::MetaData(); }))
      .def("update_meta_data", &layers::MetaData::update_meta_data)
      .def("terminate_thread", &layers::MetaData::terminate_thread)
      .def_static("set_plan",
                  [](int plan_mode, int policy, int max_pos) {
                    layers::Semaphore::get_instance()->set_plan(plan_mode, policy, max_pos);
                  },
                  py::arg("plan_mode") = int(RT_PLAN_HF), py::arg("policy") = int(RT_POLICY_REFERENCE_PATCHED),
                  py::arg("max_pos") = 4096);
}
