// pybind11 module `raptor_t`: the class surface of the reference's python/pybind.cpp:11-80
// (BertAttention, BertIntermediate, BertOutput, TensorSet, MetaData) over the MI355X
// layer functors.  Extra, optional constructor arguments carry what the reference
// hard-codes (LayerNorm eps); `set_plan` selects the random-block plan generator.
#include <pybind11/stl.h>
#include <torch/extension.h>
#include <hip/hip_runtime_api.h>

#include <cstdint>

#include "bert_attention.h"
#include "bert_intermediate.h"
#include "bert_output.h"
#include "metadata.h"

namespace py = pybind11;
using namespace sparse_transformers;

PYBIND11_MODULE(raptor_t, m) {
  m.def("timing_begin", &layers::kernels::timing_begin, py::arg("only") = std::vector<std::string>(), py::arg("every") = 1,
        "Start bracketing kernel launchers with HIP events (no synchronisation): every launcher, or only the "
        "named ones, and of those only one call in `every` (each pair of events costs the stream about 10 us).");
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
  m.def("event_pair_create", []() {
          hipEvent_t a = nullptr, b = nullptr;
          if (hipEventCreate(&a) != hipSuccess || hipEventCreate(&b) != hipSuccess) throw std::runtime_error("hipEventCreate failed");
          return std::make_pair(reinterpret_cast<std::uintptr_t>(a), reinterpret_cast<std::uintptr_t>(b));
        },
        "Two hipEvent_t as integers, for rt_time_next_launch (capi.time_next_launch) of a caller that drives the C "
        "ABI itself; event_pair_elapsed_us ends their life.");
  m.def("event_pair_elapsed_us", [](std::uintptr_t a, std::uintptr_t b) {
          hipEvent_t ea = reinterpret_cast<hipEvent_t>(a), eb = reinterpret_cast<hipEvent_t>(b);
          float ms = -1.0f;
          const bool ok = hipEventSynchronize(eb) == hipSuccess && hipEventElapsedTime(&ms, ea, eb) == hipSuccess;
          (void)hipEventDestroy(ea);
          (void)hipEventDestroy(eb);
          if (!ok) {
            (void)hipGetLastError();      // the failed query must not surface in the caller's next GPU call
            throw std::runtime_error("the events were never given to a launch, or the launch failed");
          }
          return double(ms) * 1000.0;
        },
        "Waits for the stop event, returns the microseconds between the two and destroys both.");
  // The tensor-level launchers the layer objects call, under the reference's names (layers/kernels/kernel.h):
  // for callers that drive single kernels, and so that their argument checks can be exercised without a GPU.
  {
    namespace k = layers::kernels;
    using Info = std::map<std::string, float>;
    py::module_ km = m.def_submodule("kernels", "tensor-level launchers (layers/kernels/kernel.h of the reference)");
    km.def("add_bias_and_transpose_kernel",
           [](const torch::Tensor& bias, torch::Tensor& qkv, torch::Tensor& q, torch::Tensor& kk, torch::Tensor& v,
              const torch::Tensor& seq_len_info, int batch, int heads, int block_num, int head_size, bool fusion) {
             Info info;
             k::add_bias_and_transpose_kernel(bias, qkv, q, kk, v, seq_len_info, batch, heads, block_num, head_size, info, fusion);
           },
           py::arg("bias"), py::arg("qkv"), py::arg("q"), py::arg("k"), py::arg("v"), py::arg("seq_len_info_tensor"),
           py::arg("batch_size"), py::arg("head_num"), py::arg("block_num"), py::arg("head_size") = 64,
           py::arg("kernel_fusion") = true);
    km.def("add_bias_and_layernorm_kernel",
           [](torch::Tensor& out, const torch::Tensor& residual, const torch::Tensor& bias, int seq_len, int width, float eps,
              const torch::Tensor& gamma, const torch::Tensor& beta, bool fusion) {
             Info info;
             k::add_bias_and_layernorm_kernel(out, residual, bias, seq_len, width, eps, gamma, beta, info, fusion);
           },
           py::arg("out"), py::arg("input_data"), py::arg("bias"), py::arg("seq_len"), py::arg("normalized_len"),
           py::arg("eps"), py::arg("layernorm_weight"), py::arg("layernorm_bias"), py::arg("kernel_fusion") = true);
    km.def("add_bias_act_kernel",
           [](const torch::Tensor& bias, torch::Tensor& out, int rows, int width, bool fusion) {
             Info info;
             k::add_bias_act_kernel(bias, out, rows, width, info, fusion);
           },
           py::arg("bias"), py::arg("out"), py::arg("total_seq_len"), py::arg("dim_size"), py::arg("kernel_fusion") = true);
    km.def("sparse_attention",
           [](const torch::Tensor& q, const torch::Tensor& kk, const torch::Tensor& v, torch::Tensor& out, int batch,
              const torch::Tensor& seq_len_info, const torch::Tensor& from_idx, const torch::Tensor& from_pos,
              const torch::Tensor& to_idx, const torch::Tensor& to_pos, int plan_heads, int block_limit, int block_num,
              int heads, bool balanced) {
             for (const torch::Tensor* t : {&to_idx, &to_pos})
               if (!t->defined() || !t->is_cuda() || !t->is_contiguous() || t->scalar_type() != torch::kInt32)
                 throw std::invalid_argument("sparse_attention: the block index must be contiguous int32 GPU tensors");
             if ((plan_heads != 1 && plan_heads != heads) || to_pos.numel() != int64_t(plan_heads) * block_num + 1)
               throw std::invalid_argument("sparse_attention: to_select_index_position must hold plan_heads * block_num + 1 entries");
             Info info;
             k::sparse_attention(q, kk, v, out, batch, seq_len_info, from_idx, from_pos, to_idx.data_ptr<int>(),
                                 to_pos.data_ptr<int>(), plan_heads, block_limit, block_num, heads, info, balanced);
           },
           py::arg("q"), py::arg("k"), py::arg("v"), py::arg("out"), py::arg("batch_size"), py::arg("seq_len_info_tensor"),
           py::arg("from_select_index"), py::arg("from_select_index_position"), py::arg("to_select_index"),
           py::arg("to_select_index_position"), py::arg("plan_heads"), py::arg("block_limit"), py::arg("block_num"),
           py::arg("head_num"), py::arg("balanced") = false);
  }

  m.def("plan_cache",
        [](int64_t max_bytes) {
          int64_t hits = 0, misses = 0;
          if (rt_meta_set_plan_cache(max_bytes, &hits, &misses) != RT_OK) throw std::runtime_error(rt_last_error_string());
          return std::make_pair(hits, misses);
        },
        py::arg("max_bytes") = -1,
        "Bound in bytes of the memo table of random-block plans the index workers draw from (0: keep nothing; negative: "
        "leave it as it is).  Returns (hits, misses) so far.");
  m.def("set_micro_batch_lane", &layers::set_current_lane, py::arg("lane"),
        "Selects which of the two independent sets of per-batch state (scratch tensors, published geometry, block-index "
        "pipeline, GEMM workspace) the following calls use: a caller that keeps two micro-batches in flight on two "
        "streams selects 0 or 1 before each call it makes for one of them.  Default 0.");
  m.def("micro_batch_lane", &layers::current_lane);

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
      .def_static("get_instance", []() { return layers::TensorSet::get_instance(); });

  py::class_<layers::MetaData>(m, "MetaData")
      .def(py::init([]() { return new layers::MetaData(); }))
      .def("update_meta_data", &layers::MetaData::update_meta_data)
      .def("terminate_thread", &layers::MetaData::terminate_thread)
      .def_static("set_plan",
                  [](int plan_mode, int policy, int max_pos) {
                    for (int lane = 0; lane < layers::LANES; ++lane)
                      layers::Semaphore::get_instance(lane)->set_plan(plan_mode, policy, max_pos);
                  },
                  py::arg("plan_mode") = int(RT_PLAN_HF), py::arg("policy") = int(RT_POLICY_REFERENCE_PATCHED),
                  py::arg("max_pos") = 4096)
      .def_static("set_index_check",
                  [](bool on) {
                    for (int lane = 0; lane < layers::LANES; ++lane)
                      layers::Semaphore::get_instance(lane)->set_index_check(on);
                  },
                  py::arg("on"),
                  "Debugging aid: every block index the workers build is checked on the host before it is uploaded; a "
                  "malformed one makes the attention layer raise instead of launching.");
}
