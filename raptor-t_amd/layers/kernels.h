// Tensor-level launchers used by the layer functors: the names and argument meaning of
// layers/kernels/kernel.h and layers/kernels/mat_mul.h of the reference, each a thin
// shim over the C ABI in include/raptor_t_hip.h (which is where the GPU code lives).
//
// `info`: a key that the caller has pre-seeded is accumulated with the GPU time of the
// call in microseconds, measured with HIP events on the current stream (the reference
// takes host wall-clock around an asynchronous launch, which only means something under
// CUDA_LAUNCH_BLOCKING=1; layers/kernels/add_bias_act.cu:129-132).
#pragma once
#include <torch/torch.h>

#include <map>
#include <string>
#include <vector>

#include "../../include/raptor_t_hip.h"
#include "tensor_set.h"

namespace sparse_transformers {
namespace layers {
namespace kernels {

enum class ActivationType { Gelu = 0, Tanh = 1, Relu = 2 };

void* current_stream();
int dtype_code(const torch::Tensor& t);
void check(int rc, const char* what);
// One hipBLASLt context (heuristic cache + workspace) per micro-batch lane (tensor_set.h), shared by every
// layer of the process; the reference creates a cuBLAS handle per layer object (multi_headed_attention.h:94).
// Two lanes run on two streams at once and must not share a workspace.
rt_gemm_ctx* shared_gemm_handle();

// Deferred timing: between timing_begin() and timing_collect() every launcher below
// brackets its kernel with a pair of HIP events on the current stream WITHOUT
// synchronising; timing_collect() synchronises once and returns, per launcher name,
// (total microseconds, number of launches).  Lets a harness time kernels inside an
// otherwise free-running loop.
// `every` > 1 times only one in `every` calls of each launcher: a pair of events costs the stream 5 to 10 us,
// which a measurement of whole steps should not pay at every launch.
void timing_begin(const std::vector<std::string>& only = {}, int every = 1);
std::map<std::string, std::pair<double, int64_t>> timing_collect();

// RAII timer: accumulates into info[key] only when the key already exists (synchronous),
// and feeds the deferred timing when it is active.  `own_dispatch`: the launcher starts exactly one kernel of
// the library; its events then carry the dispatch's own start and end (rt_time_next_launch), the duration a
// profiler reports.  Otherwise (vendor GEMMs) the events are recorded on the stream before and after the call
// and also count the gaps to the neighbouring kernels.
class ScopedGpuTimer {
 public:
  ScopedGpuTimer(std::map<std::string, float>& info, const char* key, bool own_dispatch = false);
  ~ScopedGpuTimer();

 private:
  float* slot_ = nullptr;
  bool deferred_ = false;
  const char* key_ = nullptr;
  void* start_ = nullptr;
  void* stop_ = nullptr;
  bool own_dispatch_ = false;
};

// kernels::MatMul (layers/kernels/mat_mul.cpp:9-96): out[M,N] = A[M,K] . B[K,N], or
// A[M,K] . B[N,K]^T with b_trans (the faster layout here: both operands contiguous along K);
// a_trans, alpha != 1 and beta != 0, which no layer uses, are refused.
void MatMul(const torch::Tensor& A, bool a_trans, const torch::Tensor& B, bool b_trans, float alpha,
            torch::Tensor& out, float beta, rt_gemm_ctx* handle, const std::string& name);

// MatMul with the bias add in the GEMM's epilogue: out[M,N] = A . B(^T) + bias[N], rounded once.  What the
// reference does with MatMul followed by a bias kernel (layers/multi_headed_attention.cpp:154-175).  Times itself
// under "MatMul".
void MatMulBias(const torch::Tensor& A, const torch::Tensor& B, bool b_trans, const torch::Tensor& bias, torch::Tensor& out,
                rt_gemm_ctx* handle, const std::string& name);

// MatMul followed by add_bias_act_kernel, as one GEMM with the bias add and the tanh GELU in
// its epilogue (what BertIntermediate's pair of calls, layers/bert_intermediate.cpp:22-30,
// computes).  Times itself under "MatMul_bias_gelu".
void MatMulBiasGelu(const torch::Tensor& A, const torch::Tensor& B, const torch::Tensor& bias, torch::Tensor& out,
                    rt_gemm_ctx* handle, std::map<std::string, float>& info, const std::string& name,
                    bool b_trans = false);
// Whether BertIntermediate uses MatMulBiasGelu when kernel_fusion is asked for (default) or
// keeps the GEMM and the bias + GELU kernel apart.
void set_gemm_epilogue_fusion(bool on);
bool gemm_epilogue_fusion();

// Whether, under kernel_fusion, the attention kernel takes its queries from the QKV projection's
// own output rows (bias and scale applied as each unit loads its tile) and the split kernel writes
// only K and V^T (default), or the split kernel materialises Q too, as the reference always does.
void set_attention_q_from_rows(bool on);
bool attention_q_from_rows();

// Start-up tuning for a server: runs the four GEMMs of an encoder layer (hidden -> 3*hidden,
// hidden -> hidden, hidden -> ffn with bias + GELU, ffn -> hidden; weights as [out, in]) once for every
// token count in `token_counts` on the shared context, so that no later batch of one of these sizes
// pays for the timing of candidates.  Uses scratch operands of its own; returns the seconds it took.
double tune_layer_gemms(const std::vector<int64_t>& token_counts, int64_t hidden, int64_t ffn, torch::ScalarType dtype);

// What `balanced = true` means for the attention launch.  The reference's balanced kernel walks the
// host's LPT partition (python/util.py:11-34); here the persistent kernel balances itself with an
// XCD-aware schedule of its own that keeps each (sequence, head) group in one L2 and measures 20 %
// faster than walking that partition, so by default (false) a balanced launch uses it and the
// partition tensors are only checked for shape.  true: walk the host's partition as the reference does.
void set_attention_host_plan(bool on);
bool attention_host_plan();

// layers/kernels/add_bias_and_transpose.cu:212-233
void add_bias_and_transpose_kernel(const torch::Tensor& bias, torch::Tensor& input_data, torch::Tensor& q,
                                   torch::Tensor& k, torch::Tensor& v, const torch::Tensor& seq_len_info_tensor,
                                   int batch_size, int head_num, int block_num, int head_size,
                                   std::map<std::string, float>& info, bool kernel_fusion);

// layers/kernels/add_bias_and_layernorm.cu:268-285
void add_bias_and_layernorm_kernel(torch::Tensor& out, const torch::Tensor& input_data, const torch::Tensor& bias,
                                   int seq_len, int normalized_len, float eps, const torch::Tensor& layernorm_weight,
                                   const torch::Tensor& layernorm_bias, std::map<std::string, float>& info,
                                   bool kernel_fusion);

// layers/kernels/add_bias_act.cu:114-133
void add_bias_act_kernel(const torch::Tensor& bias, torch::Tensor& out, int total_seq_len, int dim_size,
                         std::map<std::string, float>& info, bool kernel_fusion);

// kernels::test_gemm_1 (layers/kernels/sparse_attention.cu:3192-3228): block-sparse attention
void sparse_attention(const torch::Tensor& q, const torch::Tensor& k, const torch::Tensor& v, torch::Tensor& out,
                      int batch_size, const torch::Tensor& seq_len_info_tensor, const torch::Tensor& from_select_index,
                      const torch::Tensor& from_select_index_position, const int* to_select_index,
                      const int* to_select_index_position, int plan_heads, int block_limit, int block_num,
                      int head_num, std::map<std::string, float>& info, bool balanced,
                      const torch::Tensor& seq_tokens = torch::Tensor(), const torch::Tensor& qkv_rows = torch::Tensor(),
                      const torch::Tensor& qkv_bias = torch::Tensor());
// seq_tokens (optional, int32 on the GPU, one entry per sequence): true token counts of sequences
// whose last block ends in padding; the padded keys get no weight.
// qkv_rows + qkv_bias (optional, the [T, 3*H*64] projection output and its bias): the queries are
// read from there and `q` is ignored.

}  // namespace kernels
}  // namespace layers
}  // namespace sparse_transformers
