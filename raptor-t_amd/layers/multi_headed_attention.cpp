#include "multi_headed_attention.h"

#include <stdexcept>

namespace sparse_transformers {
namespace layers {

MultiHeadedAttention::MultiHeadedAttention(torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor,
                                           torch::Tensor, torch::Tensor dense_weight, torch::Tensor dense_bias,
                                           torch::Tensor qkv_weight, torch::Tensor qkv_bias,
                                           torch::Tensor layernorm_gamma, torch::Tensor layernorm_beta,
                                           int64_t num_attention_heads, int layer_idx, bool async,
                                           double layer_norm_eps)
    : dense_weight_(std::move(dense_weight)), dense_bias_(std::move(dense_bias)), qkv_weight_(std::move(qkv_weight)),
      qkv_bias_(std::move(qkv_bias)), layernorm_gamma_(std::move(layernorm_gamma)),
      layernorm_beta_(std::move(layernorm_beta)), num_attention_heads_(num_attention_heads), layer_idx_(layer_idx),
      async_(async), eps_(float(layer_norm_eps)) {
  if (qkv_weight_.dim() != 2 || qkv_weight_.size(1) != 3 * qkv_weight_.size(0))
    throw std::invalid_argument("qkv_weight must be [D, 3D] (Q|K|V along the output dimension)");
  const int64_t d = qkv_weight_.size(0);
  if (d % num_attention_heads != 0 || d / num_attention_heads != RT_HEAD_DIM)
    throw std::invalid_argument("hidden size must be 64 * num_attention_heads");
  if (dense_weight_.size(0) != d || dense_weight_.size(1) != d || qkv_bias_.numel() != 3 * d ||
      dense_bias_.numel() != d || layernorm_gamma_.numel() != d || layernorm_beta_.numel() != d)
    throw std::invalid_argument("attention parameter shapes do not match the hidden size");
  for (torch::Tensor* t : {&dense_weight_, &dense_bias_, &qkv_weight_, &qkv_bias_, &layernorm_gamma_, &layernorm_beta_})
    *t = t->to(torch::kCUDA).contiguous();
  // both kept as [out, in]: the GEMMs are faster with both operands contiguous along the reduction
  qkv_weight_ = qkv_weight_.t().contiguous();
  dense_weight_ = dense_weight_.t().contiguous();
  for (int lane = 0; lane < LANES; ++lane) {        // every micro-batch lane knows every layer
    TensorSet::get_instance(lane)->configure(d, qkv_weight_.scalar_type());
    Semaphore::get_instance(lane)->register_layer(layer_idx_, int(num_attention_heads), async);
  }
}

std::pair<std::vector<int>, std::vector<int>> MultiHeadedAttention::GenerateSparseBlockIndex() const {
  const std::vector<int> sb = TensorSet::get_instance()->seq_len_info_;
  if (sb.size() < 2) throw std::runtime_error("GenerateSparseBlockIndex: no batch has been published");
  // the plan the index pipeline of this lane draws (MetaData.set_plan): this function returns what the workers build
  int plan_mode = RT_PLAN_HF, policy = RT_POLICY_REFERENCE_PATCHED, max_pos = 4096;
  Semaphore::get_instance()->get_plan(&plan_mode, &policy, &max_pos);
  const int batch = int(sb.size()) - 1;
  const int plan_heads = plan_mode == RT_PLAN_REFERENCE ? 1 : int(num_attention_heads_);
  int64_t n_idx = 0, n_pos = 0;
  kernels::check(rt_meta_to_index_size(sb.data(), batch, plan_heads, &n_idx, &n_pos), "rt_meta_to_index_size");
  std::vector<int> idx(n_idx), pos(n_pos);
  kernels::check(rt_meta_build_to_index(sb.data(), batch, plan_heads, plan_mode, uint32_t(layer_idx_), max_pos, policy,
                                        nullptr, idx.data(), n_idx, pos.data(), n_pos),
                 "rt_meta_build_to_index");
  return {idx, pos};
}

bool MultiHeadedAttention::bias_in_projection(bool kernel_fusion) { return kernel_fusion && kernels::gemm_epilogue_fusion(); }

void MultiHeadedAttention::FuseGemm012AddBIasTranspose(const torch::Tensor& input_tensor, torch::Tensor& q_out,
                                                       torch::Tensor& k_out, torch::Tensor& v_out,
                                                       torch::Tensor& seq_len_info_tensor, int total_seq_len, int d_num,
                                                       std::map<std::string, float>& info, bool kernel_fusion) const {
  torch::Tensor tmp_qkv_out1 = TensorSet::get_instance()->get_tensor("tmp_qkv_out1");
  // With both fusions on, the projection adds its bias in the GEMM's epilogue (one rounding of the fp32 sum, no
  // extra pass) and the split kernel only changes the layout: the bias it is handed is undefined.
  if (bias_in_projection(kernel_fusion)) {
    kernels::MatMulBias(input_tensor, qkv_weight_, true, qkv_bias_, tmp_qkv_out1, kernels::shared_gemm_handle(),
                        "FuseGemm012AddBIasTranspose_MatMul");
    kernels::add_bias_and_transpose_kernel(torch::Tensor(), tmp_qkv_out1, q_out, k_out, v_out, seq_len_info_tensor,
                                           batch_size_, head_num_, block_num_, head_size_, info, kernel_fusion);
    return;
  }
  kernels::MatMul(input_tensor, false, qkv_weight_, true, 1, tmp_qkv_out1, 0, kernels::shared_gemm_handle(),
                  "FuseGemm012AddBIasTranspose_MatMul");
  kernels::add_bias_and_transpose_kernel(qkv_bias_, tmp_qkv_out1, q_out, k_out, v_out, seq_len_info_tensor, batch_size_,
                                         head_num_, block_num_, head_size_, info, kernel_fusion);
}

void MultiHeadedAttention::operator()(const torch::Tensor& input_tensor, const torch::Tensor attention_mask, const std::string attn_type,
                                      torch::Tensor& output, torch::Tensor, const std::vector<int> seq_len_info,
                                      torch::Tensor& seq_len_info_tensor, const int block_limit, const int head_size,
                                      const int block_size, const int d_num,
                                      const torch::Tensor& from_select_index_position_tensor,
                                      const torch::Tensor& from_select_index_tensor, std::map<std::string, float>& info,
                                      bool kernel_fusion, bool balanced) const {
  if (attn_type != "self") throw std::invalid_argument("only self attention is implemented");
  if (seq_len_info.size() < 2) throw std::invalid_argument("seq_position_info must hold at least one sequence");
  if (block_size != RT_BLOCK || head_size != RT_HEAD_DIM) throw std::invalid_argument("block size and head size must be 64");
  total_seq_len_ = seq_len_info.back() * block_size;
  batch_size_ = int(seq_len_info.size()) - 1;
  head_num_ = d_num / head_size;
  d_num_ = d_num;
  block_size_ = block_size;
  head_size_ = head_size;
  block_num_ = seq_len_info.back();
  if (input_tensor.dim() != 2 || input_tensor.size(0) != total_seq_len_ || input_tensor.size(1) != d_num ||
      output.numel() != input_tensor.numel())
    throw std::invalid_argument("input/output must be [total tokens, hidden] for the published batch");
  if (seq_len_info_tensor.numel() != int64_t(seq_len_info.size()))
    throw std::invalid_argument("seq_len_info_tensor does not match seq_position_info");
  // the scratch set, the index pipeline and the GEMM workspace of the current micro-batch lane
  const TensorSet::Ptr tensor_set = TensorSet::get_instance();
  const Semaphore::Ptr semaphore = Semaphore::get_instance();
  rt_gemm_ctx* const handle_ = kernels::shared_gemm_handle();
  if (tensor_set->seq_len_info_ != seq_len_info)
    throw std::invalid_argument("the batch passed to the layer is not the one published by MetaData::update_meta_data");

  torch::Tensor q_out = tensor_set->get_tensor("q_out");
  torch::Tensor k_out = tensor_set->get_tensor("k_out");
  torch::Tensor v_out = tensor_set->get_tensor("v_out");
  FuseGemm012AddBIasTranspose(input_tensor, q_out, k_out, v_out, seq_len_info_tensor, total_seq_len_, d_num_, info,
                              kernel_fusion);

  // hand-off from the index worker: host wait time is the reference's "pre_process"
  // (layers/multi_headed_attention.cpp:177-193)
  const int* to_idx = nullptr;
  const int* to_pos = nullptr;
  int plan_heads = 1;
  double wait_us = 0.0;
  void* stream = kernels::current_stream();
  semaphore->Wait(layer_idx_, stream, &to_idx, &to_pos, &plan_heads, &wait_us);
  auto pre = info.find("pre_process");
  if (pre != info.end()) pre->second += float(wait_us);

  torch::Tensor attention_out = tensor_set->get_tensor("attention_out");
  // under kernel_fusion the split kernel may have left Q in the projection's output (see kernels.h)
  const bool q_rows = kernel_fusion && kernels::attention_q_from_rows();
  kernels::sparse_attention(q_out, k_out, v_out, attention_out, batch_size_, seq_len_info_tensor,
                            from_select_index_tensor, from_select_index_position_tensor, to_idx, to_pos, plan_heads,
                            block_limit, block_num_, head_num_, info, balanced, attention_mask,
                            q_rows ? tensor_set->get_tensor("tmp_qkv_out1") : torch::Tensor(),
                            q_rows && !bias_in_projection(kernel_fusion) ? qkv_bias_ : torch::Tensor());
  semaphore->Release(layer_idx_, stream);

  kernels::MatMul(attention_out, false, dense_weight_, true, 1, output, 0, handle_, "Attention Output");
  kernels::add_bias_and_layernorm_kernel(output, input_tensor, dense_bias_, total_seq_len_, d_num_, eps_,
                                         layernorm_gamma_, layernorm_beta_, info, kernel_fusion);
}

}  // namespace layers
}  // namespace sparse_transformers
