// Attention sub-layer of the block-sparse encoder.
//
// Mirrors sparse_transformers::layers::MultiHeadedAttention
// (layers/multi_headed_attention.h:33-190, layers/multi_headed_attention.cpp:143-216):
// fused QKV weight [D, 3D] (Q|K|V) and bias, output projection [D, D] and bias, LayerNorm
// gamma/beta; operator() runs QKV GEMM -> bias/scale/head split -> block-sparse attention
// -> output GEMM -> bias + residual + LayerNorm, writing into the caller's `output`.
// Sizes come from the tensors, not from literals; the to-block CSR comes from the
// process-wide metadata pipeline (Semaphore) rather than a per-object worker thread.
#pragma once
#include <torch/torch.h>

#include <map>
#include <string>
#include <vector>

#include "kernels.h"
#include "semaphore.h"
#include "tensor_set.h"

namespace sparse_transformers {
namespace layers {

class MultiHeadedAttention {
 public:
  MultiHeadedAttention(torch::Tensor k_weight, torch::Tensor k_bias, torch::Tensor v_weight, torch::Tensor v_bias,
                       torch::Tensor q_weight, torch::Tensor q_bias, torch::Tensor dense_weight,
                       torch::Tensor dense_bias, torch::Tensor qkv_weight, torch::Tensor qkv_bias,
                       torch::Tensor layernorm_gamma, torch::Tensor layernorm_beta, int64_t num_attention_heads,
                       int layer_idx, bool async, double layer_norm_eps = 1e-5);

  // Host statement of the index builder kept for API compatibility
  // (layers/multi_headed_attention.cpp:15-140): builds this layer's CSR for the published
  // batch on the calling thread and returns (to_select_index, to_select_index_position).
  std::pair<std::vector<int>, std::vector<int>> GenerateSparseBlockIndex() const;

  // whether the QKV projection adds its bias in the GEMM's epilogue (both fusion switches on)
  static bool bias_in_projection(bool kernel_fusion);

  void FuseGemm012AddBIasTranspose(const torch::Tensor& input_tensor, torch::Tensor& q_out, torch::Tensor& k_out,
                                   torch::Tensor& v_out, torch::Tensor& seq_len_info_tensor, int total_seq_len,
                                   int d_num, std::map<std::string, float>& info, bool kernel_fusion) const;

  void operator()(const torch::Tensor& input_tensor, const torch::Tensor attention_mask, const std::string attn_type,
                  torch::Tensor& output, torch::Tensor att_score, const std::vector<int> seq_len_info,
                  torch::Tensor& seq_len_info_tensor, const int block_limit, const int head_size,
                  const int block_size, const int d_num, const torch::Tensor& from_select_index_position_tensor,
                  const torch::Tensor& from_select_index_tensor, std::map<std::string, float>& info,
                  bool kernel_fusion, bool balanced) const;

 protected:
  torch::Tensor dense_weight_, dense_bias_, qkv_weight_, qkv_bias_, layernorm_gamma_, layernorm_beta_;
  int64_t num_attention_heads_;
  int layer_idx_;
  bool async_;
  float eps_;
  mutable int total_seq_len_ = 0, head_num_ = 0, d_num_ = 0, block_size_ = 0, head_size_ = 0, block_num_ = 0,
              batch_size_ = 0;
};

}  // namespace layers
}  // namespace sparse_transformers
