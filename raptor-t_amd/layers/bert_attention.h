// Mirrors sparse_transformers::layers::BertAttention (layers/bert_attention.h:18-53,
// layers/bert_attention.cpp:4-12): the self-attention functor the pybind module exposes.
// head count / width are read from the weights (the reference fixes 12 / 768 / 64).
#pragma once
#include "multi_headed_attention.h"

namespace sparse_transformers {
namespace layers {

class BertAttention : public MultiHeadedAttention {
 public:
  BertAttention(torch::Tensor qkv_weight, torch::Tensor qkv_bias, torch::Tensor dense_weight, torch::Tensor dense_bias,
                torch::Tensor layer_norm_weight, torch::Tensor layer_norm_bias, int64_t num_attention_heads,
                int layer_idx, bool async = true, double layer_norm_eps = 1e-5)
      : MultiHeadedAttention(torch::empty(0), torch::empty(0), torch::empty(0), torch::empty(0), torch::empty(0),
                             torch::empty(0), std::move(dense_weight), std::move(dense_bias), std::move(qkv_weight),
                             std::move(qkv_bias), std::move(layer_norm_weight), std::move(layer_norm_bias),
                             num_attention_heads, layer_idx, async, layer_norm_eps) {
    head_num_ = num_attention_heads;
    d_num_ = qkv_weight_.size(1);   // stored as [3D, D]
    block_size_ = RT_BLOCK;
    head_size_ = d_num_ / head_num_;
  }

  std::map<std::string, float> operator()(const torch::Tensor& input_tensor, const torch::Tensor& attention_mask,
                                          torch::Tensor& output, const std::vector<int> seq_position_info,
                                          torch::Tensor& seq_len_info_tensor,
                                          const torch::Tensor& partition_part_index_tensor,
                                          const torch::Tensor& partition_part_tensor, const int block_limit,
                                          std::map<std::string, float>& info, bool kernel_fusion = true,
                                          bool balanced = true) const;

  mutable int64_t head_num_, d_num_, block_size_, head_size_;
};

}  // namespace layers
}  // namespace sparse_transformers
