// FFN down-projection + fused bias + residual + LayerNorm.  Mirrors
// sparse_transformers::layers::BertOutput (layers/bert_output.h:10-44,
// layers/bert_output.cpp:7-44); the LayerNorm width comes from the weights and eps is a
// constructor argument (the reference fixes 768 and 1e-5).
#pragma once
#include <torch/torch.h>

#include <map>
#include <string>

#include "kernels.h"

namespace sparse_transformers {
namespace layers {

class BertOutput {
 public:
  BertOutput(torch::Tensor dense_weight, torch::Tensor dense_bias, torch::Tensor layer_norm_weight,
             torch::Tensor layer_norm_bias, double layer_norm_eps = 1e-5);
  std::map<std::string, float> operator()(const torch::Tensor& hidden_states, const torch::Tensor& input_tensor,
                                          torch::Tensor& output, std::map<std::string, float>& info,
                                          bool kernel_fusion = true) const;

 private:
  torch::Tensor dense_weight_, dense_bias_, layer_norm_weight_, layer_norm_bias_;
  float eps_;
};

}  // namespace layers
}  // namespace sparse_transformers
