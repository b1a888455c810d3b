// FFN up-projection + fused bias + GELU.  Mirrors sparse_transformers::layers::BertIntermediate
// (layers/bert_intermediate.h:10-35, layers/bert_intermediate.cpp:7-29).
#pragma once
#include <torch/torch.h>

#include <map>
#include <string>

#include "kernels.h"

namespace sparse_transformers {
namespace layers {

class BertIntermediate {
 public:
  BertIntermediate(torch::Tensor dense_weight, torch::Tensor dense_bias);
  std::map<std::string, float> operator()(const torch::Tensor& input_tensor, torch::Tensor& output,
                                          std::map<std::string, float>& info, bool kernel_fusion = true) const;

 private:
  torch::Tensor dense_weight_, dense_bias_;
};

}  // namespace layers
}  // namespace sparse_transformers
