#include "bert_output.h"

#include <stdexcept>

namespace sparse_transformers {
namespace layers {

BertOutput::BertOutput(torch::Tensor dense_weight, torch::Tensor dense_bias, torch::Tensor layer_norm_weight,
                       torch::Tensor layer_norm_bias, double layer_norm_eps)
    : dense_weight_(dense_weight.to(torch::kCUDA).contiguous()), dense_bias_(dense_bias.to(torch::kCUDA).contiguous()),
      layer_norm_weight_(layer_norm_weight.to(torch::kCUDA).contiguous()),
      layer_norm_bias_(layer_norm_bias.to(torch::kCUDA).contiguous()), eps_(float(layer_norm_eps)) {
  if (dense_weight_.dim() != 2 || dense_bias_.numel() != dense_weight_.size(1) ||
      layer_norm_weight_.numel() != dense_weight_.size(1) || layer_norm_bias_.numel() != dense_weight_.size(1))
    throw std::invalid_argument("BertOutput: weight must be [F, D], bias / gamma / beta [D]");
  dense_weight_ = dense_weight_.t().contiguous();      // kept as [D, F], see BertIntermediate
}

std::map<std::string, float> BertOutput::operator()(const torch::Tensor& hidden_states, const torch::Tensor& input_tensor,
                                                    torch::Tensor& output_tensor, std::map<std::string, float>& info,
                                                    bool kernel_fusion) const {
  kernels::MatMul(hidden_states, false, dense_weight_, true, 1.0, output_tensor, 0.0, kernels::shared_gemm_handle(),
                  "BertOutput");
  const int seq_len = int(input_tensor.size(0));
  kernels::add_bias_and_layernorm_kernel(output_tensor, input_tensor, dense_bias_, seq_len, int(dense_weight_.size(0)),
                                         eps_, layer_norm_weight_, layer_norm_bias_, info, kernel_fusion);
  return info;
}

}  // namespace layers
}  // namespace sparse_transformers
