#include "bert_intermediate.h"

#include <stdexcept>

namespace sparse_transformers {
namespace layers {

BertIntermediate::BertIntermediate(torch::Tensor dense_weight, torch::Tensor dense_bias)
    : dense_weight_(dense_weight.to(torch::kCUDA).contiguous()), dense_bias_(dense_bias.to(torch::kCUDA).contiguous()) {
  if (dense_weight_.dim() != 2 || dense_bias_.numel() != dense_weight_.size(1))
    throw std::invalid_argument("BertIntermediate: weight must be [D, F] and bias [F]");
  // kept as [F, D]: the GEMM is faster with both operands contiguous along the reduction
  dense_weight_ = dense_weight_.t().contiguous();
}

std::map<std::string, float> BertIntermediate::operator()(const torch::Tensor& input_tensor, torch::Tensor& output_tensor,
                                                          std::map<std::string, float>& info, bool kernel_fusion) const {
  rt_gemm_ctx* const handle_ = kernels::shared_gemm_handle();       // the current micro-batch lane's workspace
  if (kernel_fusion && kernels::gemm_epilogue_fusion()) {
    kernels::MatMulBiasGelu(input_tensor, dense_weight_, dense_bias_, output_tensor, handle_, info, "BertIntermediate",
                            true);
    return info;
  }
  kernels::MatMul(input_tensor, false, dense_weight_, true, 1.0, output_tensor, 0.0, handle_, "BertIntermediate");
  kernels::add_bias_act_kernel(dense_bias_, output_tensor, int(input_tensor.size(0)), int(dense_bias_.size(0)), info,
                               kernel_fusion);
  return info;
}

}  // namespace layers
}  // namespace sparse_transformers
