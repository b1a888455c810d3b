// Process-wide scratch tensors of the attention sub-layer and the published batch geometry.
//
// Mirrors sparse_transformers::layers::TensorSet (layers/tensor_set.h:15-68,
// layers/tensor_set.cpp:10-34): the same names (`q_out`, `k_out`, `v_out`,
// `attention_out`, `tmp_qkv_out1`), the same `update_tensor_set` / `get_tensor` /
// `get_instance` surface.  Unlike the reference the width and dtype are not literals
// (768 / half): `configure(hidden, dtype)` re-types the set, and an unknown name throws
// instead of printing and returning an empty tensor.
#pragma once
#include <torch/torch.h>

#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

namespace sparse_transformers {
namespace layers {

// Micro-batch lanes.  The process keeps LANES independent sets of the per-batch state (scratch tensors,
// published geometry, block-index pipeline, GEMM workspace); get_instance() of TensorSet and Semaphore and
// kernels::shared_gemm_handle() return the current lane's.  A caller that runs two micro-batches on two
// streams selects the lane before every call it makes for one of them; everybody else stays on lane 0 and
// sees the reference's single set.  The selection is a plain process-wide value: calls are issued from one
// host thread.  No counterpart in the reference, which keeps one batch in flight.
constexpr int LANES = 2;
int current_lane();
void set_current_lane(int lane);

class TensorSet {
 public:
  typedef std::shared_ptr<TensorSet> Ptr;
  std::vector<int> seq_len_info_;
  int total_seq_len_ = 0;
  int to_select_index_len_ = 0;
  int to_select_index_position_len_ = 0;

  TensorSet(int64_t total_seq_len, int64_t to_select_index_len, int64_t to_select_index_position_len);

  // Width / dtype of the scratch set (defaults: 768, fp16 -- tensor_set.h:40-44).
  void configure(int64_t hidden, torch::ScalarType dtype);
  torch::Tensor get_tensor(const std::string& tensor_name);
  void update_tensor_set(int total_seq_len, int to_select_index_len, int to_select_index_position_len,
                         std::vector<int> seq_len_info);
  // int32 device copy of seq_len_info_, refreshed by update_tensor_set
  torch::Tensor seq_len_info_device();
  static Ptr get_instance();            // the current lane's set
  static Ptr get_instance(int lane);

 private:
  void allocate_locked();
  std::mutex mutex_;
  std::map<std::string, torch::Tensor> tensor_map_;
  torch::Tensor seq_len_info_dev_;
  int64_t hidden_ = 768;
  torch::ScalarType dtype_ = torch::kHalf;
  static Ptr instance_[LANES];
  static std::mutex instance_mutex_;
};

}  // namespace layers
}  // namespace sparse_transformers
