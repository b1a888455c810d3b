#include "tensor_set.h"

#include <stdexcept>

namespace sparse_transformers {
namespace layers {

TensorSet::Ptr TensorSet::instance_[LANES];
std::mutex TensorSet::instance_mutex_;

static int g_lane = 0;
int current_lane() { return g_lane; }
void set_current_lane(int lane) {
  if (lane < 0 || lane >= LANES) throw std::invalid_argument("micro-batch lane must be 0 or 1");
  g_lane = lane;
}

TensorSet::TensorSet(int64_t total_seq_len, int64_t to_select_index_len, int64_t to_select_index_position_len) {
  total_seq_len_ = int(total_seq_len);
  to_select_index_len_ = int(to_select_index_len);
  to_select_index_position_len_ = int(to_select_index_position_len);
  std::lock_guard<std::mutex> lk(mutex_);
  allocate_locked();
}

void TensorSet::allocate_locked() {
  auto opt = torch::TensorOptions().dtype(dtype_).device(torch::kCUDA);
  for (const char* name : {"q_out", "k_out", "v_out", "attention_out"})
    tensor_map_[name] = torch::empty({int64_t(total_seq_len_), hidden_}, opt);
  tensor_map_["tmp_qkv_out1"] = torch::empty({int64_t(total_seq_len_), hidden_ * 3}, opt);
}

void TensorSet::configure(int64_t hidden, torch::ScalarType dtype) {
  std::lock_guard<std::mutex> lk(mutex_);
  if (hidden == hidden_ && dtype == dtype_) return;
  hidden_ = hidden;
  dtype_ = dtype;
  allocate_locked();
}

void TensorSet::update_tensor_set(int total_seq_len, int to_select_index_len, int to_select_index_position_len,
                                  std::vector<int> seq_len_info) {
  std::lock_guard<std::mutex> lk(mutex_);
  total_seq_len_ = total_seq_len;
  to_select_index_len_ = to_select_index_len;
  to_select_index_position_len_ = to_select_index_position_len;
  seq_len_info_ = std::move(seq_len_info);
  for (auto& it : tensor_map_) {
    const int64_t width = it.first == "tmp_qkv_out1" ? hidden_ * 3 : hidden_;
    it.second.resize_({int64_t(total_seq_len), width});
  }
  seq_len_info_dev_ = torch::Tensor();
}

torch::Tensor TensorSet::seq_len_info_device() {
  std::lock_guard<std::mutex> lk(mutex_);
  if (!seq_len_info_dev_.defined() && !seq_len_info_.empty())
    seq_len_info_dev_ = torch::tensor(seq_len_info_, torch::kInt32).to(torch::kCUDA);
  return seq_len_info_dev_;
}

torch::Tensor TensorSet::get_tensor(const std::string& tensor_name) {
  std::lock_guard<std::mutex> lk(mutex_);
  auto it = tensor_map_.find(tensor_name);
  if (it == tensor_map_.end()) throw std::invalid_argument("TensorSet: no tensor named '" + tensor_name + "'");
  return it->second;
}

TensorSet::Ptr TensorSet::get_instance() { return get_instance(current_lane()); }

TensorSet::Ptr TensorSet::get_instance(int lane) {
  std::lock_guard<std::mutex> lk(instance_mutex_);
  if (instance_[lane] == nullptr) instance_[lane] = std::make_shared<TensorSet>(4096, 622, 65);   // tensor_set.h:61
  return instance_[lane];
}

}  // namespace layers
}  // namespace sparse_transformers
