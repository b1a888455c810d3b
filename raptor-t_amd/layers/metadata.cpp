#include "metadata.h"

#include <stdexcept>

namespace sparse_transformers {
namespace layers {

void MetaData::update_meta_data(int total_seq_len, int to_select_index_len, int to_select_index_position_len,
                                std::vector<int> seq_len_info) {
  if (seq_len_info.size() < 2 || seq_len_info.front() != 0)
    throw std::invalid_argument("update_meta_data: seq_len_info must be a prefix array starting at 0");
  if (int64_t(seq_len_info.back()) * RT_BLOCK != total_seq_len)
    throw std::invalid_argument("update_meta_data: total_seq_len does not match seq_len_info");
  // the current micro-batch lane's set and pipeline (lane 0 unless the caller selected the other)
  TensorSet::get_instance()->update_tensor_set(total_seq_len, to_select_index_len, to_select_index_position_len, seq_len_info);
  Semaphore::get_instance()->Signal(seq_len_info);
}

void MetaData::terminate_thread() {
  for (int lane = 0; lane < LANES; ++lane) Semaphore::get_instance(lane)->terminate();
}

}  // namespace layers
}  // namespace sparse_transformers
