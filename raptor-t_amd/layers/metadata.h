// Per-batch geometry publish.  Mirrors sparse_transformers::layers::MetaData
// (layers/metadata.h:6-21, layers/metadata.cpp:6-18).
#pragma once
#include <vector>

#include "semaphore.h"
#include "tensor_set.h"

namespace sparse_transformers {
namespace layers {

class MetaData {
 public:
  MetaData() {
    tensor_set = TensorSet::get_instance(0);
    semaphore = Semaphore::get_instance(0);
  }
  // Resizes the scratch set, stores the geometry and wakes every layer's index worker.
  // The two length arguments are kept for signature compatibility; the CSR sizes are
  // derived from seq_len_info (the reference's callers pass them swapped anyway,
  // python/benchmark/end2end.py:81).
  void update_meta_data(int total_seq_len, int to_select_index_len, int to_select_index_position_len,
                        std::vector<int> seq_len_info);
  void terminate_thread();

 private:
  TensorSet::Ptr tensor_set;
  Semaphore::Ptr semaphore;
};

}  // namespace layers
}  // namespace sparse_transformers
