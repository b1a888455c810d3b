// Hand-off between MetaData::update_meta_data and the per-layer index workers.
//
// Mirrors sparse_transformers::layers::Semaphore (layers/semaphore.h:10-44,
// layers/semaphore.cpp:8-37): `register_layer`, `Signal`, `Wait`, `terminate_single`.
// The counting, the worker threads and the copy streams live in the C-ABI pipeline
// (rt_pipeline_*); this class owns that pipeline for the process and sizes it from the
// registered layers.  A layer's counter exists from the moment it registers, so a signal
// can never be lost to a late registration.
#pragma once
#include <map>
#include <memory>
#include <mutex>
#include <vector>

#include "../../include/raptor_t_hip.h"
#include "tensor_set.h"

namespace sparse_transformers {
namespace layers {

class Semaphore {
 public:
  typedef std::shared_ptr<Semaphore> Ptr;
  bool terminate_single = false;

  ~Semaphore();
  bool get_terminate_single();
  // Publishes the batch to every registered layer (the reference's Signal() after
  // TensorSet::update_tensor_set).
  void Signal(const std::vector<int>& seq_len_info);
  // Blocks until `layer_idx`'s CSR for the published batch is queued, then makes `stream`
  // wait for the copy; returns device pointers valid until the batch after next.
  void Wait(int layer_idx, void* stream, const int** to_idx, const int** to_pos, int* plan_heads, double* wait_us);
  void Release(int layer_idx, void* stream);
  void register_layer(int layer_idx, int heads, bool async);
  void terminate();
  // plan mode / policy / max positions used for the next pipeline that is created
  void set_plan(int plan_mode, int policy, int max_pos);
  void get_plan(int* plan_mode, int* policy, int* max_pos);
  // debugging aid: every block index the workers build is checked on the host (rt_meta_check_to_index) before its
  // upload; a malformed one makes Wait throw instead of reaching a kernel
  void set_index_check(bool on);
  static Ptr get_instance();            // the current micro-batch lane's (tensor_set.h)
  static Ptr get_instance(int lane);

 private:
  Semaphore() {}
  void ensure_pipeline_locked();
  std::mutex mutex_;
  std::map<int, int> layer_cond;      // registered layers -> heads
  rt_pipeline* pipeline_ = nullptr;
  int pipeline_layers_ = 0, pipeline_heads_ = 0;
  bool pipeline_async_ = true, async_ = true, index_check_ = false;
  int plan_mode_ = RT_PLAN_HF, policy_ = RT_POLICY_REFERENCE_PATCHED, max_pos_ = 4096;
  std::vector<int> last_batch_;
  static Ptr instance_[2];
  static std::mutex instance_mutex_;
};

}  // namespace layers
}  // namespace sparse_transformers
