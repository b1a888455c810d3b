#include "semaphore.h"

#include <hip/hip_runtime_api.h>

#include <stdexcept>
#include <string>

namespace sparse_transformers {
namespace layers {

Semaphore::Ptr Semaphore::instance_[2];
std::mutex Semaphore::instance_mutex_;
static_assert(LANES == 2, "one Semaphore per micro-batch lane");

static void check(int rc, const char* what) {
  if (rc != RT_OK) throw std::runtime_error(std::string(what) + ": " + rt_last_error_string());
}

Semaphore::Ptr Semaphore::get_instance() { return get_instance(current_lane()); }

Semaphore::Ptr Semaphore::get_instance(int lane) {
  std::lock_guard<std::mutex> lk(instance_mutex_);
  if (instance_[lane] == nullptr) instance_[lane] = Ptr(new Semaphore());
  return instance_[lane];
}

Semaphore::~Semaphore() { rt_pipeline_destroy(pipeline_); }

bool Semaphore::get_terminate_single() { return terminate_single; }

void Semaphore::register_layer(int layer_idx, int heads, bool async) {
  std::lock_guard<std::mutex> lk(mutex_);
  layer_cond[layer_idx] = heads;
  async_ = async;
  terminate_single = false;      // a newly built layer re-arms a terminated pipeline
}

void Semaphore::set_plan(int plan_mode, int policy, int max_pos) {
  std::lock_guard<std::mutex> lk(mutex_);
  plan_mode_ = plan_mode;
  policy_ = policy;
  max_pos_ = max_pos;
  if (pipeline_) { rt_pipeline_destroy(pipeline_); pipeline_ = nullptr; }
}

void Semaphore::get_plan(int* plan_mode, int* policy, int* max_pos) {
  std::lock_guard<std::mutex> lk(mutex_);
  *plan_mode = plan_mode_;
  *policy = policy_;
  *max_pos = max_pos_;
}

void Semaphore::set_index_check(bool on) {
  std::lock_guard<std::mutex> lk(mutex_);
  index_check_ = on;
  if (pipeline_) check(rt_pipeline_set_index_check(pipeline_, on ? 1 : 0), "rt_pipeline_set_index_check");
}

void Semaphore::ensure_pipeline_locked() {
  if (layer_cond.empty()) throw std::runtime_error("Semaphore: no attention layer has registered");
  const int n_layers = layer_cond.rbegin()->first + 1;
  const int heads = layer_cond.rbegin()->second;
  if (pipeline_ && n_layers == pipeline_layers_ && heads == pipeline_heads_ && async_ == pipeline_async_) return;
  if (pipeline_) { rt_pipeline_destroy(pipeline_); pipeline_ = nullptr; }
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) throw std::runtime_error("Semaphore: no HIP device");
  check(rt_pipeline_create(&pipeline_, n_layers, heads, plan_mode_, max_pos_, policy_, async_ ? 1 : 0, device),
        "rt_pipeline_create");
  check(rt_pipeline_set_index_check(pipeline_, index_check_ ? 1 : 0), "rt_pipeline_set_index_check");
  pipeline_layers_ = n_layers;
  pipeline_heads_ = heads;
  pipeline_async_ = async_;
  terminate_single = false;
}

void Semaphore::Signal(const std::vector<int>& seq_len_info) {
  std::lock_guard<std::mutex> lk(mutex_);
  if (terminate_single) return;
  ensure_pipeline_locked();
  last_batch_ = seq_len_info;
  check(rt_pipeline_publish(pipeline_, seq_len_info.data(), int(seq_len_info.size()) - 1), "rt_pipeline_publish");
}

void Semaphore::Wait(int layer_idx, void* stream, const int** to_idx, const int** to_pos, int* plan_heads,
                     double* wait_us) {
  rt_pipeline* p;
  {
    std::lock_guard<std::mutex> lk(mutex_);
    if (!pipeline_ || layer_idx >= pipeline_layers_) {
      // a layer registered after the last publish: rebuild and publish the batch again
      if (last_batch_.empty()) throw std::runtime_error("attention called before MetaData::update_meta_data");
      ensure_pipeline_locked();
      check(rt_pipeline_publish(pipeline_, last_batch_.data(), int(last_batch_.size()) - 1), "rt_pipeline_publish");
    }
    p = pipeline_;
  }
  check(rt_pipeline_acquire(p, layer_idx, stream, to_idx, to_pos, plan_heads, wait_us), "rt_pipeline_acquire");
}

void Semaphore::Release(int layer_idx, void* stream) {
  std::lock_guard<std::mutex> lk(mutex_);
  if (pipeline_) check(rt_pipeline_release(pipeline_, layer_idx, stream), "rt_pipeline_release");
}

void Semaphore::terminate() {
  std::lock_guard<std::mutex> lk(mutex_);
  terminate_single = true;
  last_batch_.clear();
  layer_cond.clear();
  if (pipeline_) { rt_pipeline_destroy(pipeline_); pipeline_ = nullptr; }
}

}  // namespace layers
}  // namespace sparse_transformers
