// Metadata / stream pipeline: one worker thread per encoder layer builds that layer's
// to-block CSR as soon as a batch is published, stages it in pinned memory, copies it
// (a small kernel on a private stream) and records an event the compute stream later waits on.
//
// Replaces, from the reference: the per-layer counting semaphore
// (layers/semaphore.cpp:8-37), MetaData::update_meta_data / terminate_thread
// (layers/metadata.cpp:6-18), the std::async worker of every attention layer
// (layers/multi_headed_attention.h:102-103, .cpp:16-139) and the condition-variable
// hand-off to the main thread (.cpp:177-188).  Differences by design: a layer's counter
// exists from creation (a signal can never precede registration), every layer has its
// own mutex-protected slot instead of one file-scope flag, the copy is asynchronous on
// its own stream with an event instead of a synchronous copy on the default stream, and
// CSR buffers are double-buffered per layer so a batch can be published while the
// previous one is still executing.
#include <hip/hip_runtime.h>

#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstring>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#include "rt_common.h"

namespace {

struct Slot {                 // one generation of one layer's CSR
  int* host_idx = nullptr;    // pinned (or plain when host-only)
  int* host_pos = nullptr;
  int* dev_idx = nullptr;
  int* dev_pos = nullptr;
  int64_t cap_idx = 0, cap_pos = 0;
  hipEvent_t copied = nullptr;     // recorded on the copy stream after the H2D copies
  bool consumed_pending = false;   // a kernel that reads the slot has been launched (rt_pipeline_release)
};

struct Layer {
  std::mutex m;
  std::condition_variable cv;
  int64_t built_gen = 0;      // last generation whose CSR is queued
  int64_t build_rc = 0;       // status of that build
  std::string build_err;
  Slot slot[2];
  std::thread worker;
  hipStream_t copy_stream = nullptr;
};

}  // namespace

struct rt_pipeline {
  int n_layers = 0, heads = 0, plan_mode = 0, max_pos = 0, policy = 0, device = -1;
  bool async = true;
  // the semaphore: one count per layer, a signal increments every count
  std::mutex sem_m;
  std::condition_variable sem_cv;
  std::vector<int> sem_count;
  std::atomic<bool> terminate{false};
  // published batch geometry
  std::mutex geo_m;
  std::vector<int> seq_blocks;
  int64_t gen = 0;
  // "Every kernel of generation g that reads a slot has finished": per slot parity one event for every stream
  // readers were launched on.  A release marks its stream's entry open; the open entries of the current
  // generation are recorded (each on its own stream) behind the last layer's kernel (rt_pipeline_release of
  // layer n_layers - 1), and whatever was released after that, or in a generation whose last layer never ran,
  // by the next rt_pipeline_publish.  One record per batch and stream instead of one per layer: a record costs
  // the stream about 6 us.  Guarded by geo_m.
  struct Closing { void* stream; hipEvent_t ev; bool open; };
  std::vector<Closing> closing[2];
  std::atomic<bool> check_index{false};     // rt_pipeline_set_index_check
  std::vector<Layer> layers;
  explicit rt_pipeline(int n) : sem_count(n, 0), layers(n) {}
};

namespace {

// Copies a CSR from pinned host memory (mapped into the device's address space) to its device buffers, 16 bytes
// per thread and trip (both buffers come from the allocator, 16-byte aligned): the reads cross the host link, and
// what a small grid gets from it is set by the bytes it keeps in flight.
constexpr int UPLOAD_BLOCKS = 32;
__device__ inline void upload_array(const int* __restrict__ src, int* __restrict__ dst, int64_t n) {
  const int64_t tid = int64_t(blockIdx.x) * blockDim.x + threadIdx.x, threads = int64_t(gridDim.x) * blockDim.x;
  const int64_t quads = n >> 2;
  const int4* src4 = reinterpret_cast<const int4*>(src);
  int4* dst4 = reinterpret_cast<int4*>(dst);
  for (int64_t i = tid; i < quads; i += threads) dst4[i] = src4[i];
  for (int64_t i = 4 * quads + tid; i < n; i += threads) dst[i] = src[i];
}
__global__ __launch_bounds__(256) void upload_csr_kernel(const int* __restrict__ host_idx, int* __restrict__ dev_idx,
                                                         int64_t n_idx, const int* __restrict__ host_pos,
                                                         int* __restrict__ dev_pos, int64_t n_pos) {
  upload_array(host_idx, dev_idx, n_idx);
  upload_array(host_pos, dev_pos, n_pos);
}

int plan_heads_of(const rt_pipeline* p) { return p->plan_mode == RT_PLAN_REFERENCE ? 1 : p->heads; }

// Records the open entries of one slot parity, each behind everything queued on its stream.  Caller holds geo_m.
int close_readers_locked(rt_pipeline* p, int parity) {
  for (rt_pipeline::Closing& c : p->closing[parity]) {
    if (!c.open) continue;
    hipError_t e = hipEventRecord(c.ev, (hipStream_t)c.stream);
    if (e != hipSuccess) return rt::fail(RT_EIO, "hipEventRecord (readers finished): %s", hipGetErrorString(e));
    c.open = false;
  }
  return RT_OK;
}

#define HIP_TRY(expr)                                                              \
  do {                                                                             \
    hipError_t e_ = (expr);                                                        \
    if (e_ != hipSuccess) return rt::fail(RT_EIO, "%s: %s", #expr, hipGetErrorString(e_)); \
  } while (0)

int free_slot(rt_pipeline* p, Slot& s) {
  if (p->device >= 0) {
    if (s.host_idx) (void)hipHostFree(s.host_idx);
    if (s.host_pos) (void)hipHostFree(s.host_pos);
    if (s.dev_idx) (void)hipFree(s.dev_idx);
    if (s.dev_pos) (void)hipFree(s.dev_pos);
  } else {
    delete[] s.host_idx;
    delete[] s.host_pos;
  }
  s.host_idx = s.host_pos = s.dev_idx = s.dev_pos = nullptr;
  s.cap_idx = s.cap_pos = 0;
  return RT_OK;
}

int ensure_capacity(rt_pipeline* p, Slot& s, int64_t need_idx, int64_t need_pos) {
  if (need_idx <= s.cap_idx && need_pos <= s.cap_pos) return RT_OK;
  hipEvent_t copied = s.copied;
  free_slot(p, s);
  s.copied = copied;
  const int64_t ci = need_idx + need_idx / 2 + 64, cp = need_pos + need_pos / 2 + 64;
  if (p->device >= 0) {
    HIP_TRY(hipHostMalloc((void**)&s.host_idx, ci * sizeof(int), hipHostMallocDefault));
    HIP_TRY(hipHostMalloc((void**)&s.host_pos, cp * sizeof(int), hipHostMallocDefault));
    HIP_TRY(hipMalloc((void**)&s.dev_idx, ci * sizeof(int)));
    HIP_TRY(hipMalloc((void**)&s.dev_pos, cp * sizeof(int)));
  } else {
    s.host_idx = new int[ci];
    s.host_pos = new int[cp];
  }
  s.cap_idx = ci;
  s.cap_pos = cp;
  return RT_OK;
}

// Build generation `gen` of layer `l`: CSR -> pinned -> device, event recorded.
int build_layer(rt_pipeline* p, int l, int64_t gen, const std::vector<int>& sb) {
  Layer& L = p->layers[l];
  Slot& s = L.slot[gen & 1];
  const int batch = int(sb.size()) - 1;
  const int ph = plan_heads_of(p);
  int64_t need_idx = 0, need_pos = 0;
  int rc = rt_meta_to_index_size(sb.data(), batch, ph, &need_idx, &need_pos);
  if (rc) return rc;
  bool wait_consumer = false;
  {
    std::lock_guard<std::mutex> lk(L.m);
    wait_consumer = s.consumed_pending;
    s.consumed_pending = false;
  }
  if (p->device >= 0 && wait_consumer) {           // the kernels that read this slot two batches ago
    std::vector<hipEvent_t> readers;
    {
      std::lock_guard<std::mutex> lk(p->geo_m);
      for (const rt_pipeline::Closing& c : p->closing[gen & 1]) readers.push_back(c.ev);
    }
    for (hipEvent_t ev : readers) HIP_TRY(hipEventSynchronize(ev));
  }
  if (p->device >= 0 && s.copied) HIP_TRY(hipEventSynchronize(s.copied));
  rc = ensure_capacity(p, s, need_idx, need_pos);
  if (rc) return rc;
  rc = rt_meta_build_to_index(sb.data(), batch, ph, p->plan_mode, uint32_t(l), p->max_pos, p->policy, nullptr,
                              s.host_idx, s.cap_idx, s.host_pos, s.cap_pos);
  if (rc) return rc;
  if (p->check_index) {
    rc = rt_meta_check_to_index(s.host_idx, s.host_pos, need_idx, sb.data(), batch, ph);
    if (rc) return rc;
  }
  if (p->device >= 0) {
    // A kernel that reads the pinned buffers, not hipMemcpyAsync: a copy engine cannot wait for work on its own, so
    // the runtime makes the calling thread wait for whatever the stream's hardware queue still holds (the 13 streams
    // of a 12-layer pipeline share 4 hardware queues with the compute stream), which stalled workers for a whole
    // step's kernels.  A kernel launch never waits on the host.
    hipLaunchKernelGGL(upload_csr_kernel, dim3(UPLOAD_BLOCKS), dim3(256), 0, L.copy_stream, s.host_idx, s.dev_idx,
                       need_idx, s.host_pos, s.dev_pos, need_pos);
    HIP_TRY(hipGetLastError());
    HIP_TRY(hipEventRecord(s.copied, L.copy_stream));
  }
  return RT_OK;
}

void publish_result(Layer& L, int64_t gen, int rc) {
  std::lock_guard<std::mutex> lk(L.m);
  L.built_gen = gen;
  L.build_rc = rc;
  L.build_err = rc ? rt::error_buffer() : "";
  L.cv.notify_all();
}

void worker_main(rt_pipeline* p, int l) {
  if (p->device >= 0) (void)hipSetDevice(p->device);
  int64_t done = 0;
  for (;;) {
    {   // Semaphore::Wait(layer)
      std::unique_lock<std::mutex> lk(p->sem_m);
      p->sem_cv.wait(lk, [&] { return p->sem_count[l] > 0 || p->terminate; });
      if (p->terminate) break;
      p->sem_count[l] -= 1;
    }
    std::vector<int> sb;
    int64_t gen;
    {
      std::lock_guard<std::mutex> lk(p->geo_m);
      sb = p->seq_blocks;
      gen = p->gen;
    }
    if (gen == done) continue;            // several signals collapsed into one batch
    int rc = build_layer(p, l, gen, sb);
    done = gen;
    publish_result(p->layers[l], gen, rc);
  }
  Layer& L = p->layers[l];
  std::lock_guard<std::mutex> lk(L.m);
  L.cv.notify_all();
}

}  // namespace

extern "C" {

int rt_pipeline_create(rt_pipeline** out, int n_layers, int heads, int plan_mode, int max_pos, int policy,
                       int async, int device) {
  RT_REQUIRE(out, RT_EINVAL, "NULL output");
  RT_REQUIRE(n_layers >= 1 && n_layers <= 4096 && heads >= 1, RT_EINVAL, "bad n_layers=%d or heads=%d", n_layers, heads);
  RT_REQUIRE(plan_mode == RT_PLAN_HF || plan_mode == RT_PLAN_REFERENCE, RT_EINVAL, "plan mode %d cannot be generated by the pipeline", plan_mode);
  rt_pipeline* p = new rt_pipeline(n_layers);
  p->n_layers = n_layers; p->heads = heads; p->plan_mode = plan_mode; p->max_pos = max_pos;
  p->policy = policy; p->async = async != 0; p->device = device;
  if (device >= 0) {
    hipError_t e = hipSetDevice(device);
    if (e != hipSuccess) { delete p; return rt::fail(RT_EIO, "hipSetDevice(%d): %s", device, hipGetErrorString(e)); }
    for (Layer& L : p->layers) {
      bool ok = hipStreamCreateWithFlags(&L.copy_stream, hipStreamNonBlocking) == hipSuccess;
      for (Slot& s : L.slot) {
        ok = ok && hipEventCreateWithFlags(&s.copied, hipEventDisableTiming) == hipSuccess;
      }
      if (!ok) { rt_pipeline_destroy(p); return rt::fail(RT_EIO, "could not create the copy stream / events"); }
    }
  }
  if (p->async)
    for (int l = 0; l < n_layers; ++l) p->layers[l].worker = std::thread(worker_main, p, l);
  *out = p;
  return RT_OK;
}

int rt_pipeline_publish(rt_pipeline* p, const int* seq_blocks, int batch) {
  RT_REQUIRE(p, RT_EINVAL, "NULL pipeline");
  int64_t a, b;
  int rc = rt_meta_to_index_size(seq_blocks, batch, 1, &a, &b);   // validates the geometry
  if (rc) return rc;
  {
    std::lock_guard<std::mutex> lk(p->geo_m);
    // readers of the generation that ends here which no record covers yet (its last layer never ran, or layers
    // were launched again after it): close them now
    if (p->device >= 0) {
      rc = close_readers_locked(p, int(p->gen & 1));
      if (rc) return rc;
    }
    p->seq_blocks.assign(seq_blocks, seq_blocks + batch + 1);
    p->gen += 1;
  }
  {   // Semaphore::Signal(): every layer's count goes up by one
    std::lock_guard<std::mutex> lk(p->sem_m);
    RT_REQUIRE(!p->terminate, RT_ECANCELED, "pipeline was terminated");
    for (int& c : p->sem_count) c += 1;
  }
  p->sem_cv.notify_all();
  return RT_OK;
}

int rt_pipeline_acquire(rt_pipeline* p, int layer, void* stream, const int** to_idx, const int** to_pos,
                        int* plan_heads, double* host_wait_us) {
  RT_REQUIRE(p && to_idx && to_pos, RT_EINVAL, "NULL argument");
  RT_REQUIRE(layer >= 0 && layer < p->n_layers, RT_EINVAL, "layer %d out of range [0, %d)", layer, p->n_layers);
  const auto t0 = std::chrono::steady_clock::now();
  int64_t gen;
  std::vector<int> sb;
  {
    std::lock_guard<std::mutex> lk(p->geo_m);
    gen = p->gen;
    if (!p->async) sb = p->seq_blocks;
  }
  RT_REQUIRE(gen > 0, RT_EINVAL, "no batch has been published");
  Layer& L = p->layers[layer];
  if (p->async) {
    std::unique_lock<std::mutex> lk(L.m);
    L.cv.wait(lk, [&] { return L.built_gen >= gen || p->terminate; });
    if (L.built_gen < gen) return rt::fail(RT_ECANCELED, "pipeline was terminated before layer %d was built", layer);
    if (L.build_rc) return rt::fail(int(L.build_rc), "layer %d: %s", layer, L.build_err.c_str());
  } else if (L.built_gen < gen) {
    int rc = build_layer(p, layer, gen, sb);
    L.built_gen = gen;
    L.build_rc = rc;
    if (rc) return rc;
  }
  Slot& s = L.slot[gen & 1];
  if (p->device >= 0) {
    // The workers run ahead of the layers: the upload has usually finished long before its layer is
    // reached, and then the compute stream needs no barrier (one costs several microseconds of idle GPU).
    const hipError_t done = hipEventQuery(s.copied);
    if (done != hipSuccess) {
      (void)hipGetLastError();                       // hipErrorNotReady is not a failure
      HIP_TRY(hipStreamWaitEvent((hipStream_t)stream, s.copied, 0));
    }
    *to_idx = s.dev_idx;
    *to_pos = s.dev_pos;
  } else {
    *to_idx = s.host_idx;
    *to_pos = s.host_pos;
  }
  if (plan_heads) *plan_heads = plan_heads_of(p);
  if (host_wait_us)
    *host_wait_us = std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count();
  return RT_OK;
}

int rt_pipeline_release(rt_pipeline* p, int layer, void* stream) {
  RT_REQUIRE(p, RT_EINVAL, "NULL pipeline");
  RT_REQUIRE(layer >= 0 && layer < p->n_layers, RT_EINVAL, "layer %d out of range [0, %d)", layer, p->n_layers);
  if (p->device < 0) return RT_OK;
  int64_t gen;
  {
    std::lock_guard<std::mutex> lk(p->geo_m);
    gen = p->gen;
    std::vector<rt_pipeline::Closing>& cl = p->closing[gen & 1];
    size_t k = 0;
    while (k < cl.size() && cl[k].stream != stream) ++k;
    if (k == cl.size()) {
      hipEvent_t ev = nullptr;
      HIP_TRY(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
      cl.push_back(rt_pipeline::Closing{stream, ev, false});
    }
    cl[k].open = true;
    if (layer == p->n_layers - 1) {
      int rc = close_readers_locked(p, int(gen & 1));
      if (rc) return rc;
    }
  }
  Layer& L = p->layers[layer];
  std::lock_guard<std::mutex> lk(L.m);
  L.slot[gen & 1].consumed_pending = true;
  return RT_OK;
}

int rt_pipeline_set_index_check(rt_pipeline* p, int on) {
  RT_REQUIRE(p, RT_EINVAL, "NULL pipeline");
  p->check_index = on != 0;
  return RT_OK;
}

int rt_pipeline_destroy(rt_pipeline* p) {
  if (!p) return RT_OK;
  {   // MetaData::terminate_thread(): flag + signal
    std::lock_guard<std::mutex> lk(p->sem_m);
    p->terminate = true;
  }
  p->sem_cv.notify_all();
  for (Layer& L : p->layers) {
    { std::lock_guard<std::mutex> lk(L.m); L.cv.notify_all(); }
    if (L.worker.joinable()) L.worker.join();
  }
  if (p->device >= 0) {
    (void)hipSetDevice(p->device);
    // readers of the slots may still run: close what is open and wait for every stream's readers
    for (int parity = 0; parity < 2; ++parity) {
      (void)close_readers_locked(p, parity);
      for (const rt_pipeline::Closing& c : p->closing[parity]) (void)hipEventSynchronize(c.ev);
    }
    for (Layer& L : p->layers) {
      if (L.copy_stream) (void)hipStreamSynchronize(L.copy_stream);
      for (Slot& s : L.slot) {
        free_slot(p, s);
        if (s.copied) (void)hipEventDestroy(s.copied);
      }
      if (L.copy_stream) (void)hipStreamDestroy(L.copy_stream);
    }
    for (int parity = 0; parity < 2; ++parity)
      for (const rt_pipeline::Closing& c : p->closing[parity]) (void)hipEventDestroy(c.ev);
  } else {
    for (Layer& L : p->layers)
      for (Slot& s : L.slot) free_slot(p, s);
  }
  delete p;
  return RT_OK;
}

}  // extern "C"
