#include "kernels.h"

#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime_api.h>

#include <atomic>
#include <chrono>
#include <cmath>
#include <mutex>
#include <set>
#include <vector>
#include <stdexcept>

namespace sparse_transformers {
namespace layers {
namespace kernels {

void* current_stream() { return c10::hip::getCurrentHIPStream().stream(); }

int dtype_code(const torch::Tensor& t) {
  switch (t.scalar_type()) {
    case torch::kHalf: return RT_F16;
    case torch::kBFloat16: return RT_BF16;
    case torch::kFloat: return RT_F32;
    default: throw std::invalid_argument("unsupported tensor dtype (fp16, bf16 or fp32 expected)");
  }
}

void check(int rc, const char* what) {
  if (rc != RT_OK) throw std::runtime_error(std::string(what) + ": " + rt_last_error_string());
}

rt_gemm_ctx* shared_gemm_handle() {
  static std::mutex m;
  static rt_gemm_ctx* ctx[LANES] = {};
  const int lane = current_lane();
  std::lock_guard<std::mutex> lk(m);
  if (!ctx[lane]) check(rt_gemm_create(&ctx[lane]), "rt_gemm_create");
  return ctx[lane];
}

static void require_cuda_contiguous(const torch::Tensor& t, const char* name) {
  if (!t.defined() || !t.is_cuda() || !t.is_contiguous())
    throw std::invalid_argument(std::string(name) + " must be a contiguous GPU tensor");
}

// Every pointer below goes to a kernel as it is: a host tensor, another dtype or fewer elements than the
// launch reads would be a GPU memory fault, not an error code.  Checked before anything is launched.
static void require_data(const torch::Tensor& t, const char* name, torch::ScalarType dtype, int64_t min_numel) {
  require_cuda_contiguous(t, name);
  if (t.scalar_type() != dtype)
    throw std::invalid_argument(std::string(name) + " has dtype " + c10::toString(t.scalar_type()) + ", expected " +
                                c10::toString(dtype));
  if (t.numel() < min_numel)
    throw std::invalid_argument(std::string(name) + " holds " + std::to_string(t.numel()) + " elements, the launch needs " +
                                std::to_string(min_numel));
}

static void require_index(const torch::Tensor& t, const char* name, int64_t numel) {
  require_cuda_contiguous(t, name);
  if (t.scalar_type() != torch::kInt32) throw std::invalid_argument(std::string(name) + " must be an int32 tensor");
  if (t.numel() != numel)
    throw std::invalid_argument(std::string(name) + " holds " + std::to_string(t.numel()) + " entries, expected " +
                                std::to_string(numel));
}

// The host's work plan, checked once per tensor pair.  "The pair checked last" is recognised by its storages
// (held through weak references: while one is held, the allocator cannot hand the same storage object to a new
// tensor, and a storage that has died is never taken for a live one), offsets, sizes and versions.  Costs one
// device-to-host copy the first time a plan is seen.
static void require_valid_partition(const torch::Tensor& from_idx, const torch::Tensor& from_pos, int n_wg, int block_num,
                                    int head_num) {
  typedef c10::weak_intrusive_ptr<c10::StorageImpl> WeakStorage;
  struct Key {
    WeakStorage idx, pos;
    int64_t off_idx = 0, off_pos = 0, n_idx = 0, n_pos = 0;
    uint32_t v_idx = 0, v_pos = 0;
    int n_wg = 0, block_num = 0, head_num = 0;
    Key() : idx(WeakStorage(c10::intrusive_ptr<c10::StorageImpl>())), pos(WeakStorage(c10::intrusive_ptr<c10::StorageImpl>())) {}
  };
  static std::mutex m;
  static Key last;
  const c10::StorageImpl* si = from_idx.storage().unsafeGetStorageImpl();
  const c10::StorageImpl* sp = from_pos.storage().unsafeGetStorageImpl();
  {
    std::lock_guard<std::mutex> lk(m);
    if (!last.idx.expired() && !last.pos.expired() && last.idx._unsafe_get_target() == si &&
        last.pos._unsafe_get_target() == sp && last.off_idx == from_idx.storage_offset() &&
        last.off_pos == from_pos.storage_offset() && last.n_idx == from_idx.numel() && last.n_pos == from_pos.numel() &&
        last.v_idx == uint32_t(from_idx._version()) && last.v_pos == uint32_t(from_pos._version()) && last.n_wg == n_wg &&
        last.block_num == block_num && last.head_num == head_num)
      return;
  }
  const torch::Tensor idx_h = from_idx.cpu(), pos_h = from_pos.cpu();
  check(rt_meta_check_partition(pos_h.data_ptr<int>(), idx_h.data_ptr<int>(), n_wg, block_num, head_num),
        "balanced attention: bad work plan");
  std::lock_guard<std::mutex> lk(m);
  last.idx = from_idx.storage().getWeakStorageImpl();
  last.pos = from_pos.storage().getWeakStorageImpl();
  last.off_idx = from_idx.storage_offset();
  last.off_pos = from_pos.storage_offset();
  last.n_idx = from_idx.numel();
  last.n_pos = from_pos.numel();
  last.v_idx = uint32_t(from_idx._version());
  last.v_pos = uint32_t(from_pos._version());
  last.n_wg = n_wg;
  last.block_num = block_num;
  last.head_num = head_num;
}

namespace {
struct Deferred {
  std::mutex m;
  bool active = false;
  struct Rec { std::string key; hipEvent_t a, b; };
  std::vector<Rec> recs;
  std::set<std::string> only;          // empty: every launcher is timed
  int every = 1;                       // of a launcher's calls, one in `every` is bracketed
  std::map<std::string, int64_t> calls;
};
Deferred& deferred() { static Deferred d; return d; }
}  // namespace

void timing_begin(const std::vector<std::string>& only, int every) {
  if (every < 1) throw std::invalid_argument("timing_begin: every must be at least 1");
  Deferred& d = deferred();
  std::lock_guard<std::mutex> lk(d.m);
  d.only = std::set<std::string>(only.begin(), only.end());
  d.every = every;
  d.calls.clear();
  for (auto& r : d.recs) { (void)hipEventDestroy(r.a); (void)hipEventDestroy(r.b); }
  d.recs.clear();
  d.active = true;
}

std::map<std::string, std::pair<double, int64_t>> timing_collect() {
  Deferred& d = deferred();
  std::lock_guard<std::mutex> lk(d.m);
  d.active = false;
  std::map<std::string, std::pair<double, int64_t>> out;
  for (auto& r : d.recs) {
    float ms = 0.f;
    if (hipEventSynchronize(r.b) == hipSuccess && hipEventElapsedTime(&ms, r.a, r.b) == hipSuccess) {
      auto& slot = out[r.key];
      slot.first += double(ms) * 1000.0;
      slot.second += 1;
    } else {
      (void)hipGetLastError();          // a pair that measured nothing must not surface as the next call's error
    }
    (void)hipEventDestroy(r.a);
    (void)hipEventDestroy(r.b);
  }
  d.recs.clear();
  return out;
}

ScopedGpuTimer::ScopedGpuTimer(std::map<std::string, float>& info, const char* key, bool own_dispatch)
    : key_(key), own_dispatch_(own_dispatch) {
  auto it = info.find(key);
  if (it != info.end()) slot_ = &it->second;
  {
    Deferred& d = deferred();
    std::lock_guard<std::mutex> lk(d.m);
    deferred_ = d.active && (d.only.empty() || d.only.count(key) != 0);
    if (deferred_ && d.every > 1) deferred_ = (d.calls[key]++ % d.every) == 0;
  }
  if (!slot_ && !deferred_) return;
  hipEvent_t a, b;
  if (hipEventCreate(&a) != hipSuccess || hipEventCreate(&b) != hipSuccess) { slot_ = nullptr; deferred_ = false; return; }
  start_ = a;
  stop_ = b;
  if (own_dispatch_) (void)rt_time_next_launch(a, b);
  else (void)hipEventRecord(a, static_cast<hipStream_t>(current_stream()));
}

ScopedGpuTimer::~ScopedGpuTimer() {
  if (!slot_ && !deferred_) return;
  hipEvent_t a = static_cast<hipEvent_t>(start_), b = static_cast<hipEvent_t>(stop_);
  if (own_dispatch_) {
    if (rt_time_next_launch(nullptr, nullptr) == 1) {      // no kernel took the pair: nothing was measured
      (void)hipEventDestroy(a);
      (void)hipEventDestroy(b);
      return;
    }
  } else {
    (void)hipEventRecord(b, static_cast<hipStream_t>(current_stream()));
  }
  if (slot_) {
    (void)hipEventSynchronize(b);
    float ms = 0.f;
    if (hipEventElapsedTime(&ms, a, b) == hipSuccess) *slot_ += ms * 1000.0f;
    else (void)hipGetLastError();
  }
  if (deferred_) {
    Deferred& d = deferred();
    std::lock_guard<std::mutex> lk(d.m);
    if (d.active) { d.recs.push_back({key_, a, b}); return; }
  }
  (void)hipEventDestroy(a);
  (void)hipEventDestroy(b);
}

void MatMul(const torch::Tensor& A, bool a_trans, const torch::Tensor& B, bool b_trans, float alpha,
            torch::Tensor& out, float beta, rt_gemm_ctx* handle, const std::string& name) {
  if (a_trans || alpha != 1.0f || beta != 0.0f)
    throw std::invalid_argument(name + ": only out = A . B and out = A . B^T are supported");
  require_cuda_contiguous(A, "A");
  require_cuda_contiguous(B, "B");
  require_cuda_contiguous(out, "out");
  if (A.dim() != 2 || B.dim() != 2) throw std::invalid_argument(name + ": operands must be matrices");
  const int64_t n = b_trans ? B.size(0) : B.size(1);
  if (A.size(1) != (b_trans ? B.size(1) : B.size(0)) || out.numel() != A.size(0) * n ||
      B.scalar_type() != A.scalar_type() || out.scalar_type() != A.scalar_type())
    throw std::invalid_argument(name + ": shape or dtype mismatch");
  static std::map<std::string, float> no_info;
  ScopedGpuTimer timer(no_info, "MatMul");
  if (b_trans)
    check(rt_gemm_bt(handle, A.data_ptr(), B.data_ptr(), nullptr, out.data_ptr(), A.size(0), n, A.size(1),
                     RT_EPILOGUE_NONE, dtype_code(A), current_stream()), name.c_str());
  else
    check(rt_gemm(handle, A.data_ptr(), B.data_ptr(), out.data_ptr(), A.size(0), n, A.size(1), dtype_code(A),
                  current_stream()), name.c_str());
}

void MatMulBias(const torch::Tensor& A, const torch::Tensor& B, bool b_trans, const torch::Tensor& bias, torch::Tensor& out,
                rt_gemm_ctx* handle, const std::string& name) {
  require_cuda_contiguous(A, "A");
  require_cuda_contiguous(B, "B");
  require_cuda_contiguous(bias, "bias");
  require_cuda_contiguous(out, "out");
  if (A.dim() != 2 || B.dim() != 2) throw std::invalid_argument(name + ": operands must be matrices");
  const int64_t n = b_trans ? B.size(0) : B.size(1);
  if (A.size(1) != (b_trans ? B.size(1) : B.size(0)) || out.numel() != A.size(0) * n || bias.numel() != n ||
      bias.scalar_type() != A.scalar_type() || B.scalar_type() != A.scalar_type() || out.scalar_type() != A.scalar_type())
    throw std::invalid_argument(name + ": shape or dtype mismatch");
  static std::map<std::string, float> no_info;
  ScopedGpuTimer timer(no_info, "MatMul");
  if (b_trans)
    check(rt_gemm_bt(handle, A.data_ptr(), B.data_ptr(), bias.data_ptr(), out.data_ptr(), A.size(0), n, A.size(1),
                     RT_EPILOGUE_BIAS, dtype_code(A), current_stream()), name.c_str());
  else
    check(rt_gemm_bias_act(handle, A.data_ptr(), B.data_ptr(), bias.data_ptr(), out.data_ptr(), A.size(0), n, A.size(1),
                           RT_EPILOGUE_BIAS, dtype_code(A), current_stream()), name.c_str());
}

namespace {
std::atomic<bool> g_epilogue_fusion{true};
std::atomic<bool> g_q_from_rows{true};
std::atomic<bool> g_host_plan{false};
constexpr float kQScale = 1.4426950408889634f / 8.0f;      // log2(e) / sqrt(64): the softmax runs in base 2
}
void set_attention_host_plan(bool on) { g_host_plan.store(on); }
bool attention_host_plan() { return g_host_plan.load(); }
void set_attention_q_from_rows(bool on) { g_q_from_rows.store(on); }
bool attention_q_from_rows() { return g_q_from_rows.load(); }
void set_gemm_epilogue_fusion(bool on) { g_epilogue_fusion.store(on); }
bool gemm_epilogue_fusion() { return g_epilogue_fusion.load(); }

void MatMulBiasGelu(const torch::Tensor& A, const torch::Tensor& B, const torch::Tensor& bias, torch::Tensor& out,
                    rt_gemm_ctx* handle, std::map<std::string, float>& info, const std::string& name, bool b_trans) {
  require_cuda_contiguous(A, "A");
  require_cuda_contiguous(B, "B");
  require_cuda_contiguous(bias, "bias");
  require_cuda_contiguous(out, "out");
  if (A.dim() != 2 || B.dim() != 2) throw std::invalid_argument(name + ": operands must be matrices");
  const int64_t n = b_trans ? B.size(0) : B.size(1);
  if (A.size(1) != (b_trans ? B.size(1) : B.size(0)) || out.numel() != A.size(0) * n || bias.numel() != n ||
      bias.scalar_type() != A.scalar_type() || B.scalar_type() != A.scalar_type() || out.scalar_type() != A.scalar_type())
    throw std::invalid_argument(name + ": shape or dtype mismatch");
  ScopedGpuTimer timer(info, "MatMul_bias_gelu");
  if (b_trans)
    check(rt_gemm_bt(handle, A.data_ptr(), B.data_ptr(), bias.data_ptr(), out.data_ptr(), A.size(0), n, A.size(1),
                     RT_EPILOGUE_BIAS_GELU, dtype_code(A), current_stream()), name.c_str());
  else
    check(rt_gemm_bias_act(handle, A.data_ptr(), B.data_ptr(), bias.data_ptr(), out.data_ptr(), A.size(0), n, A.size(1),
                           RT_EPILOGUE_BIAS_GELU, dtype_code(A), current_stream()), name.c_str());
}

double tune_layer_gemms(const std::vector<int64_t>& token_counts, int64_t hidden, int64_t ffn, torch::ScalarType dtype) {
  if (token_counts.empty()) return 0.0;
  if (hidden <= 0 || ffn <= 0) throw std::invalid_argument("tune_layer_gemms: hidden and ffn must be positive");
  int64_t max_m = 0;
  for (int64_t m : token_counts) {
    if (m <= 0) throw std::invalid_argument("tune_layer_gemms: token counts must be positive");
    max_m = std::max(max_m, m);
  }
  const auto t0 = std::chrono::steady_clock::now();
  auto opt = torch::TensorOptions().dtype(dtype).device(torch::kCUDA);
  const int64_t wide = std::max(3 * hidden, ffn);
  // random operands: an all-zero product draws less power and would be timed at other clocks
  torch::Tensor a = torch::randn({max_m, wide}, opt), out = torch::empty({max_m, wide}, opt);
  torch::Tensor w = torch::randn({wide, wide}, opt) * 0.05, bias = torch::zeros({wide}, opt);
  rt_gemm_ctx* handle = shared_gemm_handle();
  void* stream = current_stream();
  const int dt = dtype_code(a);
  for (int64_t m : token_counts) {
    // the shapes and epilogues the layers run with the present switches
    const int64_t qkv_epilogue = gemm_epilogue_fusion() ? RT_EPILOGUE_BIAS : RT_EPILOGUE_NONE;
    const int64_t shapes[4][3] = {{3 * hidden, hidden, qkv_epilogue}, {hidden, hidden, RT_EPILOGUE_NONE},
                                  {ffn, hidden, RT_EPILOGUE_BIAS_GELU}, {hidden, ffn, RT_EPILOGUE_NONE}};
    for (const auto& sh : shapes)
      check(rt_gemm_bt(handle, a.data_ptr(), w.data_ptr(), sh[2] == RT_EPILOGUE_NONE ? nullptr : bias.data_ptr(),
                       out.data_ptr(), m, sh[0], sh[1], int(sh[2]), dt, stream), "tune_layer_gemms");
  }
  check(hipStreamSynchronize(static_cast<hipStream_t>(stream)) == hipSuccess ? 0 : RT_EIO, "tune_layer_gemms");
  return std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
}

void add_bias_and_transpose_kernel(const torch::Tensor& bias, torch::Tensor& input_data, torch::Tensor& q,
                                   torch::Tensor& k, torch::Tensor& v, const torch::Tensor& seq_len_info_tensor,
                                   int batch_size, int head_num, int block_num, int head_size,
                                   std::map<std::string, float>& info, bool kernel_fusion) {
  if (head_size != RT_HEAD_DIM) throw std::invalid_argument("head size must be 64");
  if (batch_size < 1 || head_num < 1 || block_num < batch_size)
    throw std::invalid_argument("add_bias_and_transpose_kernel: bad batch_size / head_num / block_num");
  {
    require_cuda_contiguous(input_data, "qkv");
    const torch::ScalarType dt = input_data.scalar_type();
    const int64_t per_tensor = int64_t(block_num) * 64 * head_num * head_size;
    if (input_data.numel() != 3 * per_tensor)
      throw std::invalid_argument("add_bias_and_transpose_kernel: qkv must be [block_num * 64, 3 * heads * 64]");
    // an undefined bias: the projection added it already (MatMulBias); only with kernel_fusion
    if (bias.defined()) require_data(bias, "qkv bias", dt, 3 * int64_t(head_num) * head_size);
    else if (!kernel_fusion) throw std::invalid_argument("add_bias_and_transpose_kernel: the unfused path needs the bias");
    if (!(kernel_fusion && attention_q_from_rows())) require_data(q, "q", dt, per_tensor);
    require_data(k, "k", dt, per_tensor);
    require_data(v, "v", dt, per_tensor);
    require_index(seq_len_info_tensor, "seq_len_info_tensor", int64_t(batch_size) + 1);
  }
  ScopedGpuTimer timer(info, "add_bias_and_transpose_kernel", kernel_fusion);
  // the attention kernel evaluates the softmax in base 2: fold log2(e) into the Q scale
  const float scale = kQScale;
  if (kernel_fusion) {
    check(rt_qkv_bias_split(input_data.data_ptr(), bias.defined() ? bias.data_ptr() : nullptr,
                            attention_q_from_rows() ? nullptr : q.data_ptr(),
                            k.data_ptr(), v.data_ptr(),
                            seq_len_info_tensor.data_ptr<int>(), batch_size, block_num, head_num, scale,
                            dtype_code(input_data), current_stream()), "rt_qkv_bias_split");
    return;
  }
  // Unfused: library ops, one sequence at a time (the reference's own fallback is a
  // reshape/permute chain, add_bias_and_transpose.cu:219-222), ending in the fragment order
  // of the packed layout: [H][n][f>>2][f&3][l>>5][l&31][e] from [H][n][32*(f>>2)+(l&31)][16*(f&3)+8*(l>>5)+e].
  auto sb = seq_len_info_tensor.cpu();
  const int* s = sb.data_ptr<int>();
  const int64_t dm = int64_t(head_num) * head_size;
  auto x = input_data + bias;
  std::vector<int64_t> slots(64);
  for (int p = 0; p < 64; ++p) {
    const int e = p & 15;
    slots[p] = (p & ~15) | ((e & 3) | ((e & 4) << 1) | ((e & 8) >> 1));
  }
  auto slot_idx = torch::tensor(slots, torch::kLong).to(x.device());
  auto qf = q.view({-1}), kf = k.view({-1}), vf = v.view({-1});
  auto frag = [&](const torch::Tensor& tiles, int64_t n) {       // [H, n, 64(row), 64(col)] -> fragment order
    return tiles.reshape({head_num, n, 2, 32, 4, 2, 8}).permute({0, 1, 2, 4, 5, 3, 6}).contiguous().view({-1});
  };
  for (int b = 0; b < batch_size; ++b) {
    const int64_t n = s[b + 1] - s[b], t0 = int64_t(s[b]) * 64, off = t0 * dm;
    auto seq = x.narrow(0, t0, n * 64);
    auto qs = (seq.narrow(1, 0, dm) * scale).view({n, 64, head_num, head_size}).permute({2, 0, 1, 3});
    auto ks = seq.narrow(1, dm, dm).view({n, 64, head_num, head_size}).permute({2, 0, 1, 3});
    auto vs = seq.narrow(1, 2 * dm, dm).view({n, 64, head_num, head_size}).permute({2, 0, 1, 3});
    qf.narrow(0, off, n * 64 * dm).copy_(frag(qs, n));
    kf.narrow(0, off, n * 64 * dm).copy_(frag(ks, n));
    vf.narrow(0, off, n * 64 * dm).copy_(frag(vs.index_select(2, slot_idx).transpose(2, 3), n));
  }
}

void add_bias_and_layernorm_kernel(torch::Tensor& out, const torch::Tensor& input_data, const torch::Tensor& bias,
                                   int seq_len, int normalized_len, float eps, const torch::Tensor& layernorm_weight,
                                   const torch::Tensor& layernorm_bias, std::map<std::string, float>& info,
                                   bool kernel_fusion) {
  if (seq_len < 0 || normalized_len < 1) throw std::invalid_argument("add_bias_and_layernorm_kernel: bad seq_len / width");
  {
    require_cuda_contiguous(out, "out");
    const torch::ScalarType dt = out.scalar_type();
    const int64_t n = int64_t(seq_len) * normalized_len;
    if (out.numel() != n)
      throw std::invalid_argument("add_bias_and_layernorm_kernel: out holds " + std::to_string(out.numel()) +
                                  " elements, seq_len x width is " + std::to_string(n));
    require_data(input_data, "residual", dt, n);
    if (input_data.numel() != n)
      throw std::invalid_argument("add_bias_and_layernorm_kernel: the residual has other rows than out");
    require_data(bias, "bias", dt, normalized_len);
    require_data(layernorm_weight, "layernorm weight", dt, normalized_len);
    require_data(layernorm_bias, "layernorm bias", dt, normalized_len);
  }
  ScopedGpuTimer timer(info, "add_bias_and_layernorm_kernel", kernel_fusion);
  if (kernel_fusion) {
    check(rt_bias_residual_layernorm(out.data_ptr(), input_data.data_ptr(), bias.data_ptr(),
                                     layernorm_weight.data_ptr(), layernorm_bias.data_ptr(), seq_len, normalized_len,
                                     eps, dtype_code(out), current_stream()), "rt_bias_residual_layernorm");
    return;
  }
  // Unfused: three library launches (add_bias_and_layernorm.cu:276-279)
  out.add_(input_data).add_(bias);
  out.copy_(torch::layer_norm(out, {normalized_len}, layernorm_weight, layernorm_bias, eps));
}

void add_bias_act_kernel(const torch::Tensor& bias, torch::Tensor& out, int total_seq_len, int dim_size,
                         std::map<std::string, float>& info, bool kernel_fusion) {
  if (total_seq_len < 0 || dim_size < 1) throw std::invalid_argument("add_bias_act_kernel: bad total_seq_len / dim_size");
  require_cuda_contiguous(out, "out");
  if (out.numel() != int64_t(total_seq_len) * dim_size)
    throw std::invalid_argument("add_bias_act_kernel: out holds " + std::to_string(out.numel()) +
                                " elements, total_seq_len x dim_size is " + std::to_string(int64_t(total_seq_len) * dim_size));
  require_data(bias, "bias", out.scalar_type(), dim_size);
  ScopedGpuTimer timer(info, "add_bias_act_kernel", kernel_fusion);
  if (kernel_fusion) {
    check(rt_bias_gelu(out.data_ptr(), bias.data_ptr(), total_seq_len, dim_size, dtype_code(out), current_stream()),
          "rt_bias_gelu");
    return;
  }
  // Unfused: add then the tanh-form GELU (the reference's fallback uses the erf form here,
  // an inconsistency with its fused kernel; add_bias_act.cu:123-126)
  out.add_(bias);
  out.copy_(torch::gelu(out, "tanh"));
}

void sparse_attention(const torch::Tensor& q, const torch::Tensor& k, const torch::Tensor& v, torch::Tensor& out,
                      int batch_size, const torch::Tensor& seq_len_info_tensor, const torch::Tensor& from_select_index,
                      const torch::Tensor& from_select_index_position, const int* to_select_index,
                      const int* to_select_index_position, int plan_heads, int block_limit, int block_num,
                      int head_num, std::map<std::string, float>& info, bool balanced, const torch::Tensor& seq_tokens,
                      const torch::Tensor& qkv_rows, const torch::Tensor& qkv_bias) {
  if (batch_size < 1 || head_num < 1 || block_num < batch_size)
    throw std::invalid_argument("sparse_attention: bad batch_size / head_num / block_num");
  if (!to_select_index || !to_select_index_position) throw std::invalid_argument("sparse_attention: no block index");
  const int64_t per_tensor = int64_t(block_num) * 64 * head_num * RT_HEAD_DIM;
  require_cuda_contiguous(out, "attention out");
  if (out.numel() != per_tensor)
    throw std::invalid_argument("sparse_attention: out must hold block_num * 64 rows of heads * 64");
  if (!qkv_rows.defined()) require_data(q, "q", out.scalar_type(), per_tensor);
  require_data(k, "k", out.scalar_type(), per_tensor);
  require_data(v, "v", out.scalar_type(), per_tensor);
  require_index(seq_len_info_tensor, "seq_len_info_tensor", int64_t(batch_size) + 1);
  ScopedGpuTimer timer(info, "attention", true);
  const int* tokens = nullptr;
  if (seq_tokens.defined() && seq_tokens.numel() > 0) {
    if (!seq_tokens.is_cuda() || !seq_tokens.is_contiguous() || seq_tokens.scalar_type() != torch::kInt32 ||
        seq_tokens.numel() != batch_size)
      throw std::invalid_argument("attention_mask must be an int32 GPU tensor with the true token count of each sequence");
    tokens = seq_tokens.data_ptr<int>();
  }
  const int* from_idx = nullptr;
  const int* from_pos = nullptr;
  int n_wg = 0;
  if (balanced) {
    if (from_select_index_position.numel() != int64_t(block_limit) + 1)
      throw std::invalid_argument("balanced attention: the plan has a different number of workgroups than block_limit");
    if (from_select_index.numel() != int64_t(block_num) * head_num)
      throw std::invalid_argument("balanced attention: the plan does not cover every (head, block) unit");
    if (attention_host_plan()) {
      if (block_limit < 1) throw std::invalid_argument("balanced attention: block_limit must be positive");
      require_index(from_select_index, "from_select_index", int64_t(block_num) * head_num);
      require_index(from_select_index_position, "from_select_index_position", int64_t(block_limit) + 1);
      require_valid_partition(from_select_index, from_select_index_position, block_limit, block_num, head_num);
      from_idx = from_select_index.data_ptr<int>();
      from_pos = from_select_index_position.data_ptr<int>();
      n_wg = block_limit;
    }
  }
  if (qkv_rows.defined()) {
    require_cuda_contiguous(qkv_rows, "qkv_rows");
    const bool with_bias = qkv_bias.defined();         // undefined: the rows carry the bias already
    if (with_bias) require_cuda_contiguous(qkv_bias, "qkv_bias");
    if (qkv_rows.dim() != 2 || qkv_rows.size(0) != int64_t(block_num) * 64 || qkv_rows.size(1) != int64_t(head_num) * 192 ||
        qkv_rows.scalar_type() != out.scalar_type() ||
        (with_bias && (qkv_bias.numel() != qkv_rows.size(1) || qkv_bias.scalar_type() != out.scalar_type())))
      throw std::invalid_argument("sparse_attention: qkv_rows must be [tokens, 3 * heads * 64] with a bias of that width");
    check(rt_bs_attention_fwd_qrows(qkv_rows.data_ptr(), with_bias ? qkv_bias.data_ptr() : nullptr, kQScale, k.data_ptr(), v.data_ptr(),
                                    out.data_ptr(), seq_len_info_tensor.data_ptr<int>(), tokens, batch_size, block_num,
                                    head_num, to_select_index, to_select_index_position, plan_heads, from_idx, from_pos,
                                    n_wg, dtype_code(out), current_stream()), "rt_bs_attention_fwd_qrows");
    return;
  }
  check(rt_bs_attention_fwd_masked(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                                   seq_len_info_tensor.data_ptr<int>(), tokens, batch_size, block_num, head_num,
                                   to_select_index, to_select_index_position, plan_heads, from_idx, from_pos, n_wg,
                                   dtype_code(out), current_stream()), "rt_bs_attention_fwd");
}

}  // namespace kernels
}  // namespace layers
}  // namespace sparse_transformers
