// Memory-bound kernels of the encoder layer for gfx950 (wave64): fused
// bias+residual+LayerNorm, bias+GELU(tanh form), the QKV bias/scale/head split that
// writes the head-major packed layout the attention kernel reads, and the embedding
// gather + LayerNorm that produces the encoder's packed input.
//
// All of them move 16 bytes per lane per access so that every wave issues full 1 KiB
// requests; statistics and the activation are computed in fp32.
//
// Replaces, from the reference: layers/kernels/add_bias_and_layernorm.cu:191-285,
// layers/kernels/add_bias_act.cu:41-48,86-133, layers/kernels/add_bias_and_transpose.cu:118-233,
// and the PyTorch operators of BertEmbeddings.__call__ (python/modeling_bert.py:47-63).
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <type_traits>

#include "rt_launch.h"

namespace {

// ---- 16-byte vectors of the storage type <-> 8 (or 4) floats --------------------------
template <typename T> struct Vec;            // VEC = elements per 16 bytes
template <> struct Vec<__half> {
  static constexpr int N = 8;
  __device__ static void load(const __half* p, float* f) {
    uint4 r = *reinterpret_cast<const uint4*>(p);
    const __half2* h = reinterpret_cast<const __half2*>(&r);
#pragma unroll
    for (int i = 0; i < 4; ++i) { float2 t = __half22float2(h[i]); f[2 * i] = t.x; f[2 * i + 1] = t.y; }
  }
  __device__ static void store(__half* p, const float* f) {
    uint4 r;
    __half2* h = reinterpret_cast<__half2*>(&r);
#pragma unroll
    for (int i = 0; i < 4; ++i) h[i] = __floats2half2_rn(f[2 * i], f[2 * i + 1]);
    *reinterpret_cast<uint4*>(p) = r;
  }
};
template <> struct Vec<__hip_bfloat16> {
  static constexpr int N = 8;
  __device__ static void load(const __hip_bfloat16* p, float* f) {
    uint4 r = *reinterpret_cast<const uint4*>(p);
    const uint32_t* w = reinterpret_cast<const uint32_t*>(&r);
#pragma unroll
    for (int i = 0; i < 4; ++i) { f[2 * i] = __uint_as_float(w[i] << 16); f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u); }
  }
  // float pair -> packed bf16, round to nearest even: one v_cvt_pk_bf16_f32 on gfx950
  __device__ static uint32_t pack2(float lo, float hi) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    const bf16x2 h = {static_cast<__bf16>(lo), static_cast<__bf16>(hi)};
    return __builtin_bit_cast(uint32_t, h);
  }
  __device__ static void store(__hip_bfloat16* p, const float* f) {
    uint4 r;
    uint32_t* w = reinterpret_cast<uint32_t*>(&r);
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = pack2(f[2 * i], f[2 * i + 1]);
    *reinterpret_cast<uint4*>(p) = r;
  }
};
template <> struct Vec<float> {
  static constexpr int N = 4;
  __device__ static void load(const float* p, float* f) {
    float4 r = *reinterpret_cast<const float4*>(p);
    f[0] = r.x; f[1] = r.y; f[2] = r.z; f[3] = r.w;
  }
  __device__ static void store(float* p, const float* f) {
    *reinterpret_cast<float4*>(p) = make_float4(f[0], f[1], f[2], f[3]);
  }
};

template <int G> __device__ inline float group_sum(float v) {   // sum over G consecutive lanes
#pragma unroll
  for (int o = G / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// ---- bias + residual + LayerNorm ------------------------------------------------------
// One row per group of G lanes (G = 32 or 64); each lane keeps CHUNKS 16-byte chunks of
// the row in registers: hidden = CHUNKS * G * Vec<T>::N.  Two passes over registers.
template <typename T, int CHUNKS, int G>
__global__ __launch_bounds__(256) void bias_residual_layernorm_kernel(
    T* __restrict__ out, const T* __restrict__ residual, const T* __restrict__ bias,
    const T* __restrict__ gamma, const T* __restrict__ beta, int64_t rows, float eps) {
  constexpr int N = Vec<T>::N;
  constexpr int HIDDEN = CHUNKS * G * N;
  const int lane = threadIdx.x % G;
  const int64_t row = int64_t(blockIdx.x) * (256 / G) + threadIdx.x / G;
  if (row >= rows) return;
  T* o = out + row * HIDDEN;
  const T* r = residual + row * HIDDEN;
  float x[CHUNKS][N];
  float sum = 0.f;
  // every request of the row goes out before the first conversion waits for one (left to itself
  // the compiler serialises them for some CHUNKS)
  uint4 ra[CHUNKS], rr[CHUNKS];
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int col = (c * G + lane) * N;
    ra[c] = *reinterpret_cast<const uint4*>(o + col);
    rr[c] = *reinterpret_cast<const uint4*>(r + col);
  }
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int col = (c * G + lane) * N;
    float a[N], b[N], d[N];
    Vec<T>::load(reinterpret_cast<const T*>(&ra[c]), a);
    Vec<T>::load(reinterpret_cast<const T*>(&rr[c]), b);
    Vec<T>::load(bias + col, d);
#pragma unroll
    for (int i = 0; i < N; ++i) { x[c][i] = a[i] + d[i] + b[i]; sum += x[c][i]; }
  }
  const float mean = group_sum<G>(sum) * (1.0f / HIDDEN);
  float sq = 0.f;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c)
#pragma unroll
    for (int i = 0; i < N; ++i) { const float t = x[c][i] - mean; sq += t * t; }
  const float rstd = rsqrtf(group_sum<G>(sq) * (1.0f / HIDDEN) + eps);
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int col = (c * G + lane) * N;
    float g[N], b[N], y[N];
    Vec<T>::load(gamma + col, g);
    Vec<T>::load(beta + col, b);
#pragma unroll
    for (int i = 0; i < N; ++i) y[i] = (x[c][i] - mean) * rstd * g[i] + b[i];
    Vec<T>::store(o + col, y);
  }
}

// Any hidden that is a multiple of the vector width: one wave per row, three sweeps.
template <typename T>
__global__ __launch_bounds__(256) void bias_residual_layernorm_generic_kernel(
    T* __restrict__ out, const T* __restrict__ residual, const T* __restrict__ bias,
    const T* __restrict__ gamma, const T* __restrict__ beta, int64_t rows, int hidden, float eps) {
  constexpr int N = Vec<T>::N;
  const int lane = threadIdx.x % 64;
  const int64_t row = int64_t(blockIdx.x) * 4 + threadIdx.x / 64;
  if (row >= rows) return;
  T* o = out + row * hidden;
  const T* r = residual + row * hidden;
  float sum = 0.f;
  for (int col = lane * N; col < hidden; col += 64 * N) {
    float a[N], b[N], d[N];
    Vec<T>::load(o + col, a); Vec<T>::load(r + col, b); Vec<T>::load(bias + col, d);
#pragma unroll
    for (int i = 0; i < N; ++i) sum += a[i] + d[i] + b[i];
  }
  const float mean = group_sum<64>(sum) / hidden;
  float sq = 0.f;
  for (int col = lane * N; col < hidden; col += 64 * N) {
    float a[N], b[N], d[N];
    Vec<T>::load(o + col, a); Vec<T>::load(r + col, b); Vec<T>::load(bias + col, d);
#pragma unroll
    for (int i = 0; i < N; ++i) { const float t = a[i] + d[i] + b[i] - mean; sq += t * t; }
  }
  const float rstd = rsqrtf(group_sum<64>(sq) / hidden + eps);
  for (int col = lane * N; col < hidden; col += 64 * N) {
    float a[N], b[N], d[N], g[N], be[N], y[N];
    Vec<T>::load(o + col, a); Vec<T>::load(r + col, b); Vec<T>::load(bias + col, d);
    Vec<T>::load(gamma + col, g); Vec<T>::load(beta + col, be);
#pragma unroll
    for (int i = 0; i < N; ++i) y[i] = (a[i] + d[i] + b[i] - mean) * rstd * g[i] + be[i];
    Vec<T>::store(o + col, y);
  }
}

template <typename T, int CHUNKS, int G>
void launch_ln(T* out, const T* res, const T* bias, const T* gamma, const T* beta, int64_t rows, float eps,
               hipStream_t st) {
  const int rows_per_wg = 256 / G;
  const unsigned grid = unsigned((rows + rows_per_wg - 1) / rows_per_wg);
  RT_LAUNCH((bias_residual_layernorm_kernel<T, CHUNKS, G>), dim3(grid), dim3(256), 0, st, out, res, bias,
                     gamma, beta, rows, eps);
}

template <typename T>
int ln_dispatch(void* out, const void* res, const void* bias, const void* gamma, const void* beta, int64_t rows,
                int hidden, float eps, hipStream_t st) {
  T* o = static_cast<T*>(out);
  const T *r = static_cast<const T*>(res), *b = static_cast<const T*>(bias), *g = static_cast<const T*>(gamma),
          *be = static_cast<const T*>(beta);
  constexpr int N = Vec<T>::N;
  const int per32 = 32 * N;
  if (hidden % per32 == 0) {
    switch (hidden / per32) {        // chunks per lane with 32 lanes per row
      case 1: launch_ln<T, 1, 32>(o, r, b, g, be, rows, eps, st); return RT_OK;
      case 2: launch_ln<T, 2, 32>(o, r, b, g, be, rows, eps, st); return RT_OK;
      case 3: launch_ln<T, 3, 32>(o, r, b, g, be, rows, eps, st); return RT_OK;   // 768 (fp16/bf16)
      case 4: launch_ln<T, 4, 32>(o, r, b, g, be, rows, eps, st); return RT_OK;   // 1024
      case 6: launch_ln<T, 3, 64>(o, r, b, g, be, rows, eps, st); return RT_OK;
      case 8: launch_ln<T, 4, 64>(o, r, b, g, be, rows, eps, st); return RT_OK;
      case 12: launch_ln<T, 6, 64>(o, r, b, g, be, rows, eps, st); return RT_OK;
      case 16: launch_ln<T, 8, 64>(o, r, b, g, be, rows, eps, st); return RT_OK;
      default: break;
    }
  }
  const unsigned grid = unsigned((rows + 3) / 4);
  RT_LAUNCH((bias_residual_layernorm_generic_kernel<T>), dim3(grid), dim3(256), 0, st, o, r, b, g, be, rows,
                     hidden, eps);
  return RT_OK;
}

// ---- embedding gather + LayerNorm ---------------------------------------------------------
// out[t] = LN(word[ids[t]] + position[pos_ids[t]] + type[type_ids[t]]) * gamma + beta, written in
// the encoder's dtype.  Tables, gamma and beta are of type TT (fp32 as the reference keeps them,
// or a 16-bit type).  Ids outside a table are clamped into it.
template <typename TT> __device__ inline void load8(const TT* p, float* f) {
  constexpr int N = Vec<TT>::N;
#pragma unroll
  for (int i = 0; i < 8; i += N) Vec<TT>::load(p + i, f + i);
}
template <typename TO> __device__ inline void store8_out(TO* p, const float* f) {
  constexpr int N = Vec<TO>::N;
#pragma unroll
  for (int i = 0; i < 8; i += N) Vec<TO>::store(p + i, f + i);
}
__device__ inline int clamp_id(int v, int n) { return v < 0 ? 0 : (v >= n ? n - 1 : v); }

template <typename TT, typename TO> struct EmbedArgs {
  const int* ids; const int* pos_ids; const int* type_ids;
  const TT* word; const TT* pos; const TT* type; const TT* gamma; const TT* beta;
  TO* out;
  int64_t rows;
  int vocab, max_pos, type_vocab;
  float eps;
};

// One row per group of G lanes; each lane keeps CHUNKS runs of 8 elements: hidden = CHUNKS * G * 8.
template <typename TT, typename TO, int CHUNKS, int G>
__global__ __launch_bounds__(256) void embed_layernorm_kernel(EmbedArgs<TT, TO> a) {
  constexpr int HIDDEN = CHUNKS * G * 8;
  const int lane = threadIdx.x % G;
  const int64_t row = int64_t(blockIdx.x) * (256 / G) + threadIdx.x / G;
  if (row >= a.rows) return;
  const TT* w = a.word + int64_t(clamp_id(a.ids[row], a.vocab)) * HIDDEN;
  const TT* p = a.pos + int64_t(clamp_id(a.pos_ids[row], a.max_pos)) * HIDDEN;
  const TT* t = a.type + int64_t(clamp_id(a.type_ids[row], a.type_vocab)) * HIDDEN;
  float x[CHUNKS][8];
  float sum = 0.f;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int col = (c * G + lane) * 8;
    float u[8], v[8], z[8];
    load8<TT>(w + col, u);
    load8<TT>(p + col, v);
    load8<TT>(t + col, z);
#pragma unroll
    for (int i = 0; i < 8; ++i) { x[c][i] = u[i] + z[i] + v[i]; sum += x[c][i]; }
  }
  const float mean = group_sum<G>(sum) * (1.0f / HIDDEN);
  float sq = 0.f;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c)
#pragma unroll
    for (int i = 0; i < 8; ++i) { const float d = x[c][i] - mean; sq += d * d; }
  const float rstd = rsqrtf(group_sum<G>(sq) * (1.0f / HIDDEN) + a.eps);
  TO* o = a.out + row * HIDDEN;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int col = (c * G + lane) * 8;
    float g[8], b[8], y[8];
    load8<TT>(a.gamma + col, g);
    load8<TT>(a.beta + col, b);
#pragma unroll
    for (int i = 0; i < 8; ++i) y[i] = (x[c][i] - mean) * rstd * g[i] + b[i];
    store8_out<TO>(o + col, y);
  }
}

// Any hidden that is a multiple of 8: one wave per row, three sweeps over the table rows.
template <typename TT, typename TO>
__global__ __launch_bounds__(256) void embed_layernorm_generic_kernel(EmbedArgs<TT, TO> a, int hidden) {
  const int lane = threadIdx.x % 64;
  const int64_t row = int64_t(blockIdx.x) * 4 + threadIdx.x / 64;
  if (row >= a.rows) return;
  const TT* w = a.word + int64_t(clamp_id(a.ids[row], a.vocab)) * hidden;
  const TT* p = a.pos + int64_t(clamp_id(a.pos_ids[row], a.max_pos)) * hidden;
  const TT* t = a.type + int64_t(clamp_id(a.type_ids[row], a.type_vocab)) * hidden;
  auto value = [&](int col, float* x) {
    float u[8], v[8], z[8];
    load8<TT>(w + col, u); load8<TT>(p + col, v); load8<TT>(t + col, z);
#pragma unroll
    for (int i = 0; i < 8; ++i) x[i] = u[i] + z[i] + v[i];
  };
  float sum = 0.f;
  for (int col = lane * 8; col < hidden; col += 512) {
    float x[8];
    value(col, x);
#pragma unroll
    for (int i = 0; i < 8; ++i) sum += x[i];
  }
  const float mean = group_sum<64>(sum) / hidden;
  float sq = 0.f;
  for (int col = lane * 8; col < hidden; col += 512) {
    float x[8];
    value(col, x);
#pragma unroll
    for (int i = 0; i < 8; ++i) { const float d = x[i] - mean; sq += d * d; }
  }
  const float rstd = rsqrtf(group_sum<64>(sq) / hidden + a.eps);
  TO* o = a.out + row * hidden;
  for (int col = lane * 8; col < hidden; col += 512) {
    float x[8], g[8], b[8], y[8];
    value(col, x);
    load8<TT>(a.gamma + col, g);
    load8<TT>(a.beta + col, b);
#pragma unroll
    for (int i = 0; i < 8; ++i) y[i] = (x[i] - mean) * rstd * g[i] + b[i];
    store8_out<TO>(o + col, y);
  }
}

template <typename TT, typename TO, int CHUNKS, int G>
void launch_embed(const EmbedArgs<TT, TO>& a, hipStream_t st) {
  const int rows_per_wg = 256 / G;
  const unsigned grid = unsigned((a.rows + rows_per_wg - 1) / rows_per_wg);
  RT_LAUNCH((embed_layernorm_kernel<TT, TO, CHUNKS, G>), dim3(grid), dim3(256), 0, st, a);
}

template <typename TT, typename TO>
void embed_dispatch(const EmbedArgs<TT, TO>& a, int hidden, hipStream_t st) {
  if (hidden % 256 == 0) {
    switch (hidden / 256) {          // chunks per lane with 32 lanes per row
      case 1: launch_embed<TT, TO, 1, 32>(a, st); return;
      case 2: launch_embed<TT, TO, 2, 32>(a, st); return;
      case 3: launch_embed<TT, TO, 3, 32>(a, st); return;      // 768
      case 4: launch_embed<TT, TO, 4, 32>(a, st); return;      // 1024
      case 6: launch_embed<TT, TO, 3, 64>(a, st); return;
      case 8: launch_embed<TT, TO, 4, 64>(a, st); return;
      default: break;
    }
  }
  const unsigned grid = unsigned((a.rows + 3) / 4);
  RT_LAUNCH((embed_layernorm_generic_kernel<TT, TO>), dim3(grid), dim3(256), 0, st, a, hidden);
}

template <typename TT>
int embed_out_dispatch(const int* ids, const int* pos_ids, const int* type_ids, const void* word, const void* pos,
                       const void* type, const void* gamma, const void* beta, void* out, int64_t rows, int hidden,
                       int vocab, int max_pos, int type_vocab, float eps, int out_dtype, hipStream_t st) {
  auto run = [&](auto* o) {
    typedef typename std::remove_pointer<decltype(o)>::type TO;
    EmbedArgs<TT, TO> a{ids, pos_ids, type_ids, static_cast<const TT*>(word), static_cast<const TT*>(pos),
                        static_cast<const TT*>(type), static_cast<const TT*>(gamma), static_cast<const TT*>(beta),
                        o, rows, vocab, max_pos, type_vocab, eps};
    embed_dispatch<TT, TO>(a, hidden, st);
  };
  if (out_dtype == RT_F16) run(static_cast<__half*>(out));
  else if (out_dtype == RT_BF16) run(static_cast<__hip_bfloat16*>(out));
  else run(static_cast<float*>(out));
  return RT_OK;
}

// ---- bias + GELU (tanh form) ------------------------------------------------------------
// gelu(x) = 0.5 x (1 + tanh(u)), u = c0 (x + c1 x^3)  ==  x / (1 + exp(-2u))
//         = x / (1 + 2^(x (k0 + k1 x^2))),  k0 = -2 c0 log2(e), k1 = k0 c1:
// three multiplies and one fma around the two transcendental instructions.
__device__ inline float gelu_tanh(float x) {
  constexpr float K0 = -2.0f * 0.7978845608028654f * 1.4426950408889634f;
  constexpr float K1 = K0 * 0.044715f;
  const float t = x * fmaf(K1, x * x, K0);
  return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(t));
}

// One workgroup per run of U * 256 vectors (16 KB of a 16-bit tensor), contiguous in memory: thread t
// takes vectors t, t + 256, ... of the run, all U requests issued before any is used.  No grid-stride
// loop: with a capped grid the U requests of a thread lay a power of two apart (16 MiB), which on
// this memory system falls into the same channel every time and costs a fifth of the bandwidth.
template <typename T>
__global__ __launch_bounds__(256) void bias_gelu_kernel(T* __restrict__ out, const T* __restrict__ bias,
                                                        int64_t n_vec, int width_vec) {
  constexpr int N = Vec<T>::N;
  constexpr int U = 4;
  const int64_t v0 = int64_t(blockIdx.x) * (U * 256) + threadIdx.x;
  const uint32_t col0 = uint32_t(v0 % width_vec);
  if (v0 + (U - 1) * 256 < n_vec) {
    float a[U][N];
#pragma unroll
    for (int u = 0; u < U; ++u) Vec<T>::load(out + (v0 + u * 256) * N, a[u]);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      float b[N];
      Vec<T>::load(bias + ((col0 + u * 256) % uint32_t(width_vec)) * N, b);
#pragma unroll
      for (int i = 0; i < N; ++i) a[u][i] = gelu_tanh(a[u][i] + b[i]);
      Vec<T>::store(out + (v0 + u * 256) * N, a[u]);
    }
    return;
  }
  for (int u = 0; u < U; ++u) {                     // the last workgroup: vector by vector
    const int64_t v = v0 + u * 256;
    if (v >= n_vec) break;
    float a[N], b[N];
    Vec<T>::load(out + v * N, a);
    Vec<T>::load(bias + ((col0 + u * 256) % uint32_t(width_vec)) * N, b);
#pragma unroll
    for (int i = 0; i < N; ++i) a[i] = gelu_tanh(a[i] + b[i]);
    Vec<T>::store(out + v * N, a);
  }
}

// ---- QKV bias + scale + head split --------------------------------------------------------
// Workgroup (g, h): global block g, head h.  Its 64x64 tiles (bias and, for Q, the scale applied)
// are written out in MFMA "fragment order": a tile is 8 fragments of 64 lanes x 8 elements,
// element e of lane l of fragment f being
//     Q, K :  tile[32*(f>>2) + (l&31)][16*(f&3) + 8*(l>>5) + e]        (row = token, col = d)
//     V    :  tile[token(16*(f&3) + 8*(l>>5) + e)][32*(f>>2) + (l&31)] (transposed; token()
//             swaps bits 2 and 3 of the slot index: the order in which a 32x32 accumulator
//             hands P back as an MFMA operand)
// so the attention kernel loads each operand with one coalesced 16-byte-per-lane request.
__device__ inline int find_seq(const int* __restrict__ seq_blocks, int batch, int g) {
  int lo = 0, hi = batch;                   // seq_blocks[lo] <= g < seq_blocks[hi]
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (seq_blocks[mid] <= g) lo = mid; else hi = mid;
  }
  return lo;
}

__device__ inline int slot_token(int p) {   // token held by slot p of a transposed V tile
  const int e = p & 15;
  return (p & ~15) | ((e & 3) | ((e & 4) << 1) | ((e & 8) >> 1));
}

template <typename T> __device__ inline void store8(T* p, const float* x) {
  constexpr int N = Vec<T>::N;
#pragma unroll
  for (int i = 0; i < 8; i += N) Vec<T>::store(p + i, x + i);
}

template <typename T, bool WITH_Q>
__global__ __launch_bounds__(256) void qkv_bias_split_kernel(const T* __restrict__ qkv, const T* __restrict__ bias,
                                                             T* __restrict__ q, T* __restrict__ k,
                                                             T* __restrict__ vt, const int* __restrict__ seq_blocks,
                                                             int batch, int heads, float q_scale) {
  constexpr int N = Vec<T>::N;              // elements per 16 bytes
  constexpr int CPR = 64 / N;               // 16-byte chunks per 64-wide row
  constexpr int ITERS = 64 * CPR / 256;     // chunks per thread and matrix
  constexpr int M0 = WITH_Q ? 0 : 1;        // without Q (left to the attention kernel) only K and V are read
  // Only V needs a transpose.  A Q / K fragment entry (8 consecutive d of one token) is a run of the
  // source row already: those two matrices are copied run by run to their permuted places.
  __shared__ float vtile[64][65];
  // heads vary fastest over the grid: workgroups running together read neighbouring 128-byte
  // pieces of the same token rows.  The head is rotated by the block index so that, with a
  // power-of-two head count, one XCD (workgroups go to the 8 XCDs round-robin) does not always get
  // the same heads' columns.
  const int g = blockIdx.x / heads, h = (blockIdx.x % heads + g) % heads;
  const int dm = heads * 64;
  const T* src = qkv + int64_t(g) * 64 * (3 * dm) + h * 64;
  // every load of the thread is issued before anything waits for one: the kernel lives on bytes in flight.
  // The projection's rows are read once and never again by this kernel: non-temporal loads keep them from
  // pushing the K / V^T tiles written below out of the caches before the attention kernel, which runs next,
  // reads them (measured in the step's kernel order: this kernel 46 -> 39 us, the attention kernel after it
  // 119 -> 105 us).
  typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
  uint4 raw[ITERS][3];
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int c = threadIdx.x + it * 256, row = c / CPR, col = (c % CPR) * N;
#pragma unroll
    for (int m = M0; m < 3; ++m) {
      const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(src + int64_t(row) * 3 * dm + m * dm + col));
      raw[it][m] = make_uint4(v.x, v.y, v.z, v.w);
    }
  }
  const int s = find_seq(seq_blocks, batch, g);
  const int g0 = seq_blocks[s], n = seq_blocks[s + 1] - g0;
  const int64_t base = (int64_t(g0) * heads + int64_t(h) * n + (g - g0)) * 4096;
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int c = threadIdx.x + it * 256, row = c / CPR, col = (c % CPR) * N;
    float x[3][N], b[3][N];
#pragma unroll
    for (int m = M0; m < 3; ++m) {
      Vec<T>::load(reinterpret_cast<const T*>(&raw[it][m]), x[m]);
      if (bias) {                               // NULL: the projection added it already (adding zero changes nothing)
        Vec<T>::load(bias + m * dm + h * 64 + col, b[m]);
      } else {
#pragma unroll
        for (int i = 0; i < N; ++i) b[m][i] = 0.f;
      }
    }
    // run `col8` (8 elements) of token `row` is lane (row & 31) + 32 * (col8 & 1) of fragment
    // 4 * (row >> 5) + (col8 >> 1); a 16-byte chunk of fp32 is half such a run
    const int col8 = col >> 3;
    const int dst = ((4 * (row >> 5) + (col8 >> 1)) * 64 + (row & 31) + 32 * (col8 & 1)) * 8 + (col & 7);
#pragma unroll
    for (int i = 0; i < N; ++i) {
      if (WITH_Q) {
        // The product is pinned in fp32 before it is rounded to the output type: left alone the
        // compiler may fuse multiply and rounding into one instruction that rounds once, and
        // the attention kernel's own copy of this arithmetic must give the same bits.
        float y = (x[0][i] + b[0][i]) * q_scale;
        asm volatile("" : "+v"(y));
        x[0][i] = y;
      }
      x[1][i] = x[1][i] + b[1][i];
      vtile[row][col + i] = x[2][i] + b[2][i];
    }
    if (WITH_Q) Vec<T>::store(q + base + dst, x[0]);
    Vec<T>::store(k + base + dst, x[1]);
  }
  __syncthreads();
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    const int c = threadIdx.x + it * 256;
    const int f = c >> 6, l = c & 63;
    const int r32 = 32 * (f >> 2) + (l & 31), c8 = 16 * (f & 3) + 8 * (l >> 5);
    float x[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = vtile[slot_token(c8 + e)][r32];
    store8<T>(vt + base + c * 8, x);
  }
}

// Inverse of the fragment order for inspection: packed tiles -> token-major [T, H*64].
// transposed = 0 for Q / K tiles, 1 for V tiles.
template <typename T>
__global__ __launch_bounds__(256) void unpack_head_tiles_kernel(const T* __restrict__ packed, T* __restrict__ dst,
                                                                const int* __restrict__ seq_blocks, int batch,
                                                                int heads, int transposed) {
  const int g = blockIdx.x, h = blockIdx.y;
  const int s = find_seq(seq_blocks, batch, g);
  const int g0 = seq_blocks[s], n = seq_blocks[s + 1] - g0;
  const int64_t base = (int64_t(g0) * heads + int64_t(h) * n + (g - g0)) * 4096;
  const int dm = heads * 64;
  for (int x = threadIdx.x; x < 4096; x += 256) {
    const int c = x >> 3, e = x & 7, f = c >> 6, l = c & 63;
    const int r32 = 32 * (f >> 2) + (l & 31), c8 = 16 * (f & 3) + 8 * (l >> 5) + e;
    const int token = transposed ? slot_token(c8) : r32;
    const int d = transposed ? r32 : c8;
    dst[(int64_t(g) * 64 + token) * dm + h * 64 + d] = packed[base + x];
  }
}

// ---- sequence pooling + pooler head ---------------------------------------------------
// One workgroup per (sequence, 8 chunks of 16 bytes): 32 token lanes stride over the sequence's
// tokens, fp32 sum / max per column, combined through LDS.
template <typename T>
__global__ __launch_bounds__(256) void sequence_pool_kernel(const T* __restrict__ hidden,
                                                            const int* __restrict__ seq_blocks,
                                                            const int* __restrict__ seq_tokens, int width, int mode,
                                                            T* __restrict__ out) {
  constexpr int N = Vec<T>::N;
  __shared__ float red[32][8 * N + 1];
  const int s = blockIdx.x;
  const int cw = threadIdx.x & 7, tl = threadIdx.x >> 3;
  const int col = (blockIdx.y * 8 + cw) * N;
  const int64_t t0 = int64_t(seq_blocks[s]) * 64;
  int count = (seq_blocks[s + 1] - seq_blocks[s]) * 64;
  if (seq_tokens) count = min(max(seq_tokens[s], 1), count);
  int first = 0, last = count;
  if (mode == RT_POOL_FIRST) last = 1;
  else if (mode == RT_POOL_LAST) first = count - 1;
  float acc[N];
#pragma unroll
  for (int i = 0; i < N; ++i) acc[i] = mode == RT_POOL_MAX ? -INFINITY : 0.f;
  if (col < width)
    for (int t = first + tl; t < last; t += 32) {
      float x[N];
      Vec<T>::load(hidden + (t0 + t) * width + col, x);
#pragma unroll
      for (int i = 0; i < N; ++i) acc[i] = mode == RT_POOL_MAX ? fmaxf(acc[i], x[i]) : acc[i] + x[i];
    }
#pragma unroll
  for (int i = 0; i < N; ++i) red[tl][cw * N + i] = acc[i];
  __syncthreads();
  if (threadIdx.x < 8 * N) {
    const int c = blockIdx.y * 8 * N + threadIdx.x;
    float v = red[0][threadIdx.x];
    for (int r = 1; r < 32; ++r) v = mode == RT_POOL_MAX ? fmaxf(v, red[r][threadIdx.x]) : v + red[r][threadIdx.x];
    if (mode == RT_POOL_MEAN) v /= float(last - first);
    if (c < width) out[int64_t(s) * width + c] = static_cast<T>(v);
  }
}

// out[b, j] = tanh(bias[j] + sum_i x[b, i] * w[j, i]), weights as [out, in]: one wave per output column.
template <typename T>
__global__ __launch_bounds__(256) void pooler_dense_tanh_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                                const T* __restrict__ bias, T* __restrict__ out,
                                                                int batch, int d_in, int d_out) {
  constexpr int N = Vec<T>::N;
  const int lane = threadIdx.x & 63, j = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (j >= d_out) return;
  const T* wr = w + int64_t(j) * d_in;
  const float bj = float(bias[j]);
  for (int b = 0; b < batch; ++b) {
    const T* xr = x + int64_t(b) * d_in;
    float acc = 0.f;
    for (int c = lane * N; c < d_in; c += 64 * N) {
      float a[N], v[N];
      Vec<T>::load(wr + c, a);
      Vec<T>::load(xr + c, v);
#pragma unroll
      for (int i = 0; i < N; ++i) acc = fmaf(a[i], v[i], acc);
    }
    acc = group_sum<64>(acc);
    if (lane == 0) out[int64_t(b) * d_out + j] = static_cast<T>(tanhf(acc + bj));
  }
}

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return rt::fail(RT_EIO, "%s launch failed: %s", what, hipGetErrorString(e));
  return RT_OK;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace

extern "C" {

int rt_bias_residual_layernorm(void* out, const void* residual, const void* bias, const void* gamma,
                               const void* beta, int64_t rows, int hidden, float eps, int dtype, void* stream) {
  RT_REQUIRE(out && residual && bias && gamma && beta, RT_EINVAL, "NULL pointer");
  RT_REQUIRE(rows >= 0 && rows < (int64_t(1) << 31), RT_EINVAL, "rows=%lld out of range", (long long)rows);
  const int n = dtype == RT_F32 ? 4 : 8;
  RT_REQUIRE(dtype == RT_F16 || dtype == RT_BF16 || dtype == RT_F32, RT_EINVAL, "unknown dtype %d", dtype);
  RT_REQUIRE(hidden > 0 && hidden % n == 0, RT_EINVAL, "hidden=%d must be a positive multiple of %d", hidden, n);
  RT_REQUIRE(aligned16(out) && aligned16(residual) && aligned16(bias) && aligned16(gamma) && aligned16(beta),
             RT_EINVAL, "pointers must be 16-byte aligned");
  if (rows == 0) return RT_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == RT_F16) ln_dispatch<__half>(out, residual, bias, gamma, beta, rows, hidden, eps, st);
  else if (dtype == RT_BF16) ln_dispatch<__hip_bfloat16>(out, residual, bias, gamma, beta, rows, hidden, eps, st);
  else ln_dispatch<float>(out, residual, bias, gamma, beta, rows, hidden, eps, st);
  return check_launch("bias_residual_layernorm");
}

int rt_bias_gelu(void* out, const void* bias, int64_t rows, int width, int dtype, void* stream) {
  RT_REQUIRE(out && bias, RT_EINVAL, "NULL pointer");
  RT_REQUIRE(dtype == RT_F16 || dtype == RT_BF16 || dtype == RT_F32, RT_EINVAL, "unknown dtype %d", dtype);
  const int n = dtype == RT_F32 ? 4 : 8;
  RT_REQUIRE(rows >= 0 && width > 0 && width % n == 0, RT_EINVAL, "rows=%lld width=%d: width must be a positive multiple of %d",
             (long long)rows, width, n);
  RT_REQUIRE(aligned16(out) && aligned16(bias), RT_EINVAL, "pointers must be 16-byte aligned");
  if (rows == 0) return RT_OK;
  const int64_t n_vec = rows * (width / n);
  const int64_t want = (n_vec + 256 * 4 - 1) / (256 * 4);     // four vectors per thread
  RT_REQUIRE(want < (int64_t(1) << 31), RT_EINVAL, "rows=%lld x width=%d is too large for one launch", (long long)rows, width);
  const unsigned grid = unsigned(want);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == RT_F16)
    RT_LAUNCH(bias_gelu_kernel<__half>, dim3(grid), dim3(256), 0, st, (__half*)out, (const __half*)bias, n_vec, width / n);
  else if (dtype == RT_BF16)
    RT_LAUNCH(bias_gelu_kernel<__hip_bfloat16>, dim3(grid), dim3(256), 0, st, (__hip_bfloat16*)out, (const __hip_bfloat16*)bias, n_vec, width / n);
  else
    RT_LAUNCH(bias_gelu_kernel<float>, dim3(grid), dim3(256), 0, st, (float*)out, (const float*)bias, n_vec, width / n);
  return check_launch("bias_gelu");
}

int rt_qkv_bias_split(const void* qkv, const void* bias, void* q, void* k, void* vt, const int* seq_blocks_dev,
                      int batch, int total_blocks, int heads, float q_scale, int dtype, void* stream) {
  RT_REQUIRE(qkv && k && vt && seq_blocks_dev, RT_EINVAL, "NULL pointer");       // q may be NULL: not written; bias: none added
  RT_REQUIRE(batch >= 1 && total_blocks >= batch && heads >= 1 && int64_t(total_blocks) * heads < (int64_t(1) << 31),
             RT_EINVAL, "bad geometry: batch=%d total_blocks=%d heads=%d", batch, total_blocks, heads);
  RT_REQUIRE(dtype == RT_F16 || dtype == RT_BF16 || dtype == RT_F32, RT_EINVAL, "unknown dtype %d", dtype);
  RT_REQUIRE(aligned16(qkv) && aligned16(bias) && aligned16(q) && aligned16(k) && aligned16(vt), RT_EINVAL,
             "pointers must be 16-byte aligned");
  hipStream_t st = static_cast<hipStream_t>(stream);
  dim3 grid(unsigned(heads) * unsigned(total_blocks));
  auto launch = [&](auto tag) {
    typedef decltype(tag) T;
    if (q)
      RT_LAUNCH((qkv_bias_split_kernel<T, true>), grid, dim3(256), 0, st, (const T*)qkv, (const T*)bias, (T*)q,
                         (T*)k, (T*)vt, seq_blocks_dev, batch, heads, q_scale);
    else
      RT_LAUNCH((qkv_bias_split_kernel<T, false>), grid, dim3(256), 0, st, (const T*)qkv, (const T*)bias,
                         (T*)nullptr, (T*)k, (T*)vt, seq_blocks_dev, batch, heads, q_scale);
  };
  if (dtype == RT_F16) launch(__half());
  else if (dtype == RT_BF16) launch(__hip_bfloat16());
  else launch(float());
  return check_launch("qkv_bias_split");
}

int rt_unpack_head_tiles(const void* packed, void* dst, const int* seq_blocks_dev, int batch, int total_blocks,
                         int heads, int transposed, int dtype, void* stream) {
  RT_REQUIRE(packed && dst && seq_blocks_dev, RT_EINVAL, "NULL pointer");
  RT_REQUIRE(batch >= 1 && total_blocks >= batch && heads >= 1 && heads <= 65535, RT_EINVAL,
             "bad geometry: batch=%d total_blocks=%d heads=%d", batch, total_blocks, heads);
  hipStream_t st = static_cast<hipStream_t>(stream);
  dim3 grid(total_blocks, heads);
  const int tr = transposed ? 1 : 0;
  if (dtype == RT_F16)
    RT_LAUNCH(unpack_head_tiles_kernel<__half>, grid, dim3(256), 0, st, (const __half*)packed, (__half*)dst, seq_blocks_dev, batch, heads, tr);
  else if (dtype == RT_BF16)
    RT_LAUNCH(unpack_head_tiles_kernel<__hip_bfloat16>, grid, dim3(256), 0, st, (const __hip_bfloat16*)packed, (__hip_bfloat16*)dst, seq_blocks_dev, batch, heads, tr);
  else if (dtype == RT_F32)
    RT_LAUNCH(unpack_head_tiles_kernel<float>, grid, dim3(256), 0, st, (const float*)packed, (float*)dst, seq_blocks_dev, batch, heads, tr);
  else
    return rt::fail(RT_EINVAL, "unknown dtype %d", dtype);
  return check_launch("unpack_head_tiles");
}

int rt_embed_layernorm(const int* input_ids, const int* position_ids, const int* token_type_ids, const void* word,
                       const void* position, const void* token_type, const void* gamma, const void* beta, void* out,
                       int64_t rows, int hidden, int vocab, int max_pos, int type_vocab, float eps, int table_dtype,
                       int out_dtype, void* stream) {
  RT_REQUIRE(rows >= 0 && rows < (int64_t(1) << 31), RT_EINVAL, "rows=%lld out of range", (long long)rows);
  RT_REQUIRE(word && position && token_type && gamma && beta, RT_EINVAL, "NULL table pointer");
  RT_REQUIRE(rows == 0 || (input_ids && position_ids && token_type_ids && out), RT_EINVAL, "NULL id or output pointer");
  RT_REQUIRE(hidden > 0 && hidden % 8 == 0, RT_EINVAL, "hidden=%d must be a positive multiple of 8", hidden);
  RT_REQUIRE(vocab > 0 && max_pos > 0 && type_vocab > 0, RT_EINVAL, "empty table: vocab=%d max_pos=%d type_vocab=%d", vocab,
             max_pos, type_vocab);
  RT_REQUIRE(table_dtype == RT_F16 || table_dtype == RT_BF16 || table_dtype == RT_F32, RT_EINVAL, "unknown table dtype %d",
             table_dtype);
  RT_REQUIRE(out_dtype == RT_F16 || out_dtype == RT_BF16 || out_dtype == RT_F32, RT_EINVAL, "unknown output dtype %d",
             out_dtype);
  RT_REQUIRE(aligned16(word) && aligned16(position) && aligned16(token_type) && aligned16(gamma) && aligned16(beta) &&
                 aligned16(out), RT_EINVAL, "tables, gamma, beta and out must be 16-byte aligned");
  if (rows == 0) return RT_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (table_dtype == RT_F32)
    embed_out_dispatch<float>(input_ids, position_ids, token_type_ids, word, position, token_type, gamma, beta, out, rows,
                              hidden, vocab, max_pos, type_vocab, eps, out_dtype, st);
  else if (table_dtype == RT_F16)
    embed_out_dispatch<__half>(input_ids, position_ids, token_type_ids, word, position, token_type, gamma, beta, out, rows,
                               hidden, vocab, max_pos, type_vocab, eps, out_dtype, st);
  else
    embed_out_dispatch<__hip_bfloat16>(input_ids, position_ids, token_type_ids, word, position, token_type, gamma, beta,
                                       out, rows, hidden, vocab, max_pos, type_vocab, eps, out_dtype, st);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return rt::fail(RT_EIO, "embed_layernorm launch failed: %s", hipGetErrorString(e));
  return RT_OK;
}

int rt_sequence_pool(const void* hidden, const int* seq_blocks_dev, const int* seq_tokens_dev, int batch, int width,
                     int mode, void* out, int dtype, void* stream) {
  RT_REQUIRE(hidden && seq_blocks_dev && out, RT_EINVAL, "NULL pointer");
  RT_REQUIRE(batch >= 1 && batch <= 65535, RT_EINVAL, "batch=%d out of range [1, 65535]", batch);
  RT_REQUIRE(width > 0 && width % 8 == 0, RT_EINVAL, "width=%d must be a positive multiple of 8", width);
  RT_REQUIRE(mode == RT_POOL_FIRST || mode == RT_POOL_LAST || mode == RT_POOL_MEAN || mode == RT_POOL_MAX, RT_EINVAL,
             "unknown pooling mode %d", mode);
  RT_REQUIRE(aligned16(hidden), RT_EINVAL, "hidden must be 16-byte aligned");
  hipStream_t st = static_cast<hipStream_t>(stream);
  auto launch = [&](auto tag) {
    typedef decltype(tag) T;
    const int per_wg = 8 * Vec<T>::N;
    RT_LAUNCH(sequence_pool_kernel<T>, dim3(batch, (width + per_wg - 1) / per_wg), dim3(256), 0, st,
                       (const T*)hidden, seq_blocks_dev, seq_tokens_dev, width, mode, (T*)out);
  };
  if (dtype == RT_F16) launch(__half());
  else if (dtype == RT_BF16) launch(__hip_bfloat16());
  else if (dtype == RT_F32) launch(float());
  else return rt::fail(RT_EINVAL, "unknown dtype %d", dtype);
  return check_launch("sequence_pool");
}

int rt_pooler_dense_tanh(const void* pooled, const void* weight_t, const void* bias, void* out, int batch, int d_in,
                         int d_out, int dtype, void* stream) {
  RT_REQUIRE(pooled && weight_t && bias && out, RT_EINVAL, "NULL pointer");
  RT_REQUIRE(batch >= 1 && d_out >= 1, RT_EINVAL, "bad shape: batch=%d d_out=%d", batch, d_out);
  RT_REQUIRE(d_in > 0 && d_in % 8 == 0, RT_EINVAL, "d_in=%d must be a positive multiple of 8", d_in);
  RT_REQUIRE(aligned16(pooled) && aligned16(weight_t), RT_EINVAL, "pooled and weight_t must be 16-byte aligned");
  hipStream_t st = static_cast<hipStream_t>(stream);
  auto launch = [&](auto tag) {
    typedef decltype(tag) T;
    RT_LAUNCH(pooler_dense_tanh_kernel<T>, dim3((d_out + 3) / 4), dim3(256), 0, st, (const T*)pooled,
                       (const T*)weight_t, (const T*)bias, (T*)out, batch, d_in, d_out);
  };
  if (dtype == RT_F16) launch(__half());
  else if (dtype == RT_BF16) launch(__hip_bfloat16());
  else if (dtype == RT_F32) launch(float());
  else return rt::fail(RT_EINVAL, "unknown dtype %d", dtype);
  return check_launch("pooler_dense_tanh");
}

}  // extern "C"
