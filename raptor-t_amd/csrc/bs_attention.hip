// Block-sparse (BigBird-pattern) attention forward for gfx950, d = 64, 64-token blocks.
//
// Work unit = (sequence, head, from-block): 64 queries against the key blocks its CSR
// row lists (7/8 blocks for sparse rows, all n blocks for the two global rows).
//
// Workgroup = 4 waves.  Wave w owns 32 queries (w & 1) and every second listed key block
// (w >> 1): the two waves that share a key block share its K and V tiles in LDS, the two
// key-block streams keep independent online-softmax states that are merged through LDS
// once per unit.  Splitting the key list two ways halves the serial depth of the dense
// rows and needs no exchange inside the loop.
//
// MFMA formulation (v_mfma_f32_32x32x16_{f16,bf16}, fp32 accumulators):
//   S^T[key][query] = K[key][:] . Q[query][:]      A = K tile from LDS, B = Q (registers)
//   O^T[d][query]  += V^T[d][key] . P^T[key][query] A = V^T tile from LDS, B = P (registers)
// Both products put the query on the accumulator's column (lane & 31), so row max, row
// sum, the rescale factor and the final 1/sum are per-lane scalars, and the accumulator
// registers of S^T are, after exp, exactly the B operand of the second product: P never
// goes through LDS.  The V tile is stored transposed with its 64 key slots in accumulator
// order by the QKV split kernel.
//
// LDS rows are padded from 128 to 144 bytes so that the 16-byte operand reads of 16
// consecutive rows fall in distinct banks.
//
// Replaces, from the reference: layers/kernels/sparse_attention.cu:2953-3190 (balanced,
// persistent workgroups over the LPT plan), :2111-2403 (one workgroup per unit) and the
// dispatcher :3192-3228.
#include <hip/hip_runtime.h>

#include "rt_common.h"

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

template <typename T> struct Mma;
template <> struct Mma<_Float16> {
  typedef f16x8 v8;
  typedef f16x4 v4;
  __device__ static f32x16 run(v8 a, v8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
};
template <> struct Mma<__bf16> {
  typedef bf16x8 v8;
  typedef bf16x4 v4;
  __device__ static f32x16 run(v8 a, v8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
};

constexpr int ROW = 72;                 // padded LDS row, in elements (144 bytes)
constexpr int TILE = 64 * ROW;          // one K or V^T tile in LDS
constexpr float LOG2E = 1.4426950408889634f;

__device__ inline int find_seq_by_unit(const int* __restrict__ seq_blocks, int batch, int heads, int unit) {
  int lo = 0, hi = batch;               // seq_blocks[lo]*heads <= unit < seq_blocks[hi]*heads
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (seq_blocks[mid] * heads <= unit) lo = mid; else hi = mid;
  }
  return lo;
}

template <typename T>
__global__ __launch_bounds__(256, 2) void bs_attention_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ vt, T* __restrict__ out,
    const int* __restrict__ seq_blocks, int batch, int heads, int nb_total, const int* __restrict__ to_idx,
    const int* __restrict__ to_pos, int plan_heads, const int* __restrict__ from_idx,
    const int* __restrict__ from_pos) {
  typedef typename Mma<T>::v8 v8;
  typedef typename Mma<T>::v4 v4;
  __shared__ __attribute__((aligned(16))) T smem[2 * 2 * TILE];     // [key stream][K | V^T]

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int qh = wave & 1, ks = wave >> 1;           // query half, key stream
  const int l32 = lane & 31, hi = lane >> 5;
  const int ptid = tid & 127;                        // thread index inside the key stream's pair of waves
  T* lds_k = smem + ks * 2 * TILE;
  T* lds_v = lds_k + TILE;

  int u_begin, u_end;
  if (from_pos) { u_begin = from_pos[blockIdx.x]; u_end = from_pos[blockIdx.x + 1]; }
  else { u_begin = blockIdx.x; u_end = u_begin + 1; }
  const int n_units = nb_total * heads;

  for (int ui = u_begin; ui < u_end; ++ui) {
    const int unit = from_idx ? from_idx[ui] : ui;
    if (unit < 0 || unit >= n_units) continue;       // uniform over the workgroup
    const int s = find_seq_by_unit(seq_blocks, batch, heads, unit);
    const int g0 = seq_blocks[s], n = seq_blocks[s + 1] - g0;
    const int rem = unit - g0 * heads;
    const int h = rem / n, i = rem - h * n;
    const int64_t base = (int64_t(g0) * heads + int64_t(h) * n) * 4096;
    const int row = (plan_heads > 1 ? h : 0) * nb_total + g0 + i;
    const int p0 = to_pos[row];
    const int cnt = to_pos[row + 1] - p0;
    const int iters = (cnt + 1) >> 1;

    // Q fragments: B operand of S^T, Q[query = 32*qh + l32][d = 16*c + 8*hi .. +7]
    v8 qf[4];
    {
      const T* qp = q + base + int64_t(i) * 4096 + (32 * qh + l32) * 64 + 8 * hi;
#pragma unroll
      for (int c = 0; c < 4; ++c) qf[c] = *reinterpret_cast<const v8*>(qp + 16 * c);
    }
    f32x16 o_acc[2];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int e = 0; e < 16; ++e) o_acc[t][e] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;

    v8 pk[4], pv[4];                                  // this thread's 64 bytes of the next K and V^T tiles
    auto gload = [&](int j) {
      int blk = to_idx[p0 + j];
      blk = blk < 0 ? 0 : (blk >= n ? n - 1 : blk);
      const T* kp = k + base + int64_t(blk) * 4096;
      const T* vp = vt + base + int64_t(blk) * 4096;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        pk[c] = *reinterpret_cast<const v8*>(kp + (ptid + 128 * c) * 8);
        pv[c] = *reinterpret_cast<const v8*>(vp + (ptid + 128 * c) * 8);
      }
    };
    if (ks < cnt) gload(ks);

    for (int it = 0; it < iters; ++it) {
      const int j = 2 * it + ks;
      const bool valid = j < cnt;
      __syncthreads();                                // every wave is done reading the previous tiles
      if (valid) {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const int chunk = ptid + 128 * c;
          const int off = (chunk >> 3) * ROW + (chunk & 7) * 8;
          *reinterpret_cast<v8*>(lds_k + off) = pk[c];
          *reinterpret_cast<v8*>(lds_v + off) = pv[c];
        }
      }
      __syncthreads();                                // tiles visible
      if (j + 2 < cnt) gload(j + 2);                  // in flight during the MFMAs below
      if (!valid) continue;

      f32x16 sc[2];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
#pragma unroll
        for (int e = 0; e < 16; ++e) sc[t][e] = 0.f;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const v8 a = *reinterpret_cast<const v8*>(lds_k + (32 * t + l32) * ROW + 16 * c + 8 * hi);
          sc[t] = Mma<T>::run(a, qf[c], sc[t]);
        }
      }
      // online softmax; the lane holds 32 of its query's 64 scores, lane ^ 32 the others
      float mx = sc[0][0];
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) mx = fmaxf(mx, sc[t][e]);
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float m_new = fmaxf(m_run, mx);
      const float alpha = __builtin_amdgcn_exp2f((m_run - m_new) * LOG2E);
      const float mb = m_new * LOG2E;
      float psum = 0.f;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          sc[t][e] = __builtin_amdgcn_exp2f(sc[t][e] * LOG2E - mb);
          psum += sc[t][e];
        }
      l_run = l_run * alpha + psum;
      m_run = m_new;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) o_acc[t][e] *= alpha;
      // P as the B operand: step st takes accumulator registers 8*(st&1)..+7 of tile st>>1
      v8 pb[4];
#pragma unroll
      for (int st = 0; st < 4; ++st)
#pragma unroll
        for (int e = 0; e < 8; ++e) pb[st][e] = static_cast<T>(sc[st >> 1][8 * (st & 1) + e]);
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int st = 0; st < 4; ++st) {
          const v8 a = *reinterpret_cast<const v8*>(lds_v + (32 * t + l32) * ROW + 16 * st + 8 * hi);
          o_acc[t] = Mma<T>::run(a, pb[st], o_acc[t]);
        }
    }

    // merge the two key streams: stream 1 parks (O, m, l) in LDS, stream 0 combines and stores
    l_run += __shfl_xor(l_run, 32, 64);
    __syncthreads();                                  // all tile reads finished before LDS is reused
    float* park = reinterpret_cast<float*>(smem) + qh * (34 * 64);
    if (ks == 1) {
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) park[(16 * t + e) * 64 + lane] = o_acc[t][e];
      park[32 * 64 + lane] = m_run;
      park[33 * 64 + lane] = l_run;
    }
    __syncthreads();
    if (ks == 0) {
      const float m1 = park[32 * 64 + lane], l1 = park[33 * 64 + lane];
      const float m_tot = fmaxf(fmaxf(m_run, m1), -1e30f);      // finite even for an empty row
      const float a0 = __builtin_amdgcn_exp2f((m_run - m_tot) * LOG2E);
      const float a1 = __builtin_amdgcn_exp2f((m1 - m_tot) * LOG2E);
      const float inv = 1.0f / fmaxf(l_run * a0 + l1 * a1, 1e-30f);
      const float w0 = a0 * inv, w1 = a1 * inv;
      // O^T[d = 32*t + 8*(e>>2) + 4*hi + (e&3)][query l32] -> out[token][h*64 + d]
      T* op = out + (int64_t(g0 + i) * 64 + 32 * qh + l32) * (int64_t(heads) * 64) + h * 64 + 4 * hi;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int c4 = 0; c4 < 4; ++c4) {
          v4 r;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int v = 4 * c4 + e;
            r[e] = static_cast<T>(o_acc[t][v] * w0 + park[(16 * t + v) * 64 + lane] * w1);
          }
          *reinterpret_cast<v4*>(op + 32 * t + 8 * c4) = r;
        }
    }
  }
}

}  // namespace

extern "C" int rt_bs_attention_fwd(const void* q, const void* k, const void* vt, void* out, const int* seq_blocks_dev,
                                   int batch, int total_blocks, int heads, const int* to_idx, const int* to_pos,
                                   int plan_heads, const int* from_idx, const int* from_pos, int n_wg, int dtype,
                                   void* stream) {
  RT_REQUIRE(q && k && vt && out && seq_blocks_dev && to_idx && to_pos, RT_EINVAL, "NULL pointer");
  RT_REQUIRE(batch >= 1 && total_blocks >= batch && heads >= 1, RT_EINVAL, "bad geometry: batch=%d total_blocks=%d heads=%d",
             batch, total_blocks, heads);
  RT_REQUIRE(plan_heads == 1 || plan_heads == heads, RT_EINVAL, "plan_heads=%d must be 1 or heads=%d", plan_heads, heads);
  RT_REQUIRE((from_idx == nullptr) == (from_pos == nullptr), RT_EINVAL, "from_idx and from_pos go together");
  RT_REQUIRE(int64_t(total_blocks) * heads < (int64_t(1) << 31), RT_EINVAL, "too many units");
  RT_REQUIRE(((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(vt) |
               reinterpret_cast<uintptr_t>(out)) & 15u) == 0, RT_EINVAL, "q, k, vt, out must be 16-byte aligned");
  if (dtype == RT_F32) return rt::fail(RT_ENOSYS, "block-sparse attention runs in fp16 or bf16 (fp32 accumulation)");
  RT_REQUIRE(dtype == RT_F16 || dtype == RT_BF16, RT_EINVAL, "unknown dtype %d", dtype);
  unsigned grid;
  if (from_idx) {
    RT_REQUIRE(n_wg >= 1, RT_EINVAL, "balanced launch needs n_wg >= 1, got %d", n_wg);
    grid = unsigned(n_wg);
  } else {
    grid = unsigned(total_blocks) * unsigned(heads);
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == RT_F16)
    hipLaunchKernelGGL(bs_attention_kernel<_Float16>, dim3(grid), dim3(256), 0, st, (const _Float16*)q, (const _Float16*)k,
                       (const _Float16*)vt, (_Float16*)out, seq_blocks_dev, batch, heads, total_blocks, to_idx, to_pos,
                       plan_heads, from_idx, from_pos);
  else
    hipLaunchKernelGGL(bs_attention_kernel<__bf16>, dim3(grid), dim3(256), 0, st, (const __bf16*)q, (const __bf16*)k,
                       (const __bf16*)vt, (__bf16*)out, seq_blocks_dev, batch, heads, total_blocks, to_idx, to_pos,
                       plan_heads, from_idx, from_pos);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return rt::fail(RT_EIO, "bs_attention launch failed: %s", hipGetErrorString(e));
  return RT_OK;
}
