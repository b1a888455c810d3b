// Block-sparse attention in fp32: the accuracy mode of the layer (the reference dispatches an
// fp32-output kernel when the attention buffer is fp32, layers/multi_headed_attention.cpp:198-199,
// layers/kernels/sparse_attention.cu:785-1120, :1582-1599).  Same inputs, plans and outputs as the
// fp16 / bf16 kernel of bs_attention.hip, with every tensor in fp32 and the tile products on
// v_mfma_f32_16x16x4_f32.  Written for exactness and simplicity, not speed: fp32 matrix
// throughput is a sixteenth of fp16's, so this path is MFMA bound at a few hundred microseconds
// for a batch the fp16 kernel finishes in a hundred.
//
// One workgroup of four waves per unit (64 queries of one head against the unit's list of key
// blocks); wave w owns queries 16w .. 16w+15.  Per key block the K and V^T tiles (fragment order
// in memory, as rt_qkv_bias_split writes them) are copied into LDS in plain [row][col] order, then
//   S^T[key][q] = sum_d K[key][d] Q[q][d]        4 tiles of 16 keys, 16 MFMAs each
//   online softmax per query (a lane's column), moving maximum, base 2 (the scale log2(e)/sqrt(d)
//   is folded into Q)
//   O^T[d][q] += sum_key V^T[d][key] P^T[key][q]  4 tiles of 16 d, 16 MFMAs each
// A lane of an S^T accumulator holds keys 16 kt + 4 (lane >> 4) + i of query lane & 15, which is the
// B operand of the second product for the key subset {4 g + i : g = 0..3}: the V^T operand is read
// from LDS for the same subset, so P never leaves its registers.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "rt_launch.h"

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int PITCH = 68;            // floats per LDS row: 16-byte aligned rows, rows 4 banks apart

struct ArgsF32 {
  const float* q; const float* k; const float* vt; float* out;
  const int* seq_blocks; int batch; int heads; int nb_total;
  const int* to_idx; const int* to_pos; int plan_heads;
  const int* from_idx; const int* from_pos;
  const int* seq_tokens;
  const float* q_rows; const float* q_bias; float q_scale;
};

// element (row, col) of a 64 x 64 tile in fragment order
__device__ __forceinline__ int frag_index(int row, int col) {
  return ((4 * (row >> 5) + (col >> 4)) * 64 + (row & 31) + 32 * ((col >> 3) & 1)) * 8 + (col & 7);
}

// token whose V column sits in slot p of a V^T tile (tokens 4-7 and 8-11 of every 16 swap places)
__device__ __forceinline__ int slot_token(int p) {
  const int e = p & 15;
  return (p & ~15) | ((e & 3) | ((e & 4) << 1) | ((e & 8) >> 1));
}

// Copies one tile from fragment order into LDS as dst[row][col].  Thread t takes 16 floats: four
// runs of 4 consecutive columns.  `V`: the tile is V^T[d][slot]; it is stored as dst[d][token].
template <bool V>
__device__ __forceinline__ void stage_tile(const float* __restrict__ src, float (*dst)[PITCH]) {
#pragma unroll
  for (int it = 0; it < 4; ++it) {
    const int e = (threadIdx.x + it * 256) * 4;       // first element of the run, fragment order
    const f32x4 x = *reinterpret_cast<const f32x4*>(src + e);
    const int frag = e >> 9, lane = (e >> 3) & 63, sub = e & 7;
    const int row = 32 * (frag >> 2) + (lane & 31);
    const int col = 16 * (frag & 3) + 8 * (lane >> 5) + sub;
    if (V) {
#pragma unroll
      for (int i = 0; i < 4; ++i) dst[row][slot_token(col + i)] = x[i];
    } else {
      *reinterpret_cast<f32x4*>(&dst[row][col]) = x;
    }
  }
}

__device__ __forceinline__ float group_max(float v) {     // over the four lanes that share lane & 15
  v = fmaxf(v, __shfl_xor(v, 16));
  return fmaxf(v, __shfl_xor(v, 32));
}
__device__ __forceinline__ float group_sum(float v) {
  v += __shfl_xor(v, 16);
  return v + __shfl_xor(v, 32);
}

template <bool MASKED>
__device__ void run_unit(const ArgsF32& a, int unit, float (*ks)[PITCH], float (*vs)[PITCH]) {
  // flat unit id = block + head * n_s + first block of the sequence * heads
  int lo = 0, hi = a.batch;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (a.seq_blocks[mid] * a.heads <= unit) lo = mid; else hi = mid;
  }
  const int g0 = a.seq_blocks[lo], n = a.seq_blocks[lo + 1] - g0;
  const int rem = unit - g0 * a.heads;
  const int h = rem / n, i = rem - h * n;
  // blocks that hold real tokens and the real tokens of the last of them; at least one (a tile with every key
  // masked has no finite maximum); blocks from nbv on are padding as a whole and are left out
  const int tokens = MASKED ? min(max(a.seq_tokens[lo], 1), 64 * n) : 64 * n;
  const int nbv = (tokens + 63) >> 6, tail = tokens - 64 * (nbv - 1);
  const int row = (a.plan_heads > 1 ? h : 0) * a.nb_total + g0 + i;
  const int p0 = a.to_pos[row], p1 = a.to_pos[row + 1];
  const int64_t head_base = (int64_t(g0) * a.heads + int64_t(h) * n) * 4096;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int qcol = lane & 15, grp = lane >> 4;
  const int dm = a.heads * 64;

  // Q^T operand: lane holds Q[16 wave + qcol][4 step + grp] for step = 0..15
  float qreg[16];
  {
    const int qrow = 16 * wave + qcol;
    if (a.q_rows) {
      const float* src = a.q_rows + (int64_t(g0 + i) * 64 + qrow) * (3 * dm) + h * 64;
#pragma unroll
      for (int s = 0; s < 16; ++s) {
        const int d = 4 * s + grp;
        qreg[s] = (src[d] + (a.q_bias ? a.q_bias[h * 64 + d] : 0.f)) * a.q_scale;
      }
    } else {
      const float* src = a.q + head_base + int64_t(i) * 4096;
#pragma unroll
      for (int s = 0; s < 16; ++s) qreg[s] = src[frag_index(qrow, 4 * s + grp)];
    }
  }

  f32x4 o[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) o[t] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;

  for (int p = p0; p < p1; ++p) {
    const int blk = min(max(a.to_idx[p], 0), n - 1);   // a malformed index must not lead outside the (sequence, head)
    if (MASKED && blk >= nbv) continue;                // the same in every thread of the workgroup
    __syncthreads();                                   // the previous tile's readers are done
    stage_tile<false>(a.k + head_base + int64_t(blk) * 4096, ks);
    stage_tile<true>(a.vt + head_base + int64_t(blk) * 4096, vs);
    __syncthreads();
    f32x4 s[4];
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) {
      s[kt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int st = 0; st < 16; ++st)
        s[kt] = __builtin_amdgcn_mfma_f32_16x16x4f32(ks[16 * kt + qcol][4 * st + grp], qreg[st], s[kt], 0, 0, 0);
    }
    if (MASKED && blk == nbv - 1 && tail < 64) {
#pragma unroll
      for (int kt = 0; kt < 4; ++kt)
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (16 * kt + 4 * grp + e >= tail) s[kt][e] = -INFINITY;
    }
    float mx = s[0][0];
#pragma unroll
    for (int kt = 0; kt < 4; ++kt)
#pragma unroll
      for (int e = 0; e < 4; ++e) mx = fmaxf(mx, s[kt][e]);
    mx = group_max(mx);
    const float m_new = fmaxf(m, mx);                  // finite: key 0 of a block is never padding
    const float c = exp2f(m - m_new);
    float part = 0.f;
#pragma unroll
    for (int kt = 0; kt < 4; ++kt)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        s[kt][e] = exp2f(s[kt][e] - m_new);
        part += s[kt][e];
      }
    l = l * c + group_sum(part);
    m = m_new;
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) {
      o[dt] *= c;
#pragma unroll
      for (int kt = 0; kt < 4; ++kt)
#pragma unroll
        for (int e = 0; e < 4; ++e)
          o[dt] = __builtin_amdgcn_mfma_f32_16x16x4f32(vs[16 * dt + qcol][16 * kt + 4 * grp + e], s[kt][e], o[dt], 0, 0, 0);
    }
  }
  // O^T accumulator dt: lane holds d = 16 dt + 4 grp + e for query qcol
  const float inv = 1.0f / fmaxf(l, 1e-30f);          // a row that lists nothing but padding writes zeros
  float* dst = a.out + (int64_t(g0 + i) * 64 + 16 * wave + qcol) * dm + h * 64;
#pragma unroll
  for (int dt = 0; dt < 4; ++dt) *reinterpret_cast<f32x4*>(dst + 16 * dt + 4 * grp) = o[dt] * inv;
}

template <bool MASKED>
__global__ __launch_bounds__(256) void bs_attention_f32_kernel(ArgsF32 a) {
  __shared__ __attribute__((aligned(16))) float ks[64][PITCH];
  __shared__ __attribute__((aligned(16))) float vs[64][PITCH];
  const int n_units = a.nb_total * a.heads;
  if (a.from_pos) {
    // a plan the host has not checked must not lead outside from_idx: clamp the slice, skip bad ids
    const int begin = min(max(a.from_pos[blockIdx.x], 0), n_units);
    const int end = min(max(a.from_pos[blockIdx.x + 1], begin), n_units);
    for (int p = begin; p < end; ++p) {
      const int unit = a.from_idx[p];
      if (unit >= 0 && unit < n_units) run_unit<MASKED>(a, unit, ks, vs);
    }
    return;
  }
  // Without a plan: one unit per workgroup.  The two rows of a sparse sequence that list every
  // block take ten times as long as the others; they are the units of blocks 0 and n - 1, spread
  // evenly over the grid by the flat numbering, and the hardware hands workgroups out in order.
  run_unit<MASKED>(a, blockIdx.x, ks, vs);
}

}  // namespace

namespace rt {

int launch_attention_f32(const void* q, const void* q_rows, const void* q_bias, float q_scale, const void* k,
                         const void* vt, void* out, const int* seq_blocks_dev, const int* seq_tokens_dev, int batch,
                         int total_blocks, int heads, const int* to_idx, const int* to_pos, int plan_heads,
                         const int* from_idx, const int* from_pos, int n_wg, void* stream) {
  const ArgsF32 a{(const float*)q, (const float*)k, (const float*)vt, (float*)out, seq_blocks_dev, batch, heads,
                  total_blocks, to_idx, to_pos, plan_heads, from_idx, from_pos, seq_tokens_dev,
                  (const float*)q_rows, (const float*)q_bias, q_scale};
  const unsigned grid = from_idx ? unsigned(n_wg) : unsigned(total_blocks) * unsigned(heads);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (seq_tokens_dev) RT_LAUNCH(bs_attention_f32_kernel<true>, dim3(grid), dim3(256), 0, st, a);
  else RT_LAUNCH(bs_attention_f32_kernel<false>, dim3(grid), dim3(256), 0, st, a);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return rt::fail(RT_EIO, "fp32 bs_attention launch failed: %s", hipGetErrorString(e));
  return RT_OK;
}

}  // namespace rt
