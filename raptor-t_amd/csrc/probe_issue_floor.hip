// Issue-rate probes behind the attention kernel's ceiling: how fast one SIMD of gfx950 gets through the
// instruction mix of one (64 query x 64 key, d = 64) block pair when nothing but instruction issue is
// in the way (every operand in registers, no memory access, no LDS, no barrier).
//
//   variant 0   the 32 v_mfma_f32_32x32x16_f16 of a pair alone (16 for K.Q^T, 16 for V^T.P^T)
//   variant 1   + the 64 v_exp_f32 that turn a pair's 4096 scores into probabilities (and 32 v_xor that use them)
//   variant 2   + the 32 v_cvt_pk_f16_f32 that round them to the matrix operand type
//   variant 3   + the 32 packed additions of the row sums: the tile loop's whole mix, in the loop's own slot
//               order (one matrix instruction, two exponentials, one conversion, one addition per slot)
//
// Every wave runs `iters` pairs; the grid is one workgroup per CU of `waves_per_simd` x 4 waves, so each SIMD
// holds exactly waves_per_simd waves and (kernel time) / (iters x waves_per_simd) is the time one SIMD needs
// per pair.  The data flow is the tile loop's: exponentials read the score accumulators, conversions read the
// exponentials, the second product's B operand is the converted values.  Built into its own small library
// (librt_probe.so); nothing of the product links against it.
#include <hip/hip_runtime.h>

#include <cstdint>

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

#define SB() __builtin_amdgcn_sched_barrier(0)

template <int VARIANT>
__global__ __launch_bounds__(512, 1) void issue_floor_kernel(float* out, long long* clocks, int iters) {
  const int lane = threadIdx.x & 63;
  const long long c0 = clock64(), w0 = wall_clock64();
  f16x8 kf[8], vf[8], qf[2][4];
  // operands with every mantissa bit in use, of the size real K, V and scaled Q have: what the matrix pipe draws,
  // and with it the clock the part sustains, depends on how many operand bits toggle
  auto value = [&](uint32_t salt, float scale) {
    uint32_t x = (uint32_t(threadIdx.x) * 2654435761u) ^ (salt * 0x9E3779B9u) ^ (uint32_t(blockIdx.x) * 0x85EBCA6Bu);
    x ^= x >> 16; x *= 0x7FEB352Du; x ^= x >> 15; x *= 0x846CA68Bu; x ^= x >> 16;
    return static_cast<_Float16>((float(x & 0xFFFFu) * (1.0f / 65536.0f) - 0.5f) * scale);
  };
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      kf[i][e] = value(uint32_t(8 * i + e), 3.5f);
      vf[i][e] = value(uint32_t(64 + 8 * i + e), 3.5f);
      qf[i >> 2][i & 3][e] = value(uint32_t(128 + 8 * i + e), 0.6f);
    }
  f32x16 o[2][2] = {}, sc[2] = {}, negm;
#pragma unroll
  for (int e = 0; e < 16; ++e) negm[e] = -4.0f;          // scores end up mostly below the reference, as in the kernel
  f16x8 pb[2][2] = {};
  uint32_t lsum = 0;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int S = 0; S < 4; ++S) {
      const int ktn = ((S + 1) & 3) >> 1, ntn = (S + 1) & 1, ktp = ((S + 3) & 3) >> 1, ntp = (S + 3) & 1;
      f32x16& cur = sc[S & 1];
      f32x16& nxt = sc[(S + 1) & 1];
      f16x8 (&pprev)[2] = pb[(S + 1) & 1];
      float p[16];
      uint32_t w[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        SB();
        if ((i & 1) == 0) {
          const int c = i >> 1;
          // variant 0 keeps accumulating, so that no product of an earlier trip is dead code
          nxt = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[ktn * 4 + c], qf[ntn][c], (c == 0 && VARIANT > 0) ? negm : nxt, 0, 0, 0);
        } else {
          const int tt = (i >> 1) & 1, s = i >> 2;
          o[tt][ntp] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf[tt * 4 + 2 * ktp + s], pprev[s], o[tt][ntp], 0, 0, 0);
        }
        SB();
        if (VARIANT == 0) continue;                     // the matrix instructions alone; P stays what it was
        p[2 * i] = __builtin_amdgcn_exp2f(cur[2 * i]);
        p[2 * i + 1] = __builtin_amdgcn_exp2f(cur[2 * i + 1]);
        if (VARIANT >= 2) {
          w[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{p[2 * i], p[2 * i + 1]}, f16x2));
        } else {                                        // the exponentials must be used by something: one full-rate instruction
          w[i] = __builtin_bit_cast(uint32_t, p[2 * i]) ^ __builtin_bit_cast(uint32_t, p[2 * i + 1]);
        }
        if (VARIANT >= 3)
          lsum = __builtin_bit_cast(uint32_t, __builtin_bit_cast(f16x2, lsum) + __builtin_bit_cast(f16x2, w[i]));
      }
      if (VARIANT == 0) continue;
      SB();
      u32x4 lo = {w[0], w[1], w[2], w[3]}, up = {w[4], w[5], w[6], w[7]};
      pb[S & 1][0] = __builtin_bit_cast(f16x8, lo);
      pb[S & 1][1] = __builtin_bit_cast(f16x8, up);
      SB();
    }
  }
  float s = __builtin_bit_cast(float, lsum);
#pragma unroll
  for (int e = 0; e < 16; ++e) s += o[0][0][e] + o[0][1][e] + o[1][0][e] + o[1][1][e] + sc[0][e] + sc[1][e];
  out[blockIdx.x * blockDim.x + threadIdx.x] = s;
  // shader-clock cycles and ticks of the constant-rate clock this wave spent: their ratio is the clock the CU held
  if (clocks && threadIdx.x == 0) {
    clocks[2 * blockIdx.x] = clock64() - c0;
    clocks[2 * blockIdx.x + 1] = wall_clock64() - w0;
  }
}

}  // namespace

// Launches one probe on `stream`: `out` needs cus * waves_per_simd * 256 floats of device memory, `clocks` (optional)
// 2 * cus 64-bit integers: per workgroup the shader-clock cycles and the constant-rate clock's ticks its first wave
// ran for.  Returns 0, or -22 for an argument outside its range, -5 if the launch failed.
extern "C" int rt_probe_issue_floor(int variant, int waves_per_simd, int iters, int cus, float* out, long long* clocks,
                                    void* stream) {
  if (variant < 0 || variant > 3 || (waves_per_simd != 1 && waves_per_simd != 2) || iters < 1 || cus < 1 || !out) return -22;
  const dim3 grid(cus), block(256 * waves_per_simd);
  hipStream_t st = static_cast<hipStream_t>(stream);
  switch (variant) {
    case 0: hipLaunchKernelGGL(issue_floor_kernel<0>, grid, block, 0, st, out, clocks, iters); break;
    case 1: hipLaunchKernelGGL(issue_floor_kernel<1>, grid, block, 0, st, out, clocks, iters); break;
    case 2: hipLaunchKernelGGL(issue_floor_kernel<2>, grid, block, 0, st, out, clocks, iters); break;
    default: hipLaunchKernelGGL(issue_floor_kernel<3>, grid, block, 0, st, out, clocks, iters); break;
  }
  return hipGetLastError() == hipSuccess ? 0 : -5;
}
