// Block-sparse (BigBird-pattern) attention forward for gfx950, d = 64, 64-token blocks.
//
// Work unit = (sequence, head, from-block): 64 queries against the key blocks its CSR row
// lists (7/8 blocks for a sparse row, all n blocks for the two global rows).
//
// One wave owns all 64 queries of a unit and streams K / V^T tiles straight from global
// memory into MFMA operand registers: the QKV split kernel stores every 64x64 tile in
// "fragment order" (8 fragments of 64 lanes x 16 bytes), so each operand load is one fully
// coalesced 1 KiB request and the main loop needs no LDS and no barrier.  The next K tile
// is requested as soon as the last QK^T product of the current tile has issued, the next
// V^T tile after the last PV product: one register copy of each, latency covered by the
// softmax and the other product.
//
//   sparse rows : one wave per unit, 4 units (adjacent from-blocks) per workgroup
//   global rows : the 4 waves of a workgroup take every 4th key block of ONE unit and merge
//                 their online-softmax states through LDS at the end
//
// MFMA formulation (v_mfma_f32_32x32x16_{f16,bf16}, fp32 accumulators):
//   S^T[key][query] = K[key][:] . Q[query][:]       A = K fragment,   B = Q fragment
//   O^T[d][query]  += V^T[d][key] . P^T[key][query]  A = V^T fragment, B = P (registers)
// Both products put the query on the accumulator column (lane & 31): max, sum and rescale
// factors are per-lane scalars and the S^T accumulators, after exp2, are the B operand of
// the second product, so P never leaves registers.
//
// Softmax is evaluated in base 2 (q arrives pre-multiplied by log2(e)/sqrt(d)).  The S^T
// accumulator starts at minus the row's reference maximum, so the MFMA result feeds exp2
// directly; the reference is only moved (and O, l rescaled) when a lane's partial row sum of
// P = 2^(score - reference) over one key tile exceeds 2^11: a rare, wave-uniform branch that
// recomputes the half tile with a proper maximum.
//
// The kernel is persistent (two workgroups per CU).  Without a plan it makes its own
// schedule: global rows first, each XCD (one L2 per XCD; workgroups are dealt round-robin to
// the 8 XCDs) walking its own contiguous share of the (sequence, head) groups, so a group's
// K/V tiles stay in one L2.  With an LPT plan, n_wg workgroups walk their unit lists.
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
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <typename T> struct Mma;
template <> struct Mma<_Float16> {
  typedef f16x8 v8;
  typedef f16x4 v4;
  __device__ static f32x16 run(v8 a, v8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
  // a[0..7] = p[0..7] rounded to T; returns the fp32 sum of the ROUNDED values (what PV multiplies)
  __device__ static float pack(const float* p, v8& out) {
    float s = 0.f;
    u32x4 w;                                  // whole dwords: each pair stays one v_cvt_pk_f16_f32
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const f16x2 h = __builtin_convertvector(f32x2{p[2 * i], p[2 * i + 1]}, f16x2);
      w[i] = __builtin_bit_cast(uint32_t, h);
      s = __builtin_amdgcn_fdot2(h, f16x2{1, 1}, s, false);
    }
    out = __builtin_bit_cast(v8, w);
    return s;
  }
};
template <> struct Mma<__bf16> {
  typedef bf16x8 v8;
  typedef bf16x4 v4;
  __device__ static f32x16 run(v8 a, v8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
  // a[0..7] = p[0..7] rounded to bf16; returns the fp32 sum of the UNROUNDED values: converting the
  // rounded ones back would cost as many instructions again, and the rounding errors of a row's
  // sum (relative 2^-9 each, random sign) are far below what bf16 outputs resolve
  __device__ static float pack(const float* p, v8& out) {
#pragma unroll
    for (int e = 0; e < 8; ++e) out[e] = static_cast<__bf16>(p[e]);
    return ((p[0] + p[1]) + (p[2] + p[3])) + ((p[4] + p[5]) + (p[6] + p[7]));
  }
};

// A row's reference maximum only moves when the 32 values P = 2^(score - reference) a lane holds
// for one key tile add up to more than 2^11 (no single P can then exceed 2^11, far inside fp16's
// range, and P keeps its full relative precision at any magnitude): the row sum the kernel needs
// anyway doubles as the overflow test.
constexpr float SUM_LIMIT = 2048.0f;

// Online-softmax state of one wave for its 64 queries: O^T as [d tile][query tile].
struct State {
  f32x16 o[2][2];
  float m[2], l[2];      // per query tile: reference maximum (log2 units), partial row sum
};

__device__ inline void state_init(State& st) {
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int e = 0; e < 16; ++e) st.o[t][nt][e] = 0.f;
  st.m[0] = st.m[1] = -INFINITY;
  st.l[0] = st.l[1] = 0.f;
}

template <typename T>
__device__ inline void load_tile(const T* __restrict__ tile, int lane, typename Mma<T>::v8 (&f)[8]) {
  typedef typename Mma<T>::v8 v8;
#pragma unroll
  for (int i = 0; i < 8; ++i) f[i] = *reinterpret_cast<const v8*>(tile + i * 512 + lane * 8);
}

// Streams key blocks row[first], row[first + step], ... of one (sequence, head) through the
// state.  kbase / vbase point at block 0 of that (sequence, head); n = blocks in the sequence.
// The row's block ids are fetched 64 at a time into one register (lane j holds entry j) and
// handed out with v_readlane: one memory round trip per unit instead of one per key block.
template <typename T, bool MASKED>
__device__ inline void stream_tiles(const T* __restrict__ kbase, const T* __restrict__ vbase,
                                    const int* __restrict__ row, int first, int step, int cnt, int n, int tail,
                                    int lane, const typename Mma<T>::v8 (&qf)[2][4], State& st) {
  typedef typename Mma<T>::v8 v8;
  v8 kf[8], vf[8];
  bool fresh = true;                                  // no reference maximum yet
  // Rows longer than 64 entries are walked in chunks of 64: the ids are only (re)loaded between
  // chunks, so inside the tile loop the only outstanding memory operations are the tile
  // prefetches and the waits on them can be exact.
  for (int j = first; j < cnt;) {
  const int chunk = j >> 6;
  const int hi = min(cnt, (chunk + 1) * 64);
  const int ids = (chunk * 64 + lane < cnt) ? row[chunk * 64 + lane] : 0;
  auto block_of = [&](int e) {                        // e is wave-uniform and inside the chunk
    const int b = __builtin_amdgcn_readlane(ids, e & 63);
    return b < 0 ? 0 : (b >= n ? n - 1 : b);
  };
  int bcur = block_of(j);
  load_tile<T>(kbase + int64_t(bcur) * 4096, lane, kf);
  load_tile<T>(vbase + int64_t(bcur) * 4096, lane, vf);
  for (; j < hi; j += step) {
    const int jn = j + step;
    const bool more = jn < hi;
    // keys of the sequence's last block beyond its true length are padding: no weight
    const bool padded = MASKED && tail < 64 && bcur == n - 1;
    // the last iteration re-requests its own tile: loads stay unconditional, so they keep
    // their place in the instruction stream (a branch would sink them next to their use)
    const int bn = block_of(more ? jn : j);
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      f32x16 sc[2];
      v8 pb[4];
      float psum;
      auto scores = [&](float init) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
#pragma unroll
          for (int e = 0; e < 16; ++e) sc[t][e] = init;
#pragma unroll
          for (int c = 0; c < 4; ++c) sc[t] = Mma<T>::run(kf[t * 4 + c], qf[nt][c], sc[t]);
        }
        if (MASKED && padded) {                         // wave-uniform, at most one tile of a row
#pragma unroll
          for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int e = 0; e < 16; ++e)
              if (32 * t + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3) >= tail) sc[t][e] = -INFINITY;
        }
      };
      // exp2 of the (already shifted) scores -> P as the B operand of the second product:
      // step s takes accumulator registers 8*(s&1)..+7 of key tile s>>1.  Returns true when the
      // lane's 32 values of P add up to more than SUM_LIMIT (or to something not finite).
      auto exponentiate = [&]() {
        float part[4];
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          float p8[8];
#pragma unroll
          for (int e = 0; e < 8; ++e) p8[e] = __builtin_amdgcn_exp2f(sc[s >> 1][8 * (s & 1) + e]);
          part[s] = Mma<T>::pack(p8, pb[s]);
        }
        psum = (part[0] + part[1]) + (part[2] + part[3]);
        return !(psum <= SUM_LIMIT);                    // also true for an infinite or undefined sum
      };
      bool redo = fresh;
      if (!fresh) {
        scores(-st.m[nt]);
        redo = __any(exponentiate());
      }
      if (redo) {
        // rare (always on the first tile): find the true maximum and move the reference there
        scores(0.f);
        float mx = sc[0][0];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int e = 0; e < 16; ++e) mx = fmaxf(mx, sc[t][e]);
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fresh ? mx : fmaxf(mx, st.m[nt]);
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int e = 0; e < 16; ++e) sc[t][e] -= m_new;
        if (!fresh) {
          const float alpha = __builtin_amdgcn_exp2f(st.m[nt] - m_new);
          st.l[nt] *= alpha;
#pragma unroll
          for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int e = 0; e < 16; ++e) st.o[t][nt][e] *= alpha;
        }
        st.m[nt] = m_new;
        (void)exponentiate();
      }
      // the K fragments are dead once the second query tile's scores are final
      if (nt == 1) {
        __builtin_amdgcn_sched_barrier(0);
        load_tile<T>(kbase + int64_t(bn) * 4096, lane, kf);
        __builtin_amdgcn_sched_barrier(0);
      }
      st.l[nt] += psum;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int s = 0; s < 4; ++s) st.o[t][nt] = Mma<T>::run(vf[t * 4 + s], pb[s], st.o[t][nt]);
    }
    fresh = false;
    bcur = bn;
    __builtin_amdgcn_sched_barrier(0);
    load_tile<T>(vbase + int64_t(bn) * 4096, lane, vf);
    __builtin_amdgcn_sched_barrier(0);
  }
  }
}

// Writes the wave's 64x64 output tile, O^T[d = 32t + 8*(e>>2) + 4*(lane>>5) + (e&3)]
// [query 32nt + (lane&31)] * w, to out[token][h*64 + d].  The tile is transposed through a
// wave-private LDS region (64 rows of 64 + 4 elements) so that every global store covers
// whole 128-byte row segments: 8 lanes x 16 bytes per row.
constexpr int STAGE_ROW = 68;                       // elements; 136 bytes keeps ds_write_b64 conflict free
constexpr int STAGE_BYTES = 64 * STAGE_ROW * 2;     // 8704 bytes per wave

template <typename T>
__device__ inline void store_output(T* __restrict__ out_unit, int64_t row_stride, int lane, const State& st,
                                    const float (&w)[2], T* __restrict__ stage) {
  typedef typename Mma<T>::v4 v4;
  typedef typename Mma<T>::v8 v8;
  const int l32 = lane & 31, hi = lane >> 5;
#pragma unroll
  for (int nt = 0; nt < 2; ++nt) {
    T* sp = stage + (32 * nt + l32) * STAGE_ROW + 4 * hi;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int c4 = 0; c4 < 4; ++c4) {
        v4 r;
#pragma unroll
        for (int e = 0; e < 4; ++e) r[e] = static_cast<T>(st.o[t][nt][4 * c4 + e] * w[nt]);
        *reinterpret_cast<v4*>(sp + 32 * t + 8 * c4) = r;
      }
  }
  __builtin_amdgcn_wave_barrier();                  // same wave wrote it: LDS is in order per wave
  const int r8 = lane >> 3, c8 = (lane & 7) * 8;
#pragma unroll
  for (int it = 0; it < 8; ++it) {
    const int row = 8 * it + r8;
    const v4* src = reinterpret_cast<const v4*>(stage + row * STAGE_ROW + c8);   // rows are 8-byte aligned
    const v4 lo = src[0], up = src[1];
    const v8 v = {lo[0], lo[1], lo[2], lo[3], up[0], up[1], up[2], up[3]};
    *reinterpret_cast<v8*>(out_unit + int64_t(row) * row_stride + c8) = v;
  }
  __builtin_amdgcn_wave_barrier();
}

struct Unit {
  int h, i, n, g0;
  int tail;               // tokens in the sequence's last block that are real (64: none padded)
};

template <typename T> struct Args {
  const T* q; const T* k; const T* vt; T* out;
  const int* seq_blocks; int batch, heads, nb_total;
  const int* to_idx; const int* to_pos; int plan_heads;
  const int* from_idx; const int* from_pos;
  const int* seq_tokens;                 // optional: true token count per sequence (padded tail in its last block)
  // optional: Q taken from the QKV projection's own output rows [tokens, 3 * heads * 64] (columns
  // 0 .. heads*64-1), bias added and scale applied while loading; q is then unused
  const T* q_rows; const T* q_bias; float q_scale;
};

constexpr int MAX_BATCH = 1024;         // sequences per launch (geometry is kept in LDS)

// Geometry of the batch in LDS: sb = prefix blocks, gl / bu = prefix counts of the plan-free
// launch's global items and bundles (per sequence, times heads).
struct Geometry {
  int sb[MAX_BATCH + 1];
  int gl[MAX_BATCH + 1];
  int bu[MAX_BATCH + 1];
  int tail[MAX_BATCH];                  // real tokens in each sequence's last block (64 without padding)
};

__device__ inline int upper_seq(const int* __restrict__ prefix, int batch, int x) {
  int lo = 0, hi = batch;               // prefix[lo] <= x < prefix[hi]
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (prefix[mid] <= x) lo = mid; else hi = mid;
  }
  return lo;
}

__device__ inline bool is_global_row(const Unit& u) { return u.n >= RT_MIN_SPARSE_BLOCKS && (u.i == 0 || u.i == u.n - 1); }

template <typename T>
__device__ inline void load_q(const Args<T>& a, const Unit& u, int lane, typename Mma<T>::v8 (&qf)[2][4]) {
  typedef typename Mma<T>::v8 v8;
  if (a.q_rows) {
    // fragment (nt, c), lane l = dims 16c + 8(l >> 5) .. +7 of query 32nt + (l & 31): a 16-byte run of
    // the token's row.  Same arithmetic as the split kernel: (x + bias) * scale in fp32, rounded once.
    const int64_t ld = int64_t(a.heads) * 192;
    const T* src = a.q_rows + (int64_t(u.g0 + u.i) * 64 + (lane & 31)) * ld + u.h * 64 + (lane >> 5) * 8;
    const T* bsrc = a.q_bias + u.h * 64 + (lane >> 5) * 8;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const v8 b = *reinterpret_cast<const v8*>(bsrc + c * 16);
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        const v8 x = *reinterpret_cast<const v8*>(src + nt * 32 * ld + c * 16);
#pragma unroll
        for (int e = 0; e < 8; ++e) qf[nt][c][e] = static_cast<T>((float(x[e]) + float(b[e])) * a.q_scale);
      }
    }
    return;
  }
  const T* qt = a.q + (int64_t(u.g0) * a.heads + int64_t(u.h) * u.n + u.i) * 4096;
#pragma unroll
  for (int nt = 0; nt < 2; ++nt)
#pragma unroll
    for (int c = 0; c < 4; ++c) qf[nt][c] = *reinterpret_cast<const v8*>(qt + (nt * 4 + c) * 512 + lane * 8);
}

// One wave, one unit, all of its key blocks.
template <typename T, bool MASKED>
__device__ inline void run_solo(const Args<T>& a, const Unit& u, int lane, T* stage) {
  typename Mma<T>::v8 qf[2][4];
  const int row = (a.plan_heads > 1 ? u.h : 0) * a.nb_total + u.g0 + u.i;
  const int p0 = __builtin_amdgcn_readfirstlane(a.to_pos[row]);
  const int cnt = __builtin_amdgcn_readfirstlane(a.to_pos[row + 1]) - p0;
  load_q<T>(a, u, lane, qf);
  const int64_t base = (int64_t(u.g0) * a.heads + int64_t(u.h) * u.n) * 4096;
  State st;
  state_init(st);
  stream_tiles<T, MASKED>(a.k + base, a.vt + base, a.to_idx + p0, 0, 1, cnt, u.n, u.tail, lane, qf, st);
  float w[2];
#pragma unroll
  for (int nt = 0; nt < 2; ++nt) {
    const float l = st.l[nt] + __shfl_xor(st.l[nt], 32, 64);
    w[nt] = 1.0f / fmaxf(l, 1e-30f);
  }
  const int64_t stride = int64_t(a.heads) * 64;
  store_output<T>(a.out + int64_t(u.g0 + u.i) * 64 * stride + u.h * 64, stride, lane, st, w, stage);
}

// Four waves, one unit: wave w streams key blocks w, w+4, ...; tree merge through LDS.
template <typename T, bool MASKED>
__device__ inline void run_split4(const Args<T>& a, const Unit& u, int lane, int wave, float* park) {
  typename Mma<T>::v8 qf[2][4];
  const int row = (a.plan_heads > 1 ? u.h : 0) * a.nb_total + u.g0 + u.i;
  const int p0 = __builtin_amdgcn_readfirstlane(a.to_pos[row]);
  const int cnt = __builtin_amdgcn_readfirstlane(a.to_pos[row + 1]) - p0;
  load_q<T>(a, u, lane, qf);
  const int64_t base = (int64_t(u.g0) * a.heads + int64_t(u.h) * u.n) * 4096;
  State st;
  state_init(st);
  stream_tiles<T, MASKED>(a.k + base, a.vt + base, a.to_idx + p0, wave, 4, cnt, u.n, u.tail, lane, qf, st);
#pragma unroll
  for (int nt = 0; nt < 2; ++nt) st.l[nt] += __shfl_xor(st.l[nt], 32, 64);

  auto dump = [&](float* slot) {
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int e = 0; e < 16; ++e) slot[((t * 2 + nt) * 16 + e) * 64 + lane] = st.o[t][nt][e];
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      slot[(64 + nt) * 64 + lane] = st.m[nt];
      slot[(66 + nt) * 64 + lane] = st.l[nt];
    }
  };
  auto absorb = [&](const float* slot) {
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      const float m1 = slot[(64 + nt) * 64 + lane], l1 = slot[(66 + nt) * 64 + lane];
      const float mt = fmaxf(fmaxf(st.m[nt], m1), -1e30f);        // finite even if both are empty
      const float a0 = __builtin_amdgcn_exp2f(st.m[nt] - mt), a1 = __builtin_amdgcn_exp2f(m1 - mt);
      st.m[nt] = mt;
      st.l[nt] = st.l[nt] * a0 + l1 * a1;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e)
          st.o[t][nt][e] = st.o[t][nt][e] * a0 + slot[((t * 2 + nt) * 16 + e) * 64 + lane] * a1;
    }
  };
  __syncthreads();                                    // the park is free (previous item is over)
  if (wave >= 2) dump(park + (wave - 2) * (68 * 64));
  __syncthreads();
  if (wave < 2) absorb(park + wave * (68 * 64));
  __syncthreads();
  if (wave == 1) dump(park);
  __syncthreads();
  if (wave == 0) {
    absorb(park);
    float w[2];
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) w[nt] = 1.0f / fmaxf(st.l[nt], 1e-30f);
    const int64_t stride = int64_t(a.heads) * 64;
    // slot 1 of the park was consumed before the third barrier: reuse it as the staging tile
    store_output<T>(a.out + int64_t(u.g0 + u.i) * 64 * stride + u.h * 64, stride, lane, st, w,
                    reinterpret_cast<T*>(park + 68 * 64));
  }
  __syncthreads();                                    // the park is free again (solo waves stage their output in it)
}

__device__ __host__ inline int bundles_per_head(int n) {
  return n >= RT_MIN_SPARSE_BLOCKS ? (n - 2 + 3) / 4 : (n + 3) / 4;
}

// Persistent workgroups (two per CU).
//
// With an LPT plan (from_idx / from_pos): workgroup c walks its slice of the plan; global rows
// are shared by its four waves, runs of up to four other units go one per wave.
//
// Without a plan the kernel makes its own schedule.  Two kinds of items:
//   global item : one global row (first or last block of a sequence of >= 12 blocks), 4 waves
//   bundle      : up to 4 consecutive other rows of one (sequence, head), one per wave
// numbered sequence-major, then head.  Workgroups are dealt to the 8 XCDs round-robin by the
// hardware; the workgroups of XCD x share the x-th eighth of the global items FIRST (they are
// the long ones) and then the x-th eighth of the bundles, which covers (nearly) the same
// (sequence, head) groups, so a group's K/V tiles stay in one L2.
template <typename T, bool MASKED>
__global__ __launch_bounds__(256, 2) void bs_attention_kernel(Args<T> a) {
  // 34816 bytes: two parked wave states for the global-row merge, or four output staging tiles
  __shared__ __attribute__((aligned(16))) float park[2 * 68 * 64];
  __shared__ Geometry geo;
  static_assert(4 * STAGE_BYTES <= sizeof(float) * 2 * 68 * 64, "staging tiles must fit in the park");
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  T* stage = reinterpret_cast<T*>(reinterpret_cast<char*>(park) + wave * STAGE_BYTES);

  for (int i = threadIdx.x; i <= a.batch; i += 256) geo.sb[i] = a.seq_blocks[i];
  __syncthreads();
  for (int i = threadIdx.x; i < a.batch; i += 256) {
    int t = 64;
    if (MASKED) {
      t = a.seq_tokens[i] - 64 * (geo.sb[i + 1] - geo.sb[i] - 1);
      t = t < 1 ? 1 : (t > 64 ? 64 : t);
    }
    geo.tail[i] = t;
  }
  if (threadIdx.x == 0) {
    int g = 0, b = 0;
    for (int s = 0; s < a.batch; ++s) {
      geo.gl[s] = g;
      geo.bu[s] = b;
      const int n = geo.sb[s + 1] - geo.sb[s];
      g += (n >= RT_MIN_SPARSE_BLOCKS ? 2 : 0) * a.heads;
      b += bundles_per_head(n) * a.heads;
    }
    geo.gl[a.batch] = g;
    geo.bu[a.batch] = b;
  }
  __syncthreads();

  auto unit_of_flat = [&](int unit) {               // flat id = blk + head * n_s + seq_start * heads
    int lo = 0, hi = a.batch;
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (geo.sb[mid] * a.heads <= unit) lo = mid; else hi = mid;
    }
    Unit u;
    u.g0 = geo.sb[lo];
    u.n = geo.sb[lo + 1] - u.g0;
    u.tail = geo.tail[lo];
    const int rem = unit - u.g0 * a.heads;
    u.h = rem / u.n;
    u.i = rem - u.h * u.n;
    return u;
  };

  if (a.from_pos) {
    int p = a.from_pos[blockIdx.x];
    const int end = a.from_pos[blockIdx.x + 1];
    const int n_units = a.nb_total * a.heads;
    while (p < end) {
      // the next four plan entries in one round trip
      const int mine_id = (p + wave < end) ? a.from_idx[p + wave] : -1;
      int ids4[4];
#pragma unroll
      for (int w = 0; w < 4; ++w) ids4[w] = (p + w < end) ? a.from_idx[p + w] : -1;
      if (ids4[0] < 0 || ids4[0] >= n_units) { ++p; continue; }
      const Unit first = unit_of_flat(ids4[0]);
      if (is_global_row(first)) {
        run_split4<T, MASKED>(a, first, lane, wave, park);
        ++p;
        continue;
      }
      int run = 1;
      while (run < 4 && ids4[run] >= 0 && ids4[run] < n_units && !is_global_row(unit_of_flat(ids4[run]))) ++run;
      if (wave < run) run_solo<T, MASKED>(a, unit_of_flat(mine_id), lane, stage);
      p += run;
    }
    return;
  }

  const int n_glob = geo.gl[a.batch], n_bund = geo.bu[a.batch];
  const int x = blockIdx.x & 7, per_xcd = gridDim.x >> 3;
  const int g_lo = int(int64_t(n_glob) * x / 8), g_cnt = int(int64_t(n_glob) * (x + 1) / 8) - g_lo;
  const int b_lo = int(int64_t(n_bund) * x / 8), b_cnt = int(int64_t(n_bund) * (x + 1) / 8) - b_lo;
  for (int k = blockIdx.x >> 3; k < g_cnt + b_cnt; k += per_xcd) {
    Unit u;
    if (k < g_cnt) {
      const int item = g_lo + k;
      const int s = upper_seq(geo.gl, a.batch, item);
      const int rem = item - geo.gl[s];
      u.g0 = geo.sb[s];
      u.n = geo.sb[s + 1] - u.g0;
      u.tail = geo.tail[s];
      u.h = rem >> 1;
      u.i = (rem & 1) ? u.n - 1 : 0;
      run_split4<T, MASKED>(a, u, lane, wave, park);
      continue;
    }
    const int item = b_lo + (k - g_cnt);
    const int s = upper_seq(geo.bu, a.batch, item);
    const int rem = item - geo.bu[s];
    u.g0 = geo.sb[s];
    u.n = geo.sb[s + 1] - u.g0;
    u.tail = geo.tail[s];
    const int per_head = bundles_per_head(u.n);
    u.h = rem / per_head;
    const int bundle = rem - u.h * per_head;
    const bool sparse = u.n >= RT_MIN_SPARSE_BLOCKS;
    u.i = (sparse ? 1 : 0) + 4 * bundle + wave;
    if (u.i <= (sparse ? u.n - 2 : u.n - 1)) run_solo<T, MASKED>(a, u, lane, stage);
  }
}

// Two persistent workgroups per CU, a multiple of 8 so that every XCD gets the same number.
unsigned plan_free_workgroups() {
  static unsigned cached = 0;
  if (cached == 0) {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
      cus = 256;
    cached = unsigned((2 * cus + 7) / 8 * 8);
  }
  return cached;
}

}  // namespace

namespace {

int launch_attention(const void* q, const void* q_rows, const void* q_bias, float q_scale, const void* k, const void* vt,
                     void* out, const int* seq_blocks_dev, const int* seq_tokens_dev, int batch, int total_blocks,
                     int heads, const int* to_idx, const int* to_pos, int plan_heads, const int* from_idx,
                     const int* from_pos, int n_wg, int dtype, void* stream) {
  RT_REQUIRE((q || (q_rows && q_bias)) && k && vt && out && seq_blocks_dev && to_idx && to_pos, RT_EINVAL, "NULL pointer");
  RT_REQUIRE(batch >= 1 && total_blocks >= batch && heads >= 1, RT_EINVAL, "bad geometry: batch=%d total_blocks=%d heads=%d",
             batch, total_blocks, heads);
  RT_REQUIRE(plan_heads == 1 || plan_heads == heads, RT_EINVAL, "plan_heads=%d must be 1 or heads=%d", plan_heads, heads);
  RT_REQUIRE((from_idx == nullptr) == (from_pos == nullptr), RT_EINVAL, "from_idx and from_pos go together");
  RT_REQUIRE(int64_t(total_blocks) * heads < (int64_t(1) << 31), RT_EINVAL, "too many units");
  RT_REQUIRE(batch <= MAX_BATCH, RT_EINVAL, "at most %d sequences per launch, got %d", MAX_BATCH, batch);
  RT_REQUIRE(((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(q_rows) | reinterpret_cast<uintptr_t>(q_bias) |
               reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(vt) | reinterpret_cast<uintptr_t>(out)) & 15u) == 0,
             RT_EINVAL, "q (or qkv and its bias), k, vt, out must be 16-byte aligned");
  if (dtype == RT_F32) return rt::fail(RT_ENOSYS, "block-sparse attention runs in fp16 or bf16 (fp32 accumulation)");
  RT_REQUIRE(dtype == RT_F16 || dtype == RT_BF16, RT_EINVAL, "unknown dtype %d", dtype);
  unsigned grid;
  if (from_idx) {
    RT_REQUIRE(n_wg >= 1, RT_EINVAL, "balanced launch needs n_wg >= 1, got %d", n_wg);
    grid = unsigned(n_wg);
  } else {
    grid = plan_free_workgroups();
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == RT_F16) {
    Args<_Float16> a{(const _Float16*)q, (const _Float16*)k, (const _Float16*)vt, (_Float16*)out, seq_blocks_dev, batch,
                     heads, total_blocks, to_idx, to_pos, plan_heads, from_idx, from_pos, seq_tokens_dev,
                     (const _Float16*)q_rows, (const _Float16*)q_bias, q_scale};
    if (seq_tokens_dev) hipLaunchKernelGGL((bs_attention_kernel<_Float16, true>), dim3(grid), dim3(256), 0, st, a);
    else hipLaunchKernelGGL((bs_attention_kernel<_Float16, false>), dim3(grid), dim3(256), 0, st, a);
  } else {
    Args<__bf16> a{(const __bf16*)q, (const __bf16*)k, (const __bf16*)vt, (__bf16*)out, seq_blocks_dev, batch, heads,
                   total_blocks, to_idx, to_pos, plan_heads, from_idx, from_pos, seq_tokens_dev,
                   (const __bf16*)q_rows, (const __bf16*)q_bias, q_scale};
    if (seq_tokens_dev) hipLaunchKernelGGL((bs_attention_kernel<__bf16, true>), dim3(grid), dim3(256), 0, st, a);
    else hipLaunchKernelGGL((bs_attention_kernel<__bf16, false>), dim3(grid), dim3(256), 0, st, a);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return rt::fail(RT_EIO, "bs_attention launch failed: %s", hipGetErrorString(e));
  return RT_OK;
}

}  // namespace

extern "C" int rt_bs_attention_fwd_masked(const void* q, const void* k, const void* vt, void* out,
                                          const int* seq_blocks_dev, const int* seq_tokens_dev, int batch,
                                          int total_blocks, int heads, const int* to_idx, const int* to_pos,
                                          int plan_heads, const int* from_idx, const int* from_pos, int n_wg,
                                          int dtype, void* stream) {
  RT_REQUIRE(q, RT_EINVAL, "NULL pointer");
  return launch_attention(q, nullptr, nullptr, 1.0f, k, vt, out, seq_blocks_dev, seq_tokens_dev, batch, total_blocks, heads,
                          to_idx, to_pos, plan_heads, from_idx, from_pos, n_wg, dtype, stream);
}

extern "C" int rt_bs_attention_fwd_qrows(const void* qkv, const void* qkv_bias, float q_scale, const void* k,
                                         const void* vt, void* out, const int* seq_blocks_dev,
                                         const int* seq_tokens_dev, int batch, int total_blocks, int heads,
                                         const int* to_idx, const int* to_pos, int plan_heads, const int* from_idx,
                                         const int* from_pos, int n_wg, int dtype, void* stream) {
  RT_REQUIRE(qkv && qkv_bias, RT_EINVAL, "NULL pointer");
  return launch_attention(nullptr, qkv, qkv_bias, q_scale, k, vt, out, seq_blocks_dev, seq_tokens_dev, batch, total_blocks,
                          heads, to_idx, to_pos, plan_heads, from_idx, from_pos, n_wg, dtype, stream);
}

extern "C" int rt_bs_attention_fwd(const void* q, const void* k, const void* vt, void* out, const int* seq_blocks_dev,
                                   int batch, int total_blocks, int heads, const int* to_idx, const int* to_pos,
                                   int plan_heads, const int* from_idx, const int* from_pos, int n_wg, int dtype,
                                   void* stream) {
  return rt_bs_attention_fwd_masked(q, k, vt, out, seq_blocks_dev, nullptr, batch, total_blocks, heads, to_idx, to_pos,
                                    plan_heads, from_idx, from_pos, n_wg, dtype, stream);
}
