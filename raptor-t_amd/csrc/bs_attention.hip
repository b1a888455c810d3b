// Block-sparse (BigBird-pattern) attention forward for gfx950, d = 64, 64-token blocks.
//
// Work unit = (sequence, head, from-block): 64 queries against the key blocks its CSR row
// lists (7/8 blocks for a sparse row, all n blocks for the two global rows).
//
// One wave owns all 64 queries of a unit and streams K / V^T tiles straight from global
// memory into MFMA operand registers: the QKV split kernel stores every 64x64 tile in
// "fragment order" (8 fragments of 64 lanes x 16 bytes), so each operand request is one fully
// coalesced 1 KiB buffer load and the tile loop needs no LDS and no barrier.
//
// MFMA formulation (v_mfma_f32_32x32x16_{f16,bf16}, fp32 accumulators):
//   S^T[key][query] = K[key][:] . Q[query][:]       A = K fragment,   B = Q fragment
//   O^T[d][query]  += V^T[d][key] . P^T[key][query]  A = V^T fragment, B = P (registers)
// Both products put the query on the accumulator column (lane & 31): max, sum and rescale
// factors are per-lane scalars and the S^T accumulators, after exp2, are the B operand of
// the second product, so P never leaves registers.  Softmax is evaluated in base 2 (q arrives
// pre-multiplied by log2(e)/sqrt(d)).
//
// Two tile loops:
//   pipelined (common path)  a (64 query x 64 key) tile is four 32x32 accumulator tiles
//       a = (key half, query half); step j issues, one matrix instruction per handful of
//       vector instructions, S^T(a[j+1]) and O^T += V^T P^T(a[j-1]) on the matrix pipe while
//       the vector pipe turns S^T(a[j]) into P^T(a[j]).  The reference maximum is fixed per row
//       (maximum over the row's first 32 keys, shared by a lane's two queries) and enters the
//       score product as the MFMA's C operand.  Nothing is tested inside the loop: a row whose
//       scores outgrow the reference shows up as a row sum that is not finite.
//   moving maximum (fallback) such rows, rows of more than 64 entries per wave and launches with
//       padded sequences are put aside and run afterwards by the loop that tracks the maximum
//       tile by tile.  The two loops never share a loop nest: the register allocator treats
//       them apart, and the pipelined one stays free of scratch-memory traffic.
//
// Schedule: persistent workgroups (two per CU) that draw work from ticket counters in device
// memory, one pair of counters per XCD (workgroups are dealt round-robin to the 8 XCDs, and each
// XCD has its own L2): XCD x owns the x-th eighth of the (head, row) items, so the K / V^T tiles
// of a (sequence, head) are fetched into one L2.
//   phase 1  global rows (the first and last block of a sparse sequence): one workgroup per row,
//            its 4 waves take every 4th key block and merge their softmax states through LDS;
//            the two rows of a (sequence, head) are consecutive tickets, so they stream the
//            same tiles at the same time;
//   phase 2  all other rows: every wave draws single units.  While it computes unit u it knows
//            unit u+1 (ticket, CSR row bounds and block ids through scalar loads), requests
//            u+1's first K / V^T tile in u's last tile steps and u+1's queries in the same
//            steps, and draws the ticket of unit u+2: a tile loop ahead while the queue is long,
//            only after the loop near its end (a wave never holds two waiting units then).
// With an LPT plan (from_idx / from_pos) n_wg workgroups walk their unit lists instead.
//
// Replaces, from the reference: layers/kernels/sparse_attention.cu:2953-3190 (balanced,
// persistent workgroups over the LPT plan), :2111-2403 (one workgroup per unit) and the
// dispatcher :3192-3228.
#include <hip/hip_runtime.h>

#include <mutex>
#include <type_traits>

#include "rt_launch.h"


namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef const int __attribute__((address_space(4))) const_int;   // loads through it are scalar loads

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
  // pipelined loop: two values of P rounded to nearest (a value beyond fp16's range must become
  // infinite: that is how the loop's caller learns that the row outgrew its reference), their sums
  // kept in packed halves
  static constexpr bool kPackedSum = true;
  __device__ static uint32_t two(float a, float b) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{a, b}, f16x2));
  }
  __device__ static uint32_t add(uint32_t a, uint32_t b) {
    return __builtin_bit_cast(uint32_t, __builtin_bit_cast(f16x2, a) + __builtin_bit_cast(f16x2, b));
  }
  __device__ static float fold(uint32_t a, float acc) {
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, a), f16x2{1, 1}, acc, false);
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
  static constexpr bool kPackedSum = false;
  __device__ static uint32_t two(float a, float b) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{a, b}, bf16x2));
  }
  __device__ static uint32_t add(uint32_t a, uint32_t) { return a; }
  __device__ static float fold(uint32_t, float acc) { return acc; }
};

// Moving-maximum loop: a row's reference maximum only moves when the 32 values P = 2^(score -
// reference) a lane holds for one key tile add up to more than 2^11 (no single P can then exceed
// 2^11, far inside fp16's range, and P keeps its full relative precision at any magnitude): the row
// sum the kernel needs anyway doubles as the overflow test.
constexpr float SUM_LIMIT = 2048.0f;
// Pipelined loop: the lane's two queries share one reference; if their own maxima over the first 32
// keys lie further apart than this (log2 units), the smaller row's P would sink towards fp16's
// denormals and the unit takes the moving-maximum loop instead.
constexpr float MAX_REFERENCE_GAP = 8.0f;

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

// Scores of padded keys become minus infinity: no weight.  s = 32 x 32 accumulator tile of key half kt; the key of
// element e in this lane is 32 kt + 8 (e >> 2) + (e & 3) + 4 (lane >> 5), padding from `tail` on.
__device__ inline void mask_padded(f32x16& s, int kt, int tail, int lane) {
  int lim = tail - 4 * (lane >> 5);
  asm volatile("" : "+v"(lim));       // the 16 comparisons are made here, not once per kernel and kept in 32 scalar pairs
#pragma unroll
  for (int e = 0; e < 16; ++e) s[e] = (32 * kt + 8 * (e >> 2) + (e & 3) >= lim) ? -INFINITY : s[e];
}

template <typename T>
__device__ inline void load_tile(const T* __restrict__ tile, int lane, typename Mma<T>::v8 (&f)[8]) {
  typedef typename Mma<T>::v8 v8;
#pragma unroll
  for (int i = 0; i < 8; ++i) f[i] = *reinterpret_cast<const v8*>(tile + i * 512 + lane * 8);
}

// Moving-maximum loop.  Streams key blocks row[first], row[first + step], ... of one (sequence,
// head) through the state.  kbase / vbase point at block 0 of that (sequence, head); n = blocks in
// the sequence.  The row's block ids are fetched 64 at a time into one register (lane j holds
// entry j) and handed out with v_readlane: one memory round trip per unit instead of one per key block.
template <typename T, bool MASKED>
__device__ inline void stream_tiles(const T* __restrict__ kbase, const T* __restrict__ vbase,
                                    const int* __restrict__ row, int first, int step, int cnt, int n, int tail, int nbv,
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
    // keys beyond the sequence's true length are padding and get no weight: the tail of block nbv - 1 is masked, a
    // block from nbv on is left out as a whole (its tile has been requested like any other and is dropped)
    const bool padded = MASKED && tail < 64 && bcur == nbv - 1;
    const bool skipped = MASKED && bcur >= nbv;
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
          mask_padded(sc[0], 0, tail, lane);
          mask_padded(sc[1], 1, tail, lane);
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
      bool redo = fresh && !skipped;
      if (!fresh && !skipped) {
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
      if (!skipped) {
        st.l[nt] += psum;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int s = 0; s < 4; ++s) st.o[t][nt] = Mma<T>::run(vf[t * 4 + s], pb[s], st.o[t][nt]);
      }
    }
    fresh = fresh && skipped;
    bcur = bn;
    __builtin_amdgcn_sched_barrier(0);
    load_tile<T>(vbase + int64_t(bn) * 4096, lane, vf);
    __builtin_amdgcn_sched_barrier(0);
  }
  }
}

// v_permlane32_swap: the upper 32 lanes of a change places with the lower 32 lanes of b.  Written as
// assembly: through the builtin, with both operands holding the same value, the compiler used the
// first result for both.  (s_nop: a vector instruction may just have written the operands.)
__device__ inline void swap_halves(unsigned& a, unsigned& b) {
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
}
// maximum / sum over lane l and lane l ^ 32, in both lanes
__device__ inline float pair_max(float x) {
  unsigned a = __builtin_bit_cast(unsigned, x), b = a;
  swap_halves(a, b);
  return fmaxf(__builtin_bit_cast(float, a), __builtin_bit_cast(float, b));
}
__device__ inline float pair_sum(float x) {
  unsigned a = __builtin_bit_cast(unsigned, x), b = a;
  swap_halves(a, b);
  return __builtin_bit_cast(float, a) + __builtin_bit_cast(float, b);
}

// Writes the wave's 64x64 output tile, O^T[d = 32t + 8*(e>>2) + 4*(lane>>5) + (e&3)]
// [query 32nt + (lane&31)] * w, to out[token][h*64 + d], through the wave's own LDS room (64 rows, OUT_PITCH bytes
// apart; no other wave touches it, and the LDS operations of one wave execute in order).  A lane holds 4
// consecutive d of its query per accumulator quad: every lane parks its 16 quads, then lane L takes the 16-byte
// chunk (L & 7) of tokens 8k + (L >> 3), so that a store instruction writes eight whole 128-byte lines.  Stores
// straight from the accumulators (lane pairs swapping quads) write 32 bytes to each of 32 lines per instruction,
// four pieces per line: same bits, 2-3 % more kernel time.
constexpr int OUT_PITCH = 144;
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
template <typename T>
__device__ inline void store_output(T* __restrict__ out_unit, int64_t row_stride, int lane, const State& st,
                                    const float (&w)[2], char* stage) {
  const int l32 = lane & 31, hi = lane >> 5;
#pragma unroll
  for (int nt = 0; nt < 2; ++nt) {
    char* row = stage + (32 * nt + l32) * OUT_PITCH + 8 * hi;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const uint32_t x0 = Mma<T>::two(st.o[t][nt][4 * q] * w[nt], st.o[t][nt][4 * q + 1] * w[nt]);
        const uint32_t x1 = Mma<T>::two(st.o[t][nt][4 * q + 2] * w[nt], st.o[t][nt][4 * q + 3] * w[nt]);
        *reinterpret_cast<u32x2*>(row + 64 * t + 16 * q) = u32x2{x0, x1};
      }
  }
  const char* rd = stage + (lane >> 3) * OUT_PITCH + (lane & 7) * 16;
  T* dst = out_unit + int64_t(lane >> 3) * row_stride + (lane & 7) * 8;
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const u32x4 v = *reinterpret_cast<const u32x4*>(rd + k * 8 * OUT_PITCH);
    *reinterpret_cast<u32x4*>(dst + int64_t(8 * k) * row_stride) = v;
  }
}

struct Unit {
  int h, i, n, g0;
  int tail;               // real tokens in the sequence's last block that holds any (64: none padded)
  int nbv;                // blocks of the sequence that hold real tokens (n without padding): blocks from nbv on are
                          // padding as a whole and get no weight as keys
};

// One unit's row of the to-block CSR, for the wave that runs it (all fields wave-uniform).
struct Row {
  Unit u;
  int p0, cnt;            // the row is to_idx[p0 .. p0 + cnt)
  int goff;               // byte offset of the unit's (sequence, head) group inside K and V^T
  int first_off;          // byte offset of the row's first tile inside K and V^T
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
  int* queues;                           // QUEUE_INTS ints of device memory, all zero when the kernel starts and when it ends
};

constexpr int MAX_BATCH = 1024;         // sequences per launch (geometry is kept in LDS)
constexpr int MAX_BLOCKS = 4096;        // 64-token blocks per launch (the row table is kept in LDS)
constexpr int MAX_HEADS_QROWS = 64;     // heads whose query bias fits the LDS copy
// Queue counters of one launch: 24 of them (tickets of the 8 global-row queues, tickets of the 8 unit
// queues, then per XCD the number of its workgroups that have finished), each alone in a 256-byte line:
// tickets of one line are served one after the other.  Every counter is only ever touched by the
// workgroups of one XCD, through atomics that its L2 executes; the last workgroup of an XCD to finish
// puts that XCD's three counters back to zero, so a launch leaves its counters as it found them.
constexpr int QUEUE_STRIDE = 64;                    // ints between two counters
constexpr int QUEUE_COUNTERS = 24;
constexpr int QUEUE_INTS = QUEUE_COUNTERS * QUEUE_STRIDE;
constexpr int REDO_SLOTS = 32;          // units a wave may put aside for the moving-maximum loop before it runs them
constexpr int REDO_ENTRIES = 2048;      // LPT plan: entries per workgroup whose pipelined attempt is tracked

// Geometry of the batch in LDS.
struct Geometry {
  int sb[MAX_BATCH + 1];                // prefix blocks
  uint32_t rows[MAX_BLOCKS];            // j-th row that is not a global row: sequence << 16 | block inside the sequence
  uint16_t sparse_seq[MAX_BATCH];       // k-th sequence that has global rows
  uint8_t tail[MAX_BATCH];              // real tokens in each sequence's last block that holds any (64 without padding)
  uint16_t nbv[MAX_BATCH];              // blocks of each sequence that hold real tokens
  int n_rows, n_sparse;
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

// ---------------------------------------------------------------------------------------------
// memory requests of the pipelined loop: raw buffer loads, one resource per array, the tile's
// byte offset in a scalar register and the fragment's in the instruction's immediate field
// ---------------------------------------------------------------------------------------------
template <typename T> struct Buffers {
  __amdgpu_buffer_rsrc_t k, v, q;
};

template <typename T>
__device__ inline typename Mma<T>::v8 fetch(__amdgpu_buffer_rsrc_t r, int voff, int soff) {
  return __builtin_bit_cast(typename Mma<T>::v8, __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 0));
}

// Where a unit's 64x64 query tile lies, as MFMA B fragments: fragment (nt, c) is a buffer load at
// vector offset voff, scalar offset soff + nt * nt_step + c * c_step.
struct QPlan { int voff, soff, nt_step, c_step; };
template <typename T>
__device__ inline QPlan q_plan(const Args<T>& a, const Unit& u, int lane) {
  QPlan q;
  if (a.q_rows) {
    // raw projection rows: request k = 4 nt + c takes the 128-byte head slices of queries 8k .. 8k + 7 whole,
    // eight lanes per query (eight cache lines per request; taking MFMA fragments straight from the rows
    // would touch 32 lines per request and return four times as slowly).  finish_q turns the eight
    // requests' registers into fragments through LDS.
    const int ld = a.heads * 384;                                   // bytes per token row of [T, 3 * heads * 64]
    q.voff = (lane >> 3) * ld + (lane & 7) * 16;
    q.soff = (u.g0 + u.i) * 64 * ld + u.h * 128;
    q.nt_step = 32 * ld;
    q.c_step = 8 * ld;
  } else {
    q.voff = lane * 16;
    q.soff = (u.g0 * a.heads + u.h * u.n + u.i) * 8192;
    q.nt_step = 4096;
    q.c_step = 1024;
  }
  return q;
}
template <typename T>
__device__ inline typename Mma<T>::v8 fetch_q(const Buffers<T>& b, const QPlan& q, int k) {   // k = 4 nt + c
  return fetch<T>(b.q, q.voff, q.soff + (k >> 2) * q.nt_step + (k & 3) * q.c_step);
}
template <typename T>
__device__ inline void request_q(const Args<T>& a, const Buffers<T>& b, const Unit& u, int lane,
                                 typename Mma<T>::v8 (&qf)[2][4]) {
  const QPlan q = q_plan<T>(a, u, lane);
#pragma unroll
  for (int k = 0; k < 8; ++k) qf[k >> 2][k & 3] = fetch_q<T>(b, q, k);
}

// What the queries-from-rows route keeps in LDS: a copy of the query bias and, per wave, room for one 64 x 64
// query tile in row order (rows Q_STAGE_PITCH bytes apart).
constexpr int Q_STAGE_PITCH = 144;
constexpr int Q_STAGE_BYTES = 64 * Q_STAGE_PITCH;
static_assert(OUT_PITCH == Q_STAGE_PITCH, "the output tile is parked in the room of the query tile");
template <typename T> struct QSide { const T* bias; char* stage; };

// Rows -> fragments through the wave's own LDS room (no other wave touches it: LDS operations of one wave
// execute in order), then (x + bias) * scale in fp32, rounded once: the arithmetic of the split kernel.
template <typename T>
__device__ inline void finish_q(const Args<T>& a, const QSide<T>& qs, const Unit& u, int lane,
                                typename Mma<T>::v8 (&qf)[2][4]) {
  typedef typename Mma<T>::v8 v8;
  if (!a.q_rows) return;
  const T* qbias = qs.bias;
  {
    char* wr = qs.stage + (lane >> 3) * Q_STAGE_PITCH + (lane & 7) * 16;
#pragma unroll
    for (int k = 0; k < 8; ++k) *reinterpret_cast<v8*>(wr + k * 8 * Q_STAGE_PITCH) = qf[k >> 2][k & 3];
    const char* rd = qs.stage + (lane & 31) * Q_STAGE_PITCH + (lane >> 5) * 16;
#pragma unroll
    for (int k = 0; k < 8; ++k) qf[k >> 2][k & 3] = *reinterpret_cast<const v8*>(rd + (k >> 2) * 32 * Q_STAGE_PITCH + (k & 3) * 32);
  }
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const v8 bb = *reinterpret_cast<const v8*>(qbias + u.h * 64 + c * 16 + (lane >> 5) * 8);
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        // pinned in fp32 before the rounding, as in the split kernel: multiply and rounding must not fuse
        float y = (float(qf[nt][c][e]) + float(bb[e])) * a.q_scale;
        asm volatile("" : "+v"(y));
        qf[nt][c][e] = static_cast<T>(y);
      }
  }
}

// lane j: byte offset inside K / V^T of the tile of the row's entry first + j * step (the first 64 of them)
template <typename T>
__device__ inline int row_offsets(const Args<T>& a, const Row& r, int first, int step, int lane) {
  const int e = first + lane * step;
  int blk = e < r.cnt ? a.to_idx[r.p0 + e] : 0;
  blk = blk < 0 ? 0 : (blk >= r.u.n ? r.u.n - 1 : blk);
  return r.goff + blk * 8192;
}

// CSR row bounds through scalar loads
template <typename T>
__device__ inline void describe_bounds(const Args<T>& a, const Unit& u, Row& r) {
  r.u = u;
  const int row = __builtin_amdgcn_readfirstlane((a.plan_heads > 1 ? u.h : 0) * a.nb_total + u.g0 + u.i);
  const_int* pos = (const_int*)(uintptr_t)(a.to_pos);
  r.p0 = pos[row];
  r.cnt = pos[row + 1] - r.p0;
  r.goff = (u.g0 * a.heads + u.h * u.n) * 8192;
}
// the row's first block, through a scalar load
template <typename T>
__device__ inline void describe_first(const Args<T>& a, Row& r) {
  const_int* idx = (const_int*)(uintptr_t)(a.to_idx);
  int blk = r.cnt > 0 ? idx[r.p0] : 0;
  blk = blk < 0 ? 0 : (blk >= r.u.n ? r.u.n - 1 : blk);
  r.first_off = r.goff + blk * 8192;
}

// A short row's block ids through scalar loads (they do not queue behind the tile requests, and
// what they return is not a pending vector load inside the tile loop): 16 entries starting at the
// row's first.  The caller has checked that p0 + 16 does not pass the end of to_idx.
constexpr int SHORT_ROW = 16;
typedef int i32x8 __attribute__((ext_vector_type(8), aligned(4)));
typedef const i32x8 __attribute__((address_space(4))) const_ids8;
template <typename T>
__device__ inline void request_short_row(const Args<T>& a, const Row& r, int (&blk)[SHORT_ROW]) {
  const_ids8* p = (const_ids8*)(uintptr_t)(a.to_idx + r.p0);
  const i32x8 lo = p[0], hi = p[1];
#pragma unroll
  for (int j = 0; j < 8; ++j) { blk[j] = lo[j]; blk[8 + j] = hi[j]; }
}
// lane j (< 16): byte offset inside K / V^T of the tile of the row's entry j
__device__ inline int short_row_offsets(const Row& r, const int (&blk)[SHORT_ROW], int lane) {
  int ids = 0;
#pragma unroll
  for (int j = 0; j < SHORT_ROW; ++j) {
    int bj = blk[j];
    bj = bj < 0 ? 0 : (bj >= r.u.n ? r.u.n - 1 : bj);
    ids = lane == j ? r.goff + bj * 8192 : ids;
  }
  return ids;
}

#define SB() __builtin_amdgcn_sched_barrier(0)

// The pipelined loop's registers.
template <typename T> struct Tiles {
  typename Mma<T>::v8 qf[2][4], kf[8], vf[8];
};

// first tile of a row, requested in the loop's own order: K's first key half, then the halves the
// loop's first step does not request itself (so the loop's waits, which count requests still in
// flight, come out the same on its first trip as on any other)
template <typename T>
__device__ inline void request_first(const Buffers<T>& b, int so, int lane, Tiles<T>& t) {
  const int vo = lane * 16;
#pragma unroll
  for (int f = 0; f < 4; ++f) t.kf[f] = fetch<T>(b.k, vo + f * 1024, so);
  SB();
#pragma unroll
  for (int f = 4; f < 8; ++f) t.kf[f] = fetch<T>(b.k, vo + f * 1024, so);
#pragma unroll
  for (int f = 0; f < 4; ++f) t.vf[(f & 1) + 4 * (f >> 1)] = fetch<T>(b.v, vo + ((f & 1) + 4 * (f >> 1)) * 1024, so);
  SB();
  // the loop's first step multiplies an all-zero P with V^T's second key half, which is only
  // requested after it: whatever those registers hold must be finite
#pragma unroll
  for (int f = 0; f < 4; ++f)
#pragma unroll
    for (int e = 0; e < 8; ++e) t.vf[(f & 1) + 2 + 4 * (f >> 1)][e] = static_cast<T>(0.f);
}

// Padding of a sequence, for the pipelined loop (MASKED kernels).  drop_off = byte offset (inside K / V^T) of the
// sequence's first block that is padding as a whole: tiles from there on are taken off the wave's tile list.
// pad_off = offset of the tile whose keys from `tail` on are padding, -1 if there is none.  The loop masks in its
// last tile only, so a row's padded tile is moved to the end of the list (the order of a row's tiles does not matter
// to the result beyond rounding; the reference comes from the first tile).
struct Padding { int pad_off, drop_off, tail; bool last; };
__device__ inline Padding padding_of(const Unit& u, int goff) {
  Padding pd;
  pd.pad_off = u.tail < 64 ? goff + (u.nbv - 1) * 8192 : -1;
  pd.drop_off = goff + u.nbv * 8192;
  pd.tail = u.tail;
  pd.last = false;
  return pd;
}
// Lanes 0 .. my-1 of ids hold the tile offsets of the wave's entries.  Takes the tiles that are padding as a whole
// off the list (my shrinks), moves the padded tile to the last lane in use and sets pd.last.  False: the pipelined
// loop cannot run this list (the padded tile is listed more than once, or the list's first tile does not stay
// first, which a hand-over from the previous row may already have requested).
__device__ inline bool pad_to_end(int& ids, int& my, int lane, Padding& pd) {
  pd.last = false;
  const unsigned long long listed = __ballot(lane < my);
  const unsigned long long keep = __ballot(lane < my && ids < pd.drop_off);
  if (keep != listed) {
    if (!(keep & 1ull)) return false;
    // kept entries move up in order; the dropped ones go behind them, lanes beyond the list stay (a permutation)
    const unsigned long long below = (1ull << lane) - 1ull;
    const int kept = __popcll(keep);
    const bool mine = (keep >> lane) & 1ull;
    const int dest = lane >= my ? lane : (mine ? __popcll(keep & below) : kept + __popcll(listed & ~keep & below));
    ids = __builtin_amdgcn_ds_permute(dest * 4, ids);
    my = kept;
  }
  if (pd.pad_off < 0) return true;
  const unsigned long long m = __ballot(lane < my && ids == pd.pad_off);
  if (m == 0) return true;
  if (__popcll(m) > 1) return false;
  const int jp = __builtin_ctzll(m);
  if (jp == 0 && my > 1) return false;
  if (jp != my - 1) {
    const int moved = __builtin_amdgcn_readlane(ids, my - 1);
    ids = lane == jp ? moved : (lane == my - 1 ? pd.pad_off : ids);
  }
  pd.last = true;
  return true;
}

// reference of the pipelined loop: maximum over the row's first 32 keys, shared by the lane's two
// queries.  False if the two queries' maxima lie too far apart.  pad_first (MASKED only): the row's first tile
// is the padded one, so keys from the tail on do not count (there is always at least one that does).
template <typename T, bool MASKED>
__device__ inline bool fast_reference(const Tiles<T>& t, float& mref, bool pad_first, int tail, int lane) {
  typedef Mma<T> P;
  f32x16 s0 = {}, s1 = {};
  if (MASKED && pad_first) {
    mask_padded(s0, 0, tail, lane);
    s1 = s0;
  }
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    s0 = P::run(t.kf[c], t.qf[0][c], s0);
    s1 = P::run(t.kf[c], t.qf[1][c], s1);
  }
  float m0 = s0[0], m1 = s1[0];
#pragma unroll
  for (int e = 1; e < 16; ++e) { m0 = fmaxf(m0, s0[e]); m1 = fmaxf(m1, s1[e]); }
  m0 = pair_max(m0);
  m1 = pair_max(m1);
  mref = fmaxf(m0, m1);
  return !__any(!(fabsf(m0 - m1) <= MAX_REFERENCE_GAP));           // false also for NaN / infinite scores
}

// The pipelined tile loop over `my` (1..64) tiles whose byte offsets sit in the lanes of `ids`; the
// first tile is in flight or there (request_first).  so_after >= 0: the last tile's steps request that
// tile (the first one of the wave's next row) instead of a dummy.  next_q(k), k = 0..7: requests
// fragment k of the next row's queries into t.qf; called in the last tile's last two steps, once
// the score products have read the fragment it replaces.
struct NoNextQ { __device__ void operator()(int) const {} };
template <typename T, bool MASKED, typename NextQ>
__device__ inline void fast_loop(const Buffers<T>& b, int ids, int my, const int& so_after, int lane, float mref,
                                 Tiles<T>& t, State& st, NextQ next_q, const Padding& pd) {
  typedef typename Mma<T>::v8 v8;
  typedef Mma<T> P;
  state_init(st);
  st.m[0] = st.m[1] = mref;
  f32x16 negm;                                        // the score products' C operand
#pragma unroll
  for (int e = 0; e < 16; ++e) negm[e] = -mref;
  int vo = lane * 16;
  auto ldk = [&](int f, int so) { t.kf[f] = fetch<T>(b.k, vo + f * 1024, so); };
  auto ldv = [&](int f, int so) { t.vf[f] = fetch<T>(b.v, vo + f * 1024, so); };
  f32x16 sc[2];
  v8 pb[2][2];
  float l0 = 0.f, l1 = 0.f;
  int so_cur = __builtin_amdgcn_readlane(ids, 0);
  // Everything requested so far must have arrived before the loop is entered (its first step needs
  // most of it anyway).  The waits inside the loop count the requests in flight; the compiler
  // derives them from the state at the loop's entry as well as from the loop's own requests, and
  // anything still pending there turns them into waits for all requests.
  __builtin_amdgcn_s_waitcnt(0x0F70);                 // vmcnt(0)
  // Inside the loop a wave yields to the other wave of its SIMD whenever that one is between two loops (queries,
  // reference, output, the next row's description): that code is a chain of short latencies, the loop always has
  // matrix work in flight.  Worth 2 % where rows are long (8 x 4096 tokens), nothing elsewhere.
  __builtin_amdgcn_s_setprio(0);
  SB();
  // pipeline prologue: scores of the first accumulator tile; an all-zero P for the first step's PV slot
  sc[0] = negm;
#pragma unroll
  for (int c = 0; c < 4; ++c) sc[0] = P::run(t.kf[c], t.qf[0][c], sc[0]);
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int e = 0; e < 8; ++e) pb[1][s][e] = static_cast<T>(0.f);

  // one tile: four steps; `last` (a std::bool_constant): the row's last tile
  auto tile = [&](int so_next, auto last) {
    constexpr bool LAST = decltype(last)::value;
    // keeps the fragment offsets inside the loop body, where they fold into the requests' immediate fields
    asm volatile("" : "+v"(vo));
#pragma unroll
    for (int S = 0; S < 4; ++S) {
      // consume sc[S & 1] (tile a[S]), produce sc[(S + 1) & 1] (a[S + 1]), multiply pb[(S + 1) & 1] (a[S - 1])
      const int nt = S & 1;
      const int ktn = ((S + 1) & 3) >> 1, ntn = (S + 1) & 1;          // a[S + 1]
      const int ktp = ((S + 3) & 3) >> 1, ntp = (S + 3) & 1;          // a[S - 1]
      f32x16& cur = sc[S & 1];
      f32x16& nxt = sc[(S + 1) & 1];
      v8 (&pprev)[2] = pb[(S + 1) & 1];
      float p[16];
      uint32_t w[8];
      uint32_t t01 = 0, t23 = 0, t45 = 0, t67 = 0;
      float lacc = 0.f;
      // a row's padded tile is its last one (pad_to_end): its scores lose the padded keys before they are exponentiated
      if (MASKED && LAST && pd.last) mask_padded(cur, S >> 1, pd.tail, lane);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        SB();
        // matrix slot
        if ((i & 1) == 0) {
          const int c = i >> 1;
          // the last tile's last step has no following scores to start: its slots request the next row's queries
          if (!(LAST && S == 3)) nxt = P::run(t.kf[ktn * 4 + c], t.qf[ntn][c], c == 0 ? negm : nxt);
        } else {
          const int tt = (i >> 1) & 1, s = i >> 2;
          st.o[tt][ntp] = P::run(t.vf[tt * 4 + 2 * ktp + s], pprev[s], st.o[tt][ntp]);
        }
        // tile requests: one per slot in the steps whose registers are free
        if (S == 1) { if (i < 4) ldk(i, so_next); else { const int f = (i & 1) + 2 + 4 * ((i >> 1) & 1); ldv(f, so_cur); } }
        if (S == 3) { if (i < 4) ldk(4 + i, so_next); else { const int f = (i & 1) + 4 * ((i >> 1) & 1); ldv(f, so_next); } }
        // the next row's queries: first query half after this row's last use of it (step 1), second after step 2's
        if (LAST && S == 2 && (i & 1) == 1) next_q(i >> 1);
        if (LAST && S == 3 && (i & 1) == 0) next_q(4 + (i >> 1));
        SB();
        // vector slot: two exponentials, rounding and sums of the previous slot's pair
        p[2 * i] = __builtin_amdgcn_exp2f(cur[2 * i]);
        p[2 * i + 1] = __builtin_amdgcn_exp2f(cur[2 * i + 1]);
        if (i > 0) {
          w[i - 1] = P::two(p[2 * i - 2], p[2 * i - 1]);
          if (!P::kPackedSum) lacc += p[2 * i - 2] + p[2 * i - 1];
        }
        if (P::kPackedSum) {
          if (i == 2) t01 = P::add(w[0], w[1]);
          if (i == 4) t23 = P::add(w[2], w[3]);
          if (i == 5) t01 = P::add(t01, t23);
          if (i == 6) t45 = P::add(w[4], w[5]);
          if (i == 7) t01 = P::add(t01, t45);
        }
      }
      SB();
      w[7] = P::two(p[14], p[15]);
      if (P::kPackedSum) {
        t67 = P::add(w[6], w[7]);
        t01 = P::add(t01, t67);
        if (nt == 0) l0 = P::fold(t01, l0); else l1 = P::fold(t01, l1);
      } else {
        lacc += p[14] + p[15];
        if (nt == 0) l0 += lacc; else l1 += lacc;
      }
      u32x4 lo = {w[0], w[1], w[2], w[3]}, up = {w[4], w[5], w[6], w[7]};
      pb[S & 1][0] = __builtin_bit_cast(v8, lo);
      pb[S & 1][1] = __builtin_bit_cast(v8, up);
      SB();
    }
  };

  for (int e = 0; e + 1 < my; ++e) {
    const int so_next = __builtin_amdgcn_readlane(ids, (e + 1) & 63);
    tile(so_next, std::false_type{});
    so_cur = so_next;
  }
  tile(so_after >= 0 ? so_after : so_cur, std::true_type{});
  // pipeline epilogue: the last tile's a[3] (second key half, second query half)
#pragma unroll
  for (int tt = 0; tt < 2; ++tt)
#pragma unroll
    for (int s = 0; s < 2; ++s) st.o[tt][1] = P::run(t.vf[tt * 4 + 2 + s], pb[1][s], st.o[tt][1]);
  st.l[0] = l0;
  st.l[1] = l1;
  __builtin_amdgcn_s_setprio(1);
}

__device__ inline bool sums_finite(const State& st) { return !__any(!(st.l[0] < INFINITY) || !(st.l[1] < INFINITY)); }

// moving-maximum loop on entries first, first + step, ... of row r
template <typename T, bool MASKED>
__device__ inline void slow_row(const Args<T>& a, const Buffers<T>& b, const QSide<T>& qbias, const Row& r, int first, int step,
                                int lane, bool have_q, typename Mma<T>::v8 (&qf)[2][4], State& st) {
  if (!have_q) {
    request_q<T>(a, b, r.u, lane, qf);
    finish_q<T>(a, qbias, r.u, lane, qf);
  }
  state_init(st);
  const int64_t gbase = int64_t(r.goff >> 1);
  stream_tiles<T, MASKED>(a.k + gbase, a.vt + gbase, a.to_idx + r.p0, first, step, r.cnt, r.u.n, r.u.tail, r.u.nbv, lane, qf, st);
}

// Entries first, first + step, ... of row r through the state with the pipelined loop, no hand-over
// from or to another row.  False: the row has to be run with the moving-maximum loop instead (more
// than 64 entries for this wave, or scores that outgrew the reference); the state is then undefined.
template <typename T, bool MASKED>
__device__ inline bool fast_row(const Args<T>& a, const Buffers<T>& b, const QSide<T>& qbias, const Row& r, int first, int step,
                                int lane, State& st) {
  Tiles<T> t;
  state_init(st);
  first = __builtin_amdgcn_readfirstlane(first);
  int my = __builtin_amdgcn_readfirstlane((r.cnt - first + step - 1) / step);           // this wave's entries
  if (my <= 0) return true;
  if (my > 64) return false;
  int ids = row_offsets<T>(a, r, first, step, lane);
  Padding pd = padding_of(r.u, r.goff);
  if (MASKED) {
    if (!pad_to_end(ids, my, lane, pd)) return false;
    if (my == 0) return true;                          // every tile of this wave's share is padding
  }
  request_q<T>(a, b, r.u, lane, t.qf);
  request_first<T>(b, __builtin_amdgcn_readlane(ids, 0), lane, t);
  finish_q<T>(a, qbias, r.u, lane, t.qf);
  float mref;
  if (!fast_reference<T, MASKED>(t, mref, pd.last && my == 1, pd.tail, lane)) return false;
  fast_loop<T, MASKED>(b, ids, my, -1, lane, mref, t, st, NoNextQ{}, pd);
  return sums_finite(st);
}

// normalises the state and writes the unit's output tile
template <typename T>
__device__ inline void finish_unit(const Args<T>& a, const QSide<T>& qs, const Unit& u, int lane, State& st) {
  float w[2];
#pragma unroll
  for (int nt = 0; nt < 2; ++nt) w[nt] = __builtin_amdgcn_rcpf(fmaxf(pair_sum(st.l[nt]), 1e-30f));
  const int64_t stride = int64_t(a.heads) * 64;
  store_output<T>(a.out + int64_t(u.g0 + u.i) * 64 * stride + u.h * 64, stride, lane, st, w, qs.stage);
}

template <typename T>
__device__ inline Row describe(const Args<T>& a, const Unit& u) {
  Row r;
  describe_bounds<T>(a, u, r);
  describe_first<T>(a, r);
  return r;
}

// One wave, one unit, all of its key blocks.  FAST: pipelined loop; false = the unit has to be run
// again with FAST = false (nothing was written).
template <typename T, bool MASKED, bool FAST>
__device__ inline bool run_solo(const Args<T>& a, const Buffers<T>& b, const QSide<T>& qbias, const Unit& u, int lane) {
  const Row r = describe<T>(a, u);
  State st;
  if (FAST) {
    if (!fast_row<T, MASKED>(a, b, qbias, r, 0, 1, lane, st)) return false;
  } else {
    typename Mma<T>::v8 qf[2][4];
    slow_row<T, MASKED>(a, b, qbias, r, 0, 1, lane, false, qf, st);
  }
  finish_unit<T>(a, qbias, u, lane, st);
  return true;
}

// Four waves, one unit: wave w streams key blocks w, w+4, ...; tree merge through LDS.  FAST:
// pipelined loop; false (the same in all four waves) = the unit has to be run again with FAST = false.
template <typename T, bool MASKED, bool FAST>
__device__ inline bool run_split4(const Args<T>& a, const Buffers<T>& b, const QSide<T>& qbias, const Unit& u, int lane,
                                  int wave, float* park) {
  const Row r = describe<T>(a, u);
  State st;
  if (FAST) {
    const bool ok = fast_row<T, MASKED>(a, b, qbias, r, wave, 4, lane, st);
    if (__syncthreads_or(!ok)) return false;          // also: the park is free (previous item is over)
  } else {
    typename Mma<T>::v8 qf[2][4];
    slow_row<T, MASKED>(a, b, qbias, r, wave, 4, lane, false, qf, st);
    __syncthreads();                                  // the park is free (previous item is over)
  }
#pragma unroll
  for (int nt = 0; nt < 2; ++nt) st.l[nt] = pair_sum(st.l[nt]);

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
    for (int nt = 0; nt < 2; ++nt) w[nt] = __builtin_amdgcn_rcpf(fmaxf(st.l[nt], 1e-30f));
    const int64_t stride = int64_t(a.heads) * 64;
    // wave 0's room is the start of the park, which it has just finished reading
    store_output<T>(a.out + int64_t(u.g0 + u.i) * 64 * stride + u.h * 64, stride, lane, st, w, qbias.stage);
  }
  __syncthreads();                                    // the park is read: the next item may stage its queries there
  return true;
}

// One ticket of a queue counter, in lane 0: a request, not yet waited for.  A buffer atomic whose
// resource covers just the counter: every lane executes it, lanes 1..63 address past the end and
// are dropped by the hardware, so no branch (and no wait at the end of one) surrounds the request.
__device__ inline __amdgpu_buffer_rsrc_t ticket_counter(int* p) { return __builtin_amdgcn_make_buffer_rsrc(p, 0, 4, 0x00020000); }
__device__ inline int request_ticket(__amdgpu_buffer_rsrc_t counter, int lane) {
  return __builtin_amdgcn_raw_ptr_buffer_atomic_add_i32(1, counter, lane * 4, 0, 1);
}
// the same instruction; if `really` (wave-uniform) is false all lanes address past the end: nothing is drawn
__device__ inline int request_ticket_if(__amdgpu_buffer_rsrc_t counter, int lane, bool really) {
  return __builtin_amdgcn_raw_ptr_buffer_atomic_add_i32(1, counter, lane * 4 + (really ? 0 : 4), 0, 1);
}

// Persistent workgroups (two per CU).
template <typename T, bool MASKED>
__global__ __launch_bounds__(256, 2) void bs_attention_kernel(Args<T> a) {
  // 36864 bytes with two uses that never overlap in time: two parked wave states (2 x 17408 bytes) of the merge
  // that ends a row shared by the four waves, and each wave's room for a query tile in row order (finish_q)
  static_assert(4 * Q_STAGE_BYTES >= 2 * 68 * 64 * int(sizeof(float)), "the park must hold two wave states");
  __shared__ __attribute__((aligned(16))) float park[4 * Q_STAGE_BYTES / 4];
  __shared__ Geometry geo;
  __shared__ __attribute__((aligned(16))) T qbias_lds[MAX_HEADS_QROWS * 64];
  __shared__ int s_item;
  __shared__ int redo[4][REDO_SLOTS];                 // per wave: units put aside for the moving-maximum loop
  __shared__ int redo_rows[REDO_SLOTS];               // per workgroup: global rows put aside
  __shared__ uint8_t s_redo[REDO_ENTRIES];            // LPT plan: entries of the workgroup's slice to run again
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const QSide<T> qbias{qbias_lds, reinterpret_cast<char*>(park) + wave * Q_STAGE_BYTES};

  // Geometry: prefix blocks, the sequences that have global rows, the list of rows that are not global rows.  Every
  // one of the 512 workgroups builds it for itself, so it is built by all 256 threads: sequence s's place in both
  // lists follows from the number of sparse sequences before it (a ballot per wave, the waves' counts through LDS),
  // since rows before s = blocks before s - 2 * (sparse sequences before s).
  int* const row_base = reinterpret_cast<int*>(park);            // per sequence: rows listed before it (scratch use of the park)
  int* const wave_sparse = row_base + MAX_BATCH;                 // [round][wave]: sparse sequences among the wave's 64
  for (int i = threadIdx.x; i <= a.batch; i += 256) geo.sb[i] = a.seq_blocks[i];
  if (a.q_rows)                                                  // without a bias (the rows carry it already): zeros
    for (int i = threadIdx.x; i < a.heads * 64; i += 256) qbias_lds[i] = a.q_bias ? a.q_bias[i] : static_cast<T>(0.f);
  __syncthreads();
  const int rounds = (a.batch + 255) >> 8;                       // at most MAX_BATCH / 256 = 4
  int before_in_wave[MAX_BATCH / 256];
  bool is_sparse[MAX_BATCH / 256];
#pragma unroll
  for (int r = 0; r < MAX_BATCH / 256; ++r) {
    before_in_wave[r] = 0;
    is_sparse[r] = false;
    if (r < rounds) {
      const int sq = r * 256 + int(threadIdx.x);
      is_sparse[r] = sq < a.batch && geo.sb[sq + 1] - geo.sb[sq] >= RT_MIN_SPARSE_BLOCKS;
      const unsigned long long votes = __ballot(is_sparse[r]);
      before_in_wave[r] = __popcll(votes & ((1ull << lane) - 1ull));
      if (lane == 0) wave_sparse[r * 4 + wave] = __popcll(votes);
      if (sq < a.batch) {
        const int nblk = geo.sb[sq + 1] - geo.sb[sq];
        int t = 64, nv = nblk;
        if (MASKED) {                                                // at least one real token, at most the sequence
          const int tokens = min(max(a.seq_tokens[sq], 1), 64 * nblk);
          nv = (tokens + 63) >> 6;
          t = tokens - 64 * (nv - 1);
        }
        geo.nbv[sq] = uint16_t(nv);
        geo.tail[sq] = uint8_t(t);
      }
    }
  }
  __syncthreads();
  {
    int running = 0;                                             // sparse sequences before this wave's 64 of round r
#pragma unroll
    for (int r = 0; r < MAX_BATCH / 256; ++r)
      if (r < rounds) {
        int before = running;
        for (int w = 0; w < 4; ++w) {
          const int c = wave_sparse[r * 4 + w];
          if (w < wave) before += c;
          running += c;
        }
        const int sq = r * 256 + int(threadIdx.x);
        if (sq < a.batch) {
          const int k = before + before_in_wave[r];
          row_base[sq] = geo.sb[sq] - 2 * k;
          if (is_sparse[r]) geo.sparse_seq[k] = uint16_t(sq);
        }
      }
    if (threadIdx.x == 0) {
      geo.n_sparse = running;
      geo.n_rows = geo.sb[a.batch] - 2 * running;
    }
  }
  __syncthreads();
  for (int sq = wave; sq < a.batch; sq += 4) {                   // a wave per sequence, a lane per row
    const int n = geo.sb[sq + 1] - geo.sb[sq];
    const int skip = n >= RT_MIN_SPARSE_BLOCKS ? 1 : 0;          // a sparse sequence's rows 0 and n - 1 are global rows
    for (int i = skip + lane; i < n - skip; i += 64) geo.rows[row_base[sq] + i - skip] = uint32_t(sq) << 16 | uint32_t(i);
  }
  __syncthreads();

  Buffers<T> b;
  {
    const uint32_t kv_bytes = uint32_t(a.nb_total) * uint32_t(a.heads) * 8192u;
    b.k = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(a.k), 0, kv_bytes, 0x00020000);
    b.v = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(a.vt), 0, kv_bytes, 0x00020000);
    b.q = a.q_rows ? __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(a.q_rows), 0, kv_bytes * 3u, 0x00020000)
                   : __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(a.q), 0, kv_bytes, 0x00020000);
  }

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
    u.nbv = MASKED ? int(geo.nbv[lo]) : u.n;
    const int rem = unit - u.g0 * a.heads;
    u.h = rem / u.n;
    u.i = rem - u.h * u.n;
    return u;
  };

  if (a.from_pos) {
    // LPT plan: global rows are shared by the workgroup's four waves, runs of up to four other units go
    // one per wave.  Two passes over the workgroup's slice: the pipelined loop first, then, for what
    // it handed back (s_redo: one flag per plan entry of the slice, at most REDO_ENTRIES), the
    // moving-maximum loop.
    // A plan the host has not checked (rt_meta_check_partition) must not make this kernel read outside
    // from_idx: the slice is clamped to its n_units entries, ids outside [0, n_units) are skipped.
    const int n_units = a.nb_total * a.heads;
    const int begin = min(max(a.from_pos[blockIdx.x], 0), n_units);
    const int end = min(max(a.from_pos[blockIdx.x + 1], begin), n_units);
    auto walk = [&](auto fast) {
      constexpr bool FAST = decltype(fast)::value;
      int p = begin;
      while (p < end) {
        // the next four plan entries in one round trip
        const int mine_id = (p + wave < end) ? a.from_idx[p + wave] : -1;
        int ids4[4];
#pragma unroll
        for (int w = 0; w < 4; ++w) ids4[w] = (p + w < end) ? a.from_idx[p + w] : -1;
        if (ids4[0] < 0 || ids4[0] >= n_units) { ++p; continue; }
        const Unit first = unit_of_flat(ids4[0]);
        const bool tracked = p - begin < REDO_ENTRIES;         // entries past the flags take the moving-maximum loop
        if (is_global_row(first)) {
          const bool todo = FAST ? tracked : (!tracked || s_redo[p - begin] != 0);
          if (todo) {
            const bool ok = run_split4<T, MASKED, FAST>(a, b, qbias, first, lane, wave, park);
            if (FAST && threadIdx.x == 0) s_redo[p - begin] = ok ? 0 : 1;
          }
          ++p;
          continue;
        }
        int run = 1;
        while (run < 4 && ids4[run] >= 0 && ids4[run] < n_units && !is_global_row(unit_of_flat(ids4[run]))) ++run;
        if (wave < run) {
          const int e = p + wave - begin;
          const bool trk = e < REDO_ENTRIES;
          const bool todo = FAST ? trk : (!trk || s_redo[e] != 0);
          if (todo) {
            const bool ok = run_solo<T, MASKED, FAST>(a, b, qbias, unit_of_flat(mine_id), lane);
            if (FAST && lane == 0) s_redo[e] = ok ? 0 : 1;
          }
        }
        p += run;
      }
    };
    walk(std::true_type{});
    __syncthreads();
    walk(std::false_type{});
    return;
  }

  const int xcd = blockIdx.x & 7;
  const __amdgpu_buffer_rsrc_t gq = ticket_counter(a.queues + xcd * QUEUE_STRIDE);          // this XCD's global-row queue
  const __amdgpu_buffer_rsrc_t uq = ticket_counter(a.queues + (8 + xcd) * QUEUE_STRIDE);    // this XCD's unit queue

  // phase 1: global rows, one per workgroup.  A pair = the first and the last row of one (sequence,
  // head): both stream the same K / V^T tiles, so they are consecutive tickets of the same XCD.
  // Pairs are numbered head-major and XCD x owns the x-th eighth of them: the same heads whose
  // other rows it runs in phase 2.
  {
    const int n_pairs = geo.n_sparse * a.heads;
    const int p_lo = int(int64_t(n_pairs) * xcd / 8), p_hi = int(int64_t(n_pairs) * (xcd + 1) / 8);
    const int n_glob = 2 * (p_hi - p_lo);             // tickets of this XCD that are rows
    auto unit_of_row = [&](int ticket) {
      const int pair = p_lo + (ticket >> 1);
      const int h = pair / geo.n_sparse;
      const int s = geo.sparse_seq[pair - h * geo.n_sparse];
      Unit u;
      u.g0 = geo.sb[s];
      u.n = geo.sb[s + 1] - u.g0;
      u.tail = geo.tail[s];
      u.nbv = MASKED ? int(geo.nbv[s]) : u.n;
      u.h = h;
      u.i = (ticket & 1) ? u.n - 1 : 0;
      return u;
    };
    // The XCD's workgroup number w takes row w without asking; rows beyond the XCD's workgroups are drawn from the
    // counter (ticket k = row wgs + k).  A batch with no more rows than workgroups touches no counter in this phase.
    const int wgs = int(gridDim.x >> 3), wg_local = int(blockIdx.x >> 3);
    const bool drawn_rows = n_glob > wgs;
    int item = wg_local < n_glob ? wg_local : -1;
    bool drained = item < 0 && !drawn_rows;
    while (!drained) {
      int n_rows_redo = 0;
      while (n_rows_redo < REDO_SLOTS) {
        if (item < 0) {
          if (!drawn_rows) { drained = true; break; }
          if (wave == 0) {
            const int k = __builtin_amdgcn_readfirstlane(request_ticket(gq, lane));
            if (lane == 0) s_item = k;
          }
          __syncthreads();
          item = wgs + s_item;
          __syncthreads();
          if (item >= n_glob) { drained = true; break; }
        }
        const bool ok = run_split4<T, MASKED, true>(a, b, qbias, unit_of_row(item), lane, wave, park);
        if (!ok) {
          if (threadIdx.x == 0) redo_rows[n_rows_redo] = item;
          ++n_rows_redo;
        }
        item = -1;
      }
      __syncthreads();
      for (int r = 0; r < n_rows_redo; ++r)
        run_split4<T, MASKED, false>(a, b, qbias, unit_of_row(redo_rows[r]), lane, wave, park);
      __syncthreads();
    }
  }

  // phase 2: all other rows; every wave draws single units.  Item = head * n_rows + j (j-th listed
  // row), XCD x owns the x-th eighth of the items.
  {
    const int lane_id = lane;
    const int n_rows = geo.n_rows;
    const int total = n_rows * a.heads;
    const int lo = int(int64_t(total) * xcd / 8), hi = int(int64_t(total) * (xcd + 1) / 8);
    const float inv_rows = 1.0f / float(n_rows > 0 ? n_rows : 1);
    auto unit_of = [&](int item) {
      int h = int((float(item) + 0.5f) * inv_rows);
      int j = item - h * n_rows;
      if (j < 0) { --h; j += n_rows; }
      if (j >= n_rows) { ++h; j -= n_rows; }
      const uint32_t e = geo.rows[j];
      const int s = int(e >> 16);
      Unit u;
      u.g0 = geo.sb[s];
      u.n = geo.sb[s + 1] - u.g0;
      u.tail = geo.tail[s];
      u.nbv = MASKED ? int(geo.nbv[s]) : u.n;
      u.h = h;
      u.i = int(e & 0xffffu);
      return u;
    };
    auto item_of = [&](int ticket) {                  // -1: the queue is drained
      const int k = __builtin_amdgcn_readfirstlane(ticket);
      return lo + k < hi ? lo + k : -1;
    };
    const_int* pos_all = (const_int*)(uintptr_t)(a.to_pos);
    const int idx_total = pos_all[a.plan_heads * a.nb_total];       // entries in to_idx
    int n_redo = 0;
    int item = item_of(request_ticket(uq, lane));
    int item_nx = item >= 0 ? item_of(request_ticket(uq, lane)) : -1;
    while (item >= 0 || n_redo > 0) {
      // pipelined loop on one unit after the other, each handing the next one its first tile.  A wave
      // holds the unit it runs and the next one; the one after that is drawn when the tile loop ends.
      if (item >= 0) {
        Tiles<T> t;
        Row cur;
        int blk[SHORT_ROW];
        describe_bounds<T>(a, unit_of(item), cur);
        bool cur_short = cur.cnt >= 1 && cur.cnt <= SHORT_ROW && cur.p0 + SHORT_ROW <= idx_total;
        int ids = 0;
        cur.first_off = 0;
        if (cur_short) {
          request_short_row<T>(a, cur, blk);
          ids = short_row_offsets(cur, blk, lane_id);
          cur.first_off = __builtin_amdgcn_readlane(ids, 0);
        }
        bool primed = false;
        while (item >= 0 && n_redo < REDO_SLOTS) {
          // what the code below derives from the lane number is derived again for every unit, not
          // kept in registers across the tile loop
          int lane = lane_id;
          asm volatile("" : "+v"(lane));
          const bool has_next = item_nx >= 0;
          Row nx = cur;
          if (has_next) describe_bounds<T>(a, unit_of(item_nx), nx);        // scalar loads, waited for below
          State st;
          bool ok = cur_short;
          float mref = 0.f;
          Padding pd = padding_of(cur.u, cur.goff);
          int my = cur.cnt;                                 // tiles of the row that the loop runs
          if (MASKED && ok) ok = pad_to_end(ids, my, lane, pd);
          if (ok && !primed) {
            request_q<T>(a, b, cur.u, lane, t.qf);
            request_first<T>(b, cur.first_off, lane, t);
          }
          if (ok) {
            finish_q<T>(a, qbias, cur.u, lane, t.qf);
            ok = fast_reference<T, MASKED>(t, mref, pd.last && my == 1, pd.tail, lane);
          }
          // the next row's block ids: requested here, looked at in the loop's last tile
          bool nx_short = false;
          nx.first_off = -1;
          if (has_next) {
            nx_short = nx.cnt >= 1 && nx.cnt <= SHORT_ROW && nx.p0 + SHORT_ROW <= idx_total;
            if (nx_short) {
              request_short_row<T>(a, nx, blk);
              int b0 = blk[0];
              b0 = b0 < 0 ? 0 : (b0 >= nx.u.n ? nx.u.n - 1 : b0);
              nx.first_off = nx.goff + b0 * 8192;
            }
          }
          int item_after = -1;
          primed = false;
          if (ok) {
            const QPlan qn = q_plan<T>(a, nx.u, lane);      // without a next unit: this unit's queries again
            fast_loop<T, MASKED>(b, ids, my, nx.first_off, lane, mref, t, st,
                                 [&](int k) { t.qf[k >> 2][k & 3] = fetch_q<T>(b, qn, k); }, pd);
            lane = lane_id;
            asm volatile("" : "+v"(lane));
            // The unit after the next one: its ticket is drawn here, behind the tile loop, and looked at once this
            // unit's output is on its way.  (Drawn ahead of the loop, the request was still in flight at the loop's
            // entry, where everything requested must have arrived: a device round trip of waiting per unit.)  The
            // request is always issued (without a next unit it addresses nothing): no branch around it.
            const int t_next = request_ticket_if(uq, lane, has_next);
            SB();
            primed = nx_short;
            if (sums_finite(st)) {
              finish_unit<T>(a, qbias, cur.u, lane, st);
              SB();
            } else {
              if (lane == 0) redo[wave][n_redo] = item;
              ++n_redo;
            }
            item_after = has_next ? item_of(t_next) : -1;
          } else {
            if (lane == 0) redo[wave][n_redo] = item;
            ++n_redo;
            const int t_next = request_ticket_if(uq, lane, has_next);
            item_after = has_next ? item_of(t_next) : -1;
          }
          item = item_nx;
          item_nx = item_after;
          cur = nx;
          cur_short = nx_short;
          if (nx_short) ids = short_row_offsets(nx, blk, lane);
        }
      }
      // the units put aside: moving-maximum loop
      for (int r = 0; r < n_redo; ++r) {
        const int it = __builtin_amdgcn_readfirstlane(redo[wave][r]);
        run_solo<T, MASKED, false>(a, b, qbias, unit_of(it), lane_id);
      }
      n_redo = 0;
    }
  }

  // This workgroup draws no more tickets.  The last workgroup of the XCD to get here puts the XCD's counters
  // back to zero for the next launch that is handed them (same L2, same kind of access as the tickets).
  __syncthreads();
  if (wave == 0) {
    const __amdgpu_buffer_rsrc_t done = ticket_counter(a.queues + (16 + xcd) * QUEUE_STRIDE);
    const int finished = __builtin_amdgcn_readfirstlane(request_ticket(done, lane));
    if (finished == int(gridDim.x >> 3) - 1) {
      // nobody else touches them any more: read each (an addition of nothing) and take that much away
      const int g = __builtin_amdgcn_raw_ptr_buffer_atomic_add_i32(0, gq, lane * 4, 0, 1);
      const int u = __builtin_amdgcn_raw_ptr_buffer_atomic_add_i32(0, uq, lane * 4, 0, 1);
      (void)__builtin_amdgcn_raw_ptr_buffer_atomic_add_i32(-g, gq, lane * 4, 0, 0);
      (void)__builtin_amdgcn_raw_ptr_buffer_atomic_add_i32(-u, uq, lane * 4, 0, 0);
      (void)__builtin_amdgcn_raw_ptr_buffer_atomic_add_i32(-(finished + 1), done, lane * 4, 0, 0);
    }
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

// Queue counters of the library's own launches: a ring of slots, so that launches which overlap on
// different streams do not share counters.  A launch leaves its slot zeroed (the kernel's last
// workgroups do that), so the slots need no order among the launches that use them; what the ring cannot
// cover is more than QUEUE_SLOTS attention launches of the library in flight on one device at the same time.
constexpr int QUEUE_SLOTS = 64;
int* library_queues(int* err) {
  static int* base[64] = {};
  static unsigned next[64] = {};
  static std::mutex mu;
  int dev = 0;
  *err = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) { *err = 1; return nullptr; }
  std::lock_guard<std::mutex> lock(mu);
  if (!base[dev]) {
    int* p = nullptr;
    if (hipMalloc(&p, sizeof(int) * QUEUE_INTS * QUEUE_SLOTS) != hipSuccess) { *err = 2; return nullptr; }
    if (hipMemset(p, 0, sizeof(int) * QUEUE_INTS * QUEUE_SLOTS) != hipSuccess) { *err = 3; return nullptr; }
    base[dev] = p;
  }
  const unsigned slot = next[dev]++ % QUEUE_SLOTS;
  return base[dev] + slot * QUEUE_INTS;
}

}  // namespace

namespace {

int launch_attention(const void* q, const void* q_rows, const void* q_bias, float q_scale, const void* k, const void* vt,
                     void* out, const int* seq_blocks_dev, const int* seq_tokens_dev, int batch, int total_blocks,
                     int heads, const int* to_idx, const int* to_pos, int plan_heads, const int* from_idx,
                     const int* from_pos, int n_wg, int dtype, void* stream, int* own_queues = nullptr) {
  RT_REQUIRE((q || q_rows) && k && vt && out && seq_blocks_dev && to_idx && to_pos, RT_EINVAL, "NULL pointer");
  RT_REQUIRE(batch >= 1 && total_blocks >= batch && heads >= 1, RT_EINVAL, "bad geometry: batch=%d total_blocks=%d heads=%d",
             batch, total_blocks, heads);
  RT_REQUIRE(plan_heads == 1 || plan_heads == heads, RT_EINVAL, "plan_heads=%d must be 1 or heads=%d", plan_heads, heads);
  RT_REQUIRE((from_idx == nullptr) == (from_pos == nullptr), RT_EINVAL, "from_idx and from_pos go together");
  RT_REQUIRE(int64_t(total_blocks) * heads * 8192 * 3 < (int64_t(1) << 31), RT_EINVAL,
             "batch too large: %d blocks x %d heads (byte offsets are 32-bit)", total_blocks, heads);
  RT_REQUIRE(batch <= MAX_BATCH, RT_EINVAL, "at most %d sequences per launch, got %d", MAX_BATCH, batch);
  RT_REQUIRE(total_blocks <= MAX_BLOCKS, RT_EINVAL, "at most %d blocks (%d tokens) per launch, got %d blocks", MAX_BLOCKS,
             MAX_BLOCKS * 64, total_blocks);
  RT_REQUIRE(!q_rows || heads <= MAX_HEADS_QROWS, RT_EINVAL, "queries from the projection rows: at most %d heads, got %d",
             MAX_HEADS_QROWS, heads);
  RT_REQUIRE(((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(q_rows) | reinterpret_cast<uintptr_t>(q_bias) |
               reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(vt) | reinterpret_cast<uintptr_t>(out)) & 15u) == 0,
             RT_EINVAL, "q (or qkv and its bias), k, vt, out must be 16-byte aligned");
  RT_REQUIRE(dtype == RT_F16 || dtype == RT_BF16 || dtype == RT_F32, RT_EINVAL, "unknown dtype %d", dtype);
  if (dtype == RT_F32) {
    RT_REQUIRE(!from_idx || n_wg >= 1, RT_EINVAL, "balanced launch needs n_wg >= 1, got %d", n_wg);
    return rt::launch_attention_f32(q, q_rows, q_bias, q_scale, k, vt, out, seq_blocks_dev, seq_tokens_dev, batch,
                                    total_blocks, heads, to_idx, to_pos, plan_heads, from_idx, from_pos, n_wg, stream);
  }
  unsigned grid;
  int* queues = nullptr;
  if (from_idx) {
    RT_REQUIRE(n_wg >= 1, RT_EINVAL, "balanced launch needs n_wg >= 1, got %d", n_wg);
    grid = unsigned(n_wg);
  } else {
    grid = plan_free_workgroups();
    if (own_queues) {
      queues = own_queues;
    } else {
      int err = 0;
      queues = library_queues(&err);
      if (!queues) return rt::fail(RT_ENOMEM, "no device memory for the work queues (step %d)", err);
    }
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == RT_F16) {
    Args<_Float16> a{(const _Float16*)q, (const _Float16*)k, (const _Float16*)vt, (_Float16*)out, seq_blocks_dev, batch,
                     heads, total_blocks, to_idx, to_pos, plan_heads, from_idx, from_pos, seq_tokens_dev,
                     (const _Float16*)q_rows, (const _Float16*)q_bias, q_scale, queues};
    if (seq_tokens_dev) RT_LAUNCH((bs_attention_kernel<_Float16, true>), dim3(grid), dim3(256), 0, st, a);
    else RT_LAUNCH((bs_attention_kernel<_Float16, false>), dim3(grid), dim3(256), 0, st, a);
  } else {
    Args<__bf16> a{(const __bf16*)q, (const __bf16*)k, (const __bf16*)vt, (__bf16*)out, seq_blocks_dev, batch, heads,
                   total_blocks, to_idx, to_pos, plan_heads, from_idx, from_pos, seq_tokens_dev,
                   (const __bf16*)q_rows, (const __bf16*)q_bias, q_scale, queues};
    if (seq_tokens_dev) RT_LAUNCH((bs_attention_kernel<__bf16, true>), dim3(grid), dim3(256), 0, st, a);
    else RT_LAUNCH((bs_attention_kernel<__bf16, false>), dim3(grid), dim3(256), 0, st, a);
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
  RT_REQUIRE(qkv, RT_EINVAL, "NULL pointer");             // qkv_bias may be NULL: the rows carry the bias already
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

// ---- the entry point that allocates nothing -------------------------------------------------------
// Its queue counters live in this array instead of the library's allocated ring, zeroed by a fill kernel
// ahead of every launch (whatever an earlier launch that was cut short may have left there).  In host code
// the array's name is only a stand-in: its address on a device comes from hipGetSymbolAddress, once per device.
constexpr int NO_ALLOC_SCRATCH_INTS = RT_NO_ALLOC_SCRATCH_BYTES / int(sizeof(int));
static_assert(NO_ALLOC_SCRATCH_INTS >= QUEUE_INTS, "the scratch array must hold one launch's counters");
static_assert(RT_NO_ALLOC_MAX_BATCH <= MAX_BATCH && RT_NO_ALLOC_MAX_BLOCKS <= MAX_BLOCKS, "header limits exceed the kernel's");
static __device__ __align__(256) int scratch[NO_ALLOC_SCRATCH_INTS];

namespace {

__global__ void clear_queue_counters(int* counters) { counters[threadIdx.x * QUEUE_STRIDE] = 0; }

int* no_alloc_scratch() {
  static int* ptr[64] = {};
  static std::mutex mu;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
  std::lock_guard<std::mutex> lock(mu);
  if (!ptr[dev]) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return nullptr;
    ptr[dev] = static_cast<int*>(p);
  }
  return ptr[dev];
}

}  // namespace

extern "C" int rt_bs_attention_fwd_no_alloc(const void* q, const void* k, const void* vt, void* out,
                                            const int* seq_blocks_dev, const int* seq_tokens_dev, int batch,
                                            int total_blocks, int heads, const int* to_idx, const int* to_pos,
                                            int plan_heads, int dtype, void* stream) {
  RT_REQUIRE(q, RT_EINVAL, "NULL pointer");
  RT_REQUIRE(batch >= 1 && batch <= RT_NO_ALLOC_MAX_BATCH && total_blocks >= batch && total_blocks <= RT_NO_ALLOC_MAX_BLOCKS,
             RT_EINVAL, "rt_bs_attention_fwd_no_alloc takes at most %d sequences and %d blocks (%d tokens), got %d and %d",
             RT_NO_ALLOC_MAX_BATCH, RT_NO_ALLOC_MAX_BLOCKS, RT_NO_ALLOC_MAX_BLOCKS * 64, batch, total_blocks);
  int* counters = no_alloc_scratch();
  if (!counters) return rt::fail(RT_EIO, "the address of the static scratch array is not available on this device");
  hipLaunchKernelGGL(clear_queue_counters, dim3(1), dim3(QUEUE_COUNTERS), 0, static_cast<hipStream_t>(stream), counters);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return rt::fail(RT_EIO, "clearing the queue counters failed: %s", hipGetErrorString(e));
  return launch_attention(q, nullptr, nullptr, 1.0f, k, vt, out, seq_blocks_dev, seq_tokens_dev, batch, total_blocks, heads,
                          to_idx, to_pos, plan_heads, nullptr, nullptr, 0, dtype, stream, counters);
}
