/*
 * raptor_t_hip.h -- C ABI of the MI355X (gfx950) block-sparse encoder-layer library.
 *
 * Drop-in boundary for the hot path of Raptor-T: these are the entry points the
 * reference's C++ layer functors reach through `layers/kernels/kernel.h` and
 * `layers/kernels/mat_mul.h`, plus the host metadata the reference builds in
 * `layers/multi_headed_attention.cpp` and `python/util.py`.  Plain pointers and sizes
 * only; no torch types, no exceptions, no exit().
 *
 * Conventions
 *   - every function returns 0 on success or a negative errno-style code; a text for
 *     the calling thread's last failure is available from rt_last_error_string();
 *   - device pointers are borrowed (never freed here) and must belong to the current
 *     HIP device; `stream` is a hipStream_t passed as void* (NULL = default stream);
 *   - `dtype` is an rt_dtype; fp16/bf16 kernels accumulate and normalise in fp32;
 *   - a packed batch of B sequences is described by `seq_blocks` (B+1 ints): prefix
 *     sums of the per-sequence counts of 64-token blocks (`seq_len_info` of
 *     python/util.py:37,45); NB = seq_blocks[B], T = 64 * NB tokens.
 *
 * Head-major packed layout (produced by rt_qkv_bias_split, consumed by
 * rt_bs_attention_fwd): for sequence s (n blocks, first global block g0) and head h the
 * 64x64 tiles of blocks 0..n-1 start at element (g0*H + h*n) * 4096.  A tile is stored in
 * MFMA "fragment order": 8 fragments of 64 lanes x 8 elements; element e of lane l of
 * fragment f is
 *     Q, K :  tile[32*(f>>2) + (l&31)][16*(f&3) + 8*(l>>5) + e]         (row = token, col = d)
 *     V    :  tile[token(16*(f&3) + 8*(l>>5) + e)][32*(f>>2) + (l&31)]  (transposed; token()
 *             swaps bits 2 and 3 of the slot index, the order in which a 32x32 MFMA
 *             accumulator hands P back as the next MFMA's operand)
 * so that every operand load of the attention kernel is one coalesced 16-byte-per-lane
 * request.  rt_unpack_head_tiles undoes the layout for inspection.
 */
#ifndef RAPTOR_T_HIP_H
#define RAPTOR_T_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RT_BLOCK 64           /* tokens per block (bert_attention.h:39) */
#define RT_HEAD_DIM 64        /* the attention kernel is specialised for d = 64 */
#define RT_NUM_RAND 3         /* random blocks per row (multi_headed_attention.cpp:27) */
#define RT_MIN_SPARSE_BLOCKS 12  /* below this a sequence runs full attention
                                    (python/modeling_big_bird.py:2079-2094) */

typedef enum { RT_F16 = 0, RT_BF16 = 1, RT_F32 = 2 } rt_dtype;

enum {
  RT_OK = 0,
  RT_EINVAL = -22,   /* bad argument / shape the kernels do not support */
  RT_ENOMEM = -12,   /* output capacity too small or allocation failed */
  RT_EIO = -5,       /* a HIP / hipBLASLt call failed */
  RT_ENOSYS = -38,   /* combination not implemented */
  RT_ECANCELED = -125 /* pipeline was terminated */
};

/* plan modes of rt_meta_build_to_index / rt_pipeline_create */
enum {
  RT_PLAN_HF = 0,         /* per-head plan of the reference's oracle, numpy-RNG exact,
                             seed = layer index (python/modeling_big_bird.py:573-597) */
  RT_PLAN_REFERENCE = 1,  /* head-shared plan with the row rules of
                             layers/multi_headed_attention.cpp:44-125, seeded */
  RT_PLAN_EXPLICIT = 2    /* caller supplies rand_attn */
};
/* plan policies (which lengths use the truncated max-length generator) */
enum { RT_POLICY_REFERENCE_PATCHED = 0, RT_POLICY_HF_UPSTREAM = 1 };

const char* rt_last_error_string(void);
int rt_abi_version(void);

/* Timing of one kernel by its own dispatch.  The reference times a launcher with the host clock around the
 * launch (layers/kernels/add_bias_act.cu:109-131, the `info` map of every launcher); a pair of events recorded
 * around a launch also counts the gaps to the neighbouring kernels.  After this call the next kernel that one
 * of this library's kernel entry points (every one below except the vendor GEMMs; each launches one kernel,
 * rt_bs_attention_fwd_no_alloc a small clearing kernel before it that does not count) launches from the calling
 * thread writes the start and end timestamps of its dispatch into the two hipEvent_t (created by the caller,
 * either may be NULL); hipEventElapsedTime between them is the kernel's duration as a profiler reports it.
 * One launch consumes the pair; (NULL, NULL) withdraws a pair no launch has taken.  Returns 1 if the call
 * replaced or withdrew a pair that was still waiting for a launch, 0 otherwise.  Not for use while a stream
 * is being captured into a graph. */
int rt_time_next_launch(void* start_event, void* stop_event);

/* ------------------------------------------------------------------ host metadata */

/* numpy.random.seed(seed) followed by `count` calls of numpy.random.permutation(n_i):
 * writes the permutations of arange(n_i) back to back.  Exposes the RNG the plans are
 * drawn with so that it can be checked against numpy itself. */
int rt_meta_np_permutations(uint32_t seed, const int* n, int count, int* out);

/* Prefix block counts of a batch: replaces the first half of `generate_data_metainfo`
 * (python/util.py:36-37,45).  seq_lens in tokens, each a positive multiple of 64. */
int rt_meta_seq_prefix_blocks(const int* seq_lens, int batch, int* out_seq_blocks);

/* rand_attn[heads][n-2][3] for one sequence of `length` tokens, seed = layer index:
 * replaces python/modeling_big_bird.py:573-597 with :1039-1314. */
int rt_meta_rand_attn(int length, uint32_t seed, int heads, int max_pos, int policy, int* out);

/* The plans rt_meta_rand_attn / rt_meta_build_to_index (RT_PLAN_HF) draw are pure functions of (length, seed, heads,
 * max_pos, policy); the library keeps the ones it has drawn in a memo table (the oracle's own code,
 * python/modeling_big_bird.py:573-597, draws them again for every forward pass: 2 ms per layer of a 16-sequence
 * batch, which a worker thread otherwise spends per batch).  max_bytes >= 0 sets the table's bound (0: keep
 * nothing, and forget what is kept; default 64 MiB), max_bytes < 0 leaves it; hits / misses (may be NULL) receive
 * the look-up counts so far.  No counterpart in the reference. */
int rt_meta_set_plan_cache(int64_t max_bytes, int64_t* hits, int64_t* misses);

/* Sizes of the CSR that rt_meta_build_to_index will write. */
int rt_meta_to_index_size(const int* seq_blocks, int batch, int plan_heads,
                          int64_t* idx_len, int64_t* pos_len);

/* BigBird to-block CSR of a packed batch: replaces
 * MultiHeadedAttention::GenerateSparseBlockIndex (layers/multi_headed_attention.cpp:15-140).
 * Row `hp * NB + g` (plan head hp, global from-block g) lists block ids local to g's
 * sequence; duplicates are kept.  mode RT_PLAN_HF: plan_heads = heads, rand_attn NULL;
 * RT_PLAN_REFERENCE: plan_heads = 1; RT_PLAN_EXPLICIT: rand_attn holds, sequence after
 * sequence (sequences below 12 blocks contribute nothing), [plan_heads][n_s-2][3]. */
int rt_meta_build_to_index(const int* seq_blocks, int batch, int plan_heads, int mode,
                           uint32_t seed, int max_pos, int policy, const int* rand_attn,
                           int* out_idx, int64_t idx_cap, int* out_pos, int64_t pos_cap);

/* Per from-block cost [n,7,8..8,7,n] and total: python/util.py:38-46. */
int rt_meta_block_costs(const int* seq_blocks, int batch, int* out_costs, int64_t* total);

/* LPT work plan: replaces generate_parition_plan (python/util.py:11-34).
 * out_pos[n_wg+1], out_ids[heads*NB]; unit id = blk + head*n_s + seq_start*heads. */
int rt_meta_partition_lpt(const int* seq_blocks, int batch, int heads, int n_wg,
                          int* out_pos, int* out_ids);

/* Host-side check of a work plan before it is handed to a balanced attention launch (no counterpart in
 * the reference, whose kernel trusts python/util.py:11-34): from_pos[n_wg+1] runs from 0 to
 * total_blocks*heads without decreasing and from_idx lists every unit id exactly once.  RT_EINVAL otherwise.
 * The attention kernel itself skips an id outside the range (its rows stay unwritten) rather than fault;
 * a caller that builds plans of its own calls this first. */
int rt_meta_check_partition(const int* from_pos, const int* from_idx, int n_wg, int total_blocks, int heads);

/* Host-side check of a to-block index before it is handed to an attention launch (no counterpart in the
 * reference, whose kernels trust layers/multi_headed_attention.cpp:15-140): to_pos[plan_heads*NB+1] starts at 0,
 * never decreases, leaves no row empty and ends inside to_idx[idx_len]; every entry of the row of (plan head,
 * sequence s, block i) names a block of sequence s, 0 .. n_s-1.  RT_EINVAL otherwise.  The attention kernels clamp
 * a block id they are handed, so a bad entry reads the wrong tile rather than fault; row bounds they take as given. */
int rt_meta_check_to_index(const int* to_idx, const int* to_pos, int64_t idx_len, const int* seq_blocks, int batch,
                           int plan_heads);

/* --------------------------------------------------------------------- GPU kernels */

/* Replaces kernels::add_bias_and_transpose_kernel (layers/kernels/
 * add_bias_and_transpose.cu:212-233): qkv[T, 3*H*64] token-major + bias[3*H*64] ->
 * q (scaled by q_scale), k, vt in the head-major packed layout.  For rt_bs_attention_fwd
 * q_scale must be log2(e)/sqrt(64): the attention kernel evaluates the softmax in base 2.
 * q may be NULL: Q is then not written (a third less traffic), for rt_bs_attention_fwd_qrows,
 * which takes its queries from `qkv` itself.  bias may be NULL: the rows carry it already (the
 * projection added it in its epilogue, rt_gemm_bt with RT_EPILOGUE_BIAS), and the kernel is a
 * pure change of layout (plus the Q scale). */
int rt_qkv_bias_split(const void* qkv, const void* bias, void* q, void* k, void* vt,
                      const int* seq_blocks_dev, int batch, int total_blocks, int heads,
                      float q_scale, int dtype, void* stream);

/* Inverse of the packed layout: packed tiles -> dst[T, H*64] token-major; transposed = 0
 * for q / k, 1 for vt. */
int rt_unpack_head_tiles(const void* packed, void* dst, const int* seq_blocks_dev, int batch,
                         int total_blocks, int heads, int transposed, int dtype, void* stream);

/* Replaces kernels::test_gemm_1 (layers/kernels/sparse_attention.cu:3192-3228) and the
 * two live kernels behind it (:2953-3190 balanced, :2111-2403 non balanced):
 * out[T, H*64] token-major = softmax over the listed key blocks of (q . k) @ v, evaluated
 * as 2^(q.k) / sum 2^(q.k): the scale log2(e)/sqrt(d) is already folded into q.  to_idx/to_pos: device CSR from rt_meta_build_to_index
 * (plan_heads = 1 or heads).  If from_idx/from_pos are non-NULL the launch is
 * `n_wg` persistent workgroups each walking its slice of the LPT plan (balanced);
 * otherwise the kernel hands the units out itself: two persistent workgroups per CU draw
 * tickets from per-XCD counters, the two rows of each sparse (sequence, head) that list every
 * block first (four waves share such a row), then one unit per wave.
 * dtype RT_F16 / RT_BF16: fp32 accumulation, probabilities rounded to the tensor type for the
 * second product.  RT_F32 (the reference's fp32-output dispatch, sparse_attention.cu:1582-1599):
 * every tensor fp32, fp32 matrix instructions; an accuracy mode, about ten times slower.
 * Limits of one launch (RT_EINVAL beyond them): batch <= 1024 sequences, total_blocks <= 4096
 * (262144 tokens), total_blocks * heads * 24576 < 2^31 (byte offsets are 32-bit).  The first launch
 * on a device without from_idx/from_pos allocates 384 KiB of counters that the library keeps
 * (rt_bs_attention_fwd_no_alloc does not): a ring of 64 sets, one per launch, each left zeroed by the
 * launch that used it.  Launches may overlap on any number of streams and threads, in any order, as
 * long as no more than 64 of them are in flight on one device at a time. */
int rt_bs_attention_fwd(const void* q, const void* k, const void* vt, void* out,
                        const int* seq_blocks_dev, int batch, int total_blocks, int heads,
                        const int* to_idx, const int* to_pos, int plan_heads,
                        const int* from_idx, const int* from_pos, int n_wg,
                        int dtype, void* stream);

/* The same launch for a batch whose sequences end in padding (the reference only takes
 * lengths that are multiples of 64: python/util.py:36-46; this is the to_mask / band_mask /
 * rand_mask handling of its oracle, python/modeling_big_bird.py:640-760, for a packed batch).
 * seq_tokens_dev[s] = true token count of sequence s, 1 .. 64 * n_s (values outside are clamped); the
 * keys from there to the end of the sequence get no weight, whether they are the tail of one block or
 * whole blocks (a sequence kept at the width of a padded batch, so that its plan is the one the oracle
 * draws for that width).  Padded QUERY rows are computed like any other row (over the real keys their
 * rows list); the caller drops them.  NULL = no padding (rt_bs_attention_fwd). */
int rt_bs_attention_fwd_masked(const void* q, const void* k, const void* vt, void* out,
                               const int* seq_blocks_dev, const int* seq_tokens_dev, int batch,
                               int total_blocks, int heads, const int* to_idx, const int* to_pos,
                               int plan_heads, const int* from_idx, const int* from_pos, int n_wg,
                               int dtype, void* stream);

/* The same launch with the queries read where the QKV projection left them: `qkv` is the
 * [T, 3*H*64] input of rt_qkv_bias_split (columns 0 .. H*64-1 are Q), `qkv_bias` its bias; each
 * unit adds the bias and applies q_scale to its 64x64 query tile as it loads it (once per unit,
 * the same fp32 arithmetic and rounding as the split kernel, so both routes give the same bits).
 * k and vt still come from rt_qkv_bias_split (called with q = NULL).  Same stage of the
 * reference as rt_bs_attention_fwd; the reference always materialises Q
 * (layers/kernels/add_bias_and_transpose.cu:212-233).  seq_tokens_dev may be NULL.
 * qkv_bias may be NULL when the rows carry the bias already (see rt_qkv_bias_split): only q_scale
 * is applied.  At most 64 heads. */
int rt_bs_attention_fwd_qrows(const void* qkv, const void* qkv_bias, float q_scale, const void* k,
                              const void* vt, void* out, const int* seq_blocks_dev,
                              const int* seq_tokens_dev, int batch, int total_blocks, int heads,
                              const int* to_idx, const int* to_pos, int plan_heads,
                              const int* from_idx, const int* from_pos, int n_wg, int dtype,
                              void* stream);

/* rt_bs_attention_fwd_masked for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the
 * reference.  The other attention entry points take the kernel's queue counters from a ring that the
 * library allocates on a device's first launch; this one keeps them in a static device array of
 * RT_NO_ALLOC_SCRATCH_BYTES that every GPU the library runs on holds until the process ends, and calls
 * no hipMalloc, hipFree or other allocating routine.  It always runs the kernel's own enumeration (no
 * from_idx/from_pos plan; that launch uses no counters and allocates nothing in any entry point).
 * Limits: batch <= RT_NO_ALLOC_MAX_BATCH and total_blocks <= RT_NO_ALLOC_MAX_BLOCKS, else RT_EINVAL.
 * Every call on one GPU uses the same counters, cleared by a small kernel ahead of the launch: calls
 * that overlap on one GPU (two streams, two threads) race and give wrong results; calls on one stream,
 * or otherwise ordered, are fine.  The first call on a device looks the array's address up
 * (hipGetSymbolAddress): make that call outside a graph capture. */
#define RT_NO_ALLOC_SCRATCH_BYTES 8192
#define RT_NO_ALLOC_MAX_BATCH 1024
#define RT_NO_ALLOC_MAX_BLOCKS 4096
int rt_bs_attention_fwd_no_alloc(const void* q, const void* k, const void* vt, void* out,
                                 const int* seq_blocks_dev, const int* seq_tokens_dev, int batch,
                                 int total_blocks, int heads, const int* to_idx, const int* to_pos,
                                 int plan_heads, int dtype, void* stream);

/* Replaces kernels::add_bias_and_layernorm_kernel (layers/kernels/
 * add_bias_and_layernorm.cu:268-285): out = LN(out + bias + residual) * gamma + beta,
 * in place on out[rows, hidden]; hidden a multiple of 8. */
int rt_bias_residual_layernorm(void* out, const void* residual, const void* bias,
                               const void* gamma, const void* beta, int64_t rows, int hidden,
                               float eps, int dtype, void* stream);

/* Replaces kernels::add_bias_act_kernel (layers/kernels/add_bias_act.cu:114-133):
 * out = gelu_tanh(out + bias), in place on out[rows, width]; width a multiple of 8. */
int rt_bias_gelu(void* out, const void* bias, int64_t rows, int width, int dtype, void* stream);

/* Replaces the PyTorch operators of BertEmbeddings.__call__ (python/modeling_bert.py:47-63):
 * out[t] = LayerNorm(word[input_ids[t]] + position[position_ids[t]] + token_type[token_type_ids[t]])
 * * gamma + beta for the T tokens of a packed batch, written in out_dtype (the reference casts to
 * fp16).  Tables [vocab | max_pos | type_vocab, hidden], gamma and beta have table_dtype (fp32 in the
 * reference); ids are int32 device arrays and are clamped into their table; hidden a multiple of 8. */
int rt_embed_layernorm(const int* input_ids, const int* position_ids, const int* token_type_ids,
                       const void* word, const void* position, const void* token_type,
                       const void* gamma, const void* beta, void* out, int64_t rows, int hidden,
                       int vocab, int max_pos, int type_vocab, float eps, int table_dtype,
                       int out_dtype, void* stream);

/* ---------------------------------------------------------------------- dense GEMM */

/* Replaces kernels::MatMul (layers/kernels/mat_mul.cpp:9-96): row-major
 * C[M,N] = A[M,K] . B[K,N] through hipBLASLt with fp32 accumulation.  The handle owns
 * the hipBLASLt context, the heuristic cache and a workspace. */
typedef struct rt_gemm_ctx rt_gemm_ctx;
int rt_gemm_create(rt_gemm_ctx** ctx);
int rt_gemm_destroy(rt_gemm_ctx* ctx);
/* How many hipBLASLt heuristic candidates are timed (once per (N, K, dtype, epilogue), on the
 * operands of the first rt_gemm call of that kind) before one is kept: 1 = take the library's
 * first suggestion, default 64 (about 40 ms per kind); RT_GEMM_TUNE_ALL = every solution of the library that accepts
 * the problem (seconds per kind, once per process). */
#define RT_GEMM_TUNE_ALL (-1)
int rt_gemm_set_tuning(rt_gemm_ctx* ctx, int candidates);
/* A packed batch brings a new M with every batch, and the fastest solution moves with M (output
 * tiles against CUs).  The first call with a new M of a kind already tuned times only that
 * kind's `candidates` best solutions (default 6, about 3 ms; at most 8); 0 or 1 = take the
 * kind's winner untimed.  A server that knows its range of token counts runs each once at start. */
int rt_gemm_set_retuning(rt_gemm_ctx* ctx, int candidates);
int rt_gemm(rt_gemm_ctx* ctx, const void* a, const void* b, void* c,
            int64_t m, int64_t n, int64_t k, int dtype, void* stream);

/* The same product with the epilogue fused into the GEMM: C = A . B + bias[N]
 * (RT_EPILOGUE_BIAS) or C = gelu_tanh(A . B + bias[N]) (RT_EPILOGUE_BIAS_GELU).  The second
 * replaces the pair kernels::MatMul + kernels::add_bias_act_kernel of BertIntermediate
 * (layers/bert_intermediate.cpp:22-30) with one pass over the [M, N] output; bias has the
 * dtype of the operands. */
enum { RT_EPILOGUE_NONE = 0, RT_EPILOGUE_BIAS = 1, RT_EPILOGUE_BIAS_GELU = 2 };
int rt_gemm_bias_act(rt_gemm_ctx* ctx, const void* a, const void* b, const void* bias, void* c,
                     int64_t m, int64_t n, int64_t k, int epilogue, int dtype, void* stream);

/* C[M,N] = A[M,K] . Bt[N,K]^T with any of the three epilogues (bias may be NULL for
 * RT_EPILOGUE_NONE): the b_trans = true form of kernels::MatMul
 * (layers/kernels/mat_mul.cpp:9-96, which passes CUBLAS_OP_T for it).  Both operands are then
 * contiguous along K, the layout the library's kernels for these shapes are fastest on, so the
 * layer objects keep their weights as [out, in] and call this. */
int rt_gemm_bt(rt_gemm_ctx* ctx, const void* a, const void* bt, const void* bias, void* c,
               int64_t m, int64_t n, int64_t k, int epilogue, int dtype, void* stream);

/* ------------------------------------------------------------------ pooling + pooler head */

/* SequencePool of the reference (python/modeling_bert.py:270-277, a stub there; the modes are its
 * PoolingType, :298-314) for a packed batch: out[s, :] = the first / last token's row of sequence
 * s, or the mean / maximum over its tokens (fp32 accumulation).  seq_tokens_dev (optional) gives
 * the true token counts of sequences whose last block ends in padding. */
enum { RT_POOL_FIRST = 0, RT_POOL_LAST = 1, RT_POOL_MEAN = 2, RT_POOL_MAX = 3 };
int rt_sequence_pool(const void* hidden, const int* seq_blocks_dev, const int* seq_tokens_dev,
                     int batch, int width, int mode, void* out, int dtype, void* stream);

/* BertPooler (python/modeling_bert.py:279-296, commented out in the reference; HuggingFace
 * BigBirdModel.pooler + tanh): out[B, d_out] = tanh(pooled[B, d_in] . weight_t[d_out, d_in]^T + bias). */
int rt_pooler_dense_tanh(const void* pooled, const void* weight_t, const void* bias, void* out,
                         int batch, int d_in, int d_out, int dtype, void* stream);

/* ------------------------------------------------------- metadata / stream pipeline */

/* Replaces Semaphore + MetaData + the per-layer std::async index workers
 * (layers/semaphore.cpp:8-37, layers/metadata.cpp:6-18,
 * layers/multi_headed_attention.h:102-103, .cpp:16-139).  One worker thread per layer
 * waits on a counting semaphore; rt_pipeline_publish stores the batch geometry and
 * signals every layer; each worker builds its layer's CSR (seed = layer index) into
 * pinned memory, uploads it on a private stream (a small kernel that reads the pinned
 * buffer: a copy call would make the worker wait for the device) and records an event;
 * rt_pipeline_acquire blocks the host until that layer's CSR is queued, then makes the
 * caller's stream wait on the event.  device < 0 keeps everything on the host (the
 * returned pointers are host pointers) so the ordering logic can be exercised without
 * a GPU.  async = 0 builds the CSR inside rt_pipeline_acquire instead.
 * rt_pipeline_release(layer, stream) is called after the kernel that reads the layer's CSR has been launched
 * on `stream`.  Each layer keeps two CSR buffers; the one a batch used is written again two batches later,
 * once every reader of that batch has finished: per batch the pipeline records one event on every stream
 * layers were released on, behind the release of layer n_layers - 1, and for whatever was released after
 * that (or in a batch that never got that far) at the next rt_pipeline_publish.  The layers of one batch may
 * be launched in any order, on any streams, more than once, all before the next publish.
 * rt_pipeline_set_index_check(p, 1): every CSR a worker builds goes through rt_meta_check_to_index before it
 * is uploaded, and a failure comes back from rt_pipeline_acquire (a debugging aid; off by default). */
typedef struct rt_pipeline rt_pipeline;
int rt_pipeline_create(rt_pipeline** p, int n_layers, int heads, int plan_mode, int max_pos,
                       int policy, int async, int device);
int rt_pipeline_publish(rt_pipeline* p, const int* seq_blocks, int batch);
int rt_pipeline_acquire(rt_pipeline* p, int layer, void* stream, const int** to_idx,
                        const int** to_pos, int* plan_heads, double* host_wait_us);
int rt_pipeline_release(rt_pipeline* p, int layer, void* stream);
int rt_pipeline_set_index_check(rt_pipeline* p, int on);
int rt_pipeline_destroy(rt_pipeline* p);

#ifdef __cplusplus
}
#endif
#endif /* RAPTOR_T_HIP_H */
