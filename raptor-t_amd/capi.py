"""ctypes binding of `libraptor_t_hip.so` (declared in include/raptor_t_hip.h).

Thin by design: numpy arrays for host metadata, `tensor.data_ptr()` for device memory,
the current torch stream for launches.  Every wrapper raises `RaptorError` with the
library's own message on a non-zero status.
"""
import ctypes
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libraptor_t_hip.so")

RT_F16, RT_BF16, RT_F32 = 0, 1, 2
RT_PLAN_HF, RT_PLAN_REFERENCE, RT_PLAN_EXPLICIT = 0, 1, 2
RT_POLICY_REFERENCE_PATCHED, RT_POLICY_HF_UPSTREAM = 0, 1
RT_EINVAL, RT_ENOMEM, RT_EIO, RT_ENOSYS, RT_ECANCELED = -22, -12, -5, -38, -125
RT_EPILOGUE_NONE, RT_EPILOGUE_BIAS, RT_EPILOGUE_BIAS_GELU = 0, 1, 2
RT_GEMM_TUNE_ALL = -1

EXPORTS = [
    "rt_last_error_string", "rt_abi_version", "rt_time_next_launch", "rt_meta_np_permutations", "rt_meta_seq_prefix_blocks",
    "rt_meta_rand_attn", "rt_meta_set_plan_cache", "rt_meta_to_index_size", "rt_meta_build_to_index", "rt_meta_block_costs",
    "rt_meta_partition_lpt", "rt_meta_check_partition", "rt_meta_check_to_index", "rt_qkv_bias_split", "rt_unpack_head_tiles", "rt_bs_attention_fwd",
    "rt_bs_attention_fwd_masked", "rt_bs_attention_fwd_qrows", "rt_bs_attention_fwd_no_alloc",
    "rt_bias_residual_layernorm", "rt_bias_gelu", "rt_embed_layernorm", "rt_gemm_create", "rt_gemm_destroy", "rt_gemm_set_tuning", "rt_gemm_set_retuning", "rt_gemm",
    "rt_gemm_bias_act", "rt_gemm_bt", "rt_sequence_pool", "rt_pooler_dense_tanh",
    "rt_pipeline_create", "rt_pipeline_publish", "rt_pipeline_acquire", "rt_pipeline_release",
    "rt_pipeline_destroy", "rt_pipeline_set_index_check",
]


class RaptorError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("raptor_t_hip error %d: %s" % (code, message))
        self.code = code


_lib = None


def lib():
    """The loaded library; fails loudly when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError("%s is missing: run `make -C raptor-t_amd/csrc` (or __graft_entry__.build())" % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH)
        L.rt_last_error_string.restype = ctypes.c_char_p
        i32p, i64p, vp = ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int64), ctypes.c_void_p
        I, U, L64, F = ctypes.c_int, ctypes.c_uint32, ctypes.c_int64, ctypes.c_float
        L.rt_time_next_launch.argtypes = [vp, vp]
        L.rt_meta_np_permutations.argtypes = [U, i32p, I, i32p]
        L.rt_meta_seq_prefix_blocks.argtypes = [i32p, I, i32p]
        L.rt_meta_rand_attn.argtypes = [I, U, I, I, I, i32p]
        L.rt_meta_to_index_size.argtypes = [i32p, I, I, i64p, i64p]
        L.rt_meta_set_plan_cache.argtypes = [L64, i64p, i64p]
        L.rt_meta_build_to_index.argtypes = [i32p, I, I, I, U, I, I, i32p, i32p, L64, i32p, L64]
        L.rt_meta_block_costs.argtypes = [i32p, I, i32p, i64p]
        L.rt_meta_partition_lpt.argtypes = [i32p, I, I, I, i32p, i32p]
        L.rt_meta_check_partition.argtypes = [i32p, i32p, I, I, I]
        L.rt_meta_check_to_index.argtypes = [i32p, i32p, L64, i32p, I, I]
        L.rt_qkv_bias_split.argtypes = [vp, vp, vp, vp, vp, vp, I, I, I, F, I, vp]
        L.rt_unpack_head_tiles.argtypes = [vp, vp, vp, I, I, I, I, I, vp]
        L.rt_bs_attention_fwd.argtypes = [vp, vp, vp, vp, vp, I, I, I, vp, vp, I, vp, vp, I, I, vp]
        L.rt_bs_attention_fwd_masked.argtypes = [vp, vp, vp, vp, vp, vp, I, I, I, vp, vp, I, vp, vp, I, I, vp]
        L.rt_bs_attention_fwd_qrows.argtypes = [vp, vp, F, vp, vp, vp, vp, vp, I, I, I, vp, vp, I, vp, vp, I, I, vp]
        L.rt_bs_attention_fwd_no_alloc.argtypes = [vp, vp, vp, vp, vp, vp, I, I, I, vp, vp, I, I, vp]
        L.rt_bias_residual_layernorm.argtypes = [vp, vp, vp, vp, vp, L64, I, F, I, vp]
        L.rt_bias_gelu.argtypes = [vp, vp, L64, I, I, vp]
        L.rt_gemm_create.argtypes = [ctypes.POINTER(vp)]
        L.rt_gemm_destroy.argtypes = [vp]
        L.rt_gemm_set_tuning.argtypes = [vp, I]
        L.rt_gemm_set_retuning.argtypes = [vp, I]
        L.rt_gemm.argtypes = [vp, vp, vp, vp, L64, L64, L64, I, vp]
        L.rt_embed_layernorm.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, vp, L64, I, I, I, I, ctypes.c_float, I, I, vp]
        L.rt_gemm_bias_act.argtypes = [vp, vp, vp, vp, vp, L64, L64, L64, I, I, vp]
        L.rt_gemm_bt.argtypes = [vp, vp, vp, vp, vp, L64, L64, L64, I, I, vp]
        L.rt_sequence_pool.argtypes = [vp, vp, vp, I, I, I, vp, I, vp]
        L.rt_pooler_dense_tanh.argtypes = [vp, vp, vp, vp, I, I, I, I, vp]
        L.rt_pipeline_create.argtypes = [ctypes.POINTER(vp), I, I, I, I, I, I, I]
        L.rt_pipeline_publish.argtypes = [vp, i32p, I]
        L.rt_pipeline_acquire.argtypes = [vp, I, vp, ctypes.POINTER(vp), ctypes.POINTER(vp), i32p,
                                          ctypes.POINTER(ctypes.c_double)]
        L.rt_pipeline_release.argtypes = [vp, I, vp]
        L.rt_pipeline_destroy.argtypes = [vp]
        L.rt_pipeline_set_index_check.argtypes = [vp, I]
        _lib = L
    return _lib


def check(rc):
    if rc != 0:
        raise RaptorError(rc, lib().rt_last_error_string().decode("utf-8", "replace"))


def _i32(a):
    return np.ascontiguousarray(np.asarray(a, dtype=np.int32))


def _p(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_int))


# ----------------------------------------------------------------------------- host metadata
def np_permutations(seed, sizes):
    sizes = _i32(sizes)
    out = np.empty(int(sizes.sum()), dtype=np.int32)
    check(lib().rt_meta_np_permutations(seed, _p(sizes), len(sizes), _p(out)))
    return out


def seq_prefix_blocks(seq_lens):
    lens = _i32(seq_lens)
    out = np.empty(len(lens) + 1, dtype=np.int32)
    check(lib().rt_meta_seq_prefix_blocks(_p(lens), len(lens), _p(out)))
    return out


def rand_attn(length, seed, heads, max_pos=4096, policy=RT_POLICY_REFERENCE_PATCHED):
    n = max(length // 64, 2)
    out = np.empty((heads, n - 2, 3), dtype=np.int32)
    check(lib().rt_meta_rand_attn(length, seed, heads, max_pos, policy, _p(out)))
    return out


def plan_cache(max_bytes=-1):
    """Sets the bound of the library's memo table of plans (negative: leave it) and returns (hits, misses) so far."""
    h, m = ctypes.c_int64(), ctypes.c_int64()
    check(lib().rt_meta_set_plan_cache(max_bytes, ctypes.byref(h), ctypes.byref(m)))
    return h.value, m.value


def to_index_size(seq_blocks, plan_heads):
    sb = _i32(seq_blocks)
    a, b = ctypes.c_int64(), ctypes.c_int64()
    check(lib().rt_meta_to_index_size(_p(sb), len(sb) - 1, plan_heads, ctypes.byref(a), ctypes.byref(b)))
    return a.value, b.value


def build_to_index(seq_blocks, plan_heads, mode=RT_PLAN_HF, seed=0, max_pos=4096,
                   policy=RT_POLICY_REFERENCE_PATCHED, rand_attn=None):
    sb = _i32(seq_blocks)
    n_idx, n_pos = to_index_size(sb, plan_heads)
    idx = np.empty(n_idx, dtype=np.int32)
    pos = np.empty(n_pos, dtype=np.int32)
    ra = None if rand_attn is None else _i32(rand_attn).reshape(-1)
    check(lib().rt_meta_build_to_index(_p(sb), len(sb) - 1, plan_heads, mode, seed, max_pos, policy,
                                       None if ra is None else _p(ra), _p(idx), n_idx, _p(pos), n_pos))
    return idx, pos


def block_costs(seq_blocks):
    sb = _i32(seq_blocks)
    out = np.empty(int(sb[-1]), dtype=np.int32)
    tot = ctypes.c_int64()
    check(lib().rt_meta_block_costs(_p(sb), len(sb) - 1, _p(out), ctypes.byref(tot)))
    return out, tot.value


def partition_lpt(seq_blocks, heads, n_wg):
    sb = _i32(seq_blocks)
    pos = np.empty(n_wg + 1, dtype=np.int32)
    ids = np.empty(int(sb[-1]) * heads, dtype=np.int32)
    check(lib().rt_meta_partition_lpt(_p(sb), len(sb) - 1, heads, n_wg, _p(pos), _p(ids)))
    return pos, ids


def check_partition(from_pos, from_idx, total_blocks, heads):
    """Raises RaptorError unless (from_pos, from_idx) is a work plan that lists every unit exactly once."""
    pos, ids = _i32(from_pos), _i32(from_idx)
    if len(ids) != total_blocks * heads or len(pos) < 2:
        raise ValueError("from_idx needs total_blocks * heads entries and from_pos at least two")
    check(lib().rt_meta_check_partition(_p(pos), _p(ids), len(pos) - 1, total_blocks, heads))


def check_to_index(to_idx, to_pos, seq_blocks, plan_heads):
    """Raises RaptorError unless (to_idx, to_pos) is a to-block index of the batch `seq_blocks`: one non-empty row
    per (plan head, block), every entry a block of the row's own sequence."""
    idx, pos, sb = _i32(to_idx), _i32(to_pos), _i32(seq_blocks)
    if len(sb) < 2 or len(pos) != plan_heads * int(sb[-1]) + 1:
        raise ValueError("to_pos needs plan_heads * total_blocks + 1 entries")
    check(lib().rt_meta_check_to_index(_p(idx), _p(pos), len(idx), _p(sb), len(sb) - 1, plan_heads))


# ------------------------------------------------------------------------------- GPU kernels
def _dtype_code(t):
    import torch
    return {torch.float16: RT_F16, torch.bfloat16: RT_BF16, torch.float32: RT_F32}[t.dtype]


def _stream():
    import torch
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _dp(t, dtype=None, numel=None, name="tensor"):
    """Device pointer of `t` for a kernel argument (None -> NULL).  The kernels dereference it as it is, so a
    host tensor, a strided view, another dtype or too few elements is refused here: on the GPU each of these
    would be a memory fault, not an error code."""
    if t is None:
        return ctypes.c_void_p(0)
    if not t.is_cuda:
        raise ValueError("%s must be a GPU tensor, got one on %s" % (name, t.device))
    if not t.is_contiguous():
        raise ValueError("%s must be contiguous" % name)
    if dtype is not None and t.dtype != dtype:
        raise ValueError("%s must have dtype %s, got %s" % (name, dtype, t.dtype))
    if numel is not None and t.numel() < numel:
        raise ValueError("%s holds %d elements, the launch reads %d" % (name, t.numel(), numel))
    return ctypes.c_void_p(t.data_ptr())


def _ip(t, numel=None, name="index tensor"):
    """Device pointer of an int32 index tensor."""
    import torch
    return _dp(t, torch.int32, numel, name)


def _attention_args(out, k, vt, seq_blocks_dev, heads, to_idx, to_pos, plan_heads, from_idx, from_pos, seq_tokens_dev):
    """Shapes every attention entry point shares; returns (batch, blocks, n_wg)."""
    batch = seq_blocks_dev.numel() - 1
    if out.dim() != 2 or out.shape[0] % 64 or out.shape[1] != heads * 64:
        raise ValueError("out must be [tokens (a multiple of 64), heads * 64]")
    nb = out.shape[0] // 64
    n_wg = 0 if from_pos is None else from_pos.numel() - 1
    if (from_idx is None) != (from_pos is None):
        raise ValueError("from_idx and from_pos go together")
    if plan_heads not in (1, heads):
        raise ValueError("plan_heads must be 1 or heads")
    if seq_tokens_dev is not None and seq_tokens_dev.numel() != batch:
        raise ValueError("seq_tokens_dev needs one entry per sequence")
    _dp(k, out.dtype, out.numel(), "k"), _dp(vt, out.dtype, out.numel(), "vt"), _dp(out, name="out")
    _ip(seq_blocks_dev, name="seq_blocks_dev"), _ip(seq_tokens_dev, name="seq_tokens_dev")
    _ip(to_idx, name="to_idx"), _ip(to_pos, plan_heads * nb + 1, "to_pos")
    _ip(from_idx, nb * heads, "from_idx"), _ip(from_pos, name="from_pos")
    return batch, nb, n_wg


def qkv_bias_split(qkv, bias, q, k, vt, seq_blocks_dev, heads, q_scale):
    """q may be None: Q is not written (for bs_attention_fwd_qrows).  bias may be None: the rows carry it already."""
    batch = seq_blocks_dev.numel() - 1
    if qkv.dim() != 2 or qkv.shape[0] % 64 or qkv.shape[1] != 3 * heads * 64:
        raise ValueError("qkv must be [tokens (a multiple of 64), 3 * heads * 64]")
    nb = qkv.shape[0] // 64
    per = qkv.shape[0] * heads * 64
    dt = qkv.dtype
    check(lib().rt_qkv_bias_split(_dp(qkv, name="qkv"), _dp(bias, dt, 3 * heads * 64, "bias"), _dp(q, dt, per, "q"),
                                  _dp(k, dt, per, "k"), _dp(vt, dt, per, "vt"), _ip(seq_blocks_dev, name="seq_blocks_dev"),
                                  batch, nb, heads, q_scale, _dtype_code(qkv), _stream()))


def unpack_head_tiles(packed, dst, seq_blocks_dev, heads, transposed):
    batch = seq_blocks_dev.numel() - 1
    nb = dst.shape[0] // 64
    check(lib().rt_unpack_head_tiles(_dp(packed, dst.dtype, dst.numel(), "packed"), _dp(dst, name="dst"),
                                     _ip(seq_blocks_dev, name="seq_blocks_dev"), batch, nb, heads,
                                     1 if transposed else 0, _dtype_code(dst), _stream()))


LOG2E = 1.4426950408889634
Q_SCALE = LOG2E / 8.0          # log2(e) / sqrt(64): what rt_bs_attention_fwd expects folded into q


def bs_attention_fwd(q, k, vt, out, seq_blocks_dev, heads, to_idx, to_pos, plan_heads,
                     from_idx=None, from_pos=None, seq_tokens_dev=None):
    """seq_tokens_dev: optional int32 device tensor, true token count per sequence (padded tail)."""
    batch, nb, n_wg = _attention_args(out, k, vt, seq_blocks_dev, heads, to_idx, to_pos, plan_heads, from_idx, from_pos,
                                      seq_tokens_dev)
    _dp(q, out.dtype, out.numel(), "q")
    if seq_tokens_dev is None:
        check(lib().rt_bs_attention_fwd(_dp(q), _dp(k), _dp(vt), _dp(out), _dp(seq_blocks_dev), batch, nb, heads,
                                        _dp(to_idx), _dp(to_pos), plan_heads, _dp(from_idx), _dp(from_pos), n_wg,
                                        _dtype_code(out), _stream()))
        return
    check(lib().rt_bs_attention_fwd_masked(_dp(q), _dp(k), _dp(vt), _dp(out), _dp(seq_blocks_dev), _dp(seq_tokens_dev),
                                           batch, nb, heads, _dp(to_idx), _dp(to_pos), plan_heads, _dp(from_idx),
                                           _dp(from_pos), n_wg, _dtype_code(out), _stream()))


def bs_attention_fwd_no_alloc(q, k, vt, out, seq_blocks_dev, heads, to_idx, to_pos, plan_heads, seq_tokens_dev=None):
    """bs_attention_fwd through the entry point that allocates no device memory (static queue counters)."""
    batch, nb, _ = _attention_args(out, k, vt, seq_blocks_dev, heads, to_idx, to_pos, plan_heads, None, None, seq_tokens_dev)
    _dp(q, out.dtype, out.numel(), "q")
    check(lib().rt_bs_attention_fwd_no_alloc(_dp(q), _dp(k), _dp(vt), _dp(out), _dp(seq_blocks_dev), _dp(seq_tokens_dev),
                                             batch, nb, heads, _dp(to_idx), _dp(to_pos), plan_heads, _dtype_code(out),
                                             _stream()))


def bs_attention_fwd_qrows(qkv, qkv_bias, q_scale, k, vt, out, seq_blocks_dev, heads, to_idx, to_pos, plan_heads,
                           from_idx=None, from_pos=None, seq_tokens_dev=None):
    """bs_attention_fwd with the queries taken from the [T, 3*H*64] projection output `qkv` (+ qkv_bias, * q_scale)."""
    batch, nb, n_wg = _attention_args(out, k, vt, seq_blocks_dev, heads, to_idx, to_pos, plan_heads, from_idx, from_pos,
                                      seq_tokens_dev)
    _dp(qkv, out.dtype, 3 * out.numel(), "qkv"), _dp(qkv_bias, out.dtype, 3 * heads * 64, "qkv_bias")
    if qkv.shape[0] != out.shape[0] or qkv.shape[1] != 3 * heads * 64 or \
            (qkv_bias is not None and qkv_bias.numel() != 3 * heads * 64):
        raise ValueError("qkv must be [tokens, 3 * heads * 64] with a bias of the same width")
    check(lib().rt_bs_attention_fwd_qrows(_dp(qkv), _dp(qkv_bias), q_scale, _dp(k), _dp(vt), _dp(out), _dp(seq_blocks_dev),
                                          _dp(seq_tokens_dev), batch, nb, heads, _dp(to_idx), _dp(to_pos), plan_heads,
                                          _dp(from_idx), _dp(from_pos), n_wg, _dtype_code(out), _stream()))


def bias_residual_layernorm(out, residual, bias, gamma, beta, eps):
    rows, hidden = out.shape
    dt = out.dtype
    _dp(out, name="out"), _dp(residual, dt, out.numel(), "residual")
    for name, t in (("bias", bias), ("gamma", gamma), ("beta", beta)):
        _dp(t, dt, hidden, name)
    check(lib().rt_bias_residual_layernorm(_dp(out), _dp(residual), _dp(bias), _dp(gamma), _dp(beta), rows, hidden,
                                           eps, _dtype_code(out), _stream()))


def bias_gelu(out, bias):
    rows, width = out.shape
    check(lib().rt_bias_gelu(_dp(out, name="out"), _dp(bias, out.dtype, width, "bias"), rows, width, _dtype_code(out),
                             _stream()))


def time_next_launch(start_event, stop_event):
    """Hands two hipEvent_t (integers / c_void_p; None = NULL) to the calling thread's next kernel launch of the
    library, which writes its dispatch's start and end into them.  (None, None) withdraws a waiting pair.
    Returns 1 if a pair was still waiting for a launch."""
    return lib().rt_time_next_launch(start_event, stop_event)


RT_POOL_FIRST, RT_POOL_LAST, RT_POOL_MEAN, RT_POOL_MAX = 0, 1, 2, 3


def sequence_pool(hidden, seq_blocks_dev, mode, out, seq_tokens_dev=None):
    """out[s] = first / last token's row of sequence s, or the mean / max over its tokens (packed batch)."""
    batch = seq_blocks_dev.numel() - 1
    if tuple(out.shape) != (batch, hidden.shape[1]) or out.dtype != hidden.dtype:
        raise ValueError("out must be [sequences, width] in the dtype of hidden")
    if seq_tokens_dev is not None and seq_tokens_dev.numel() != batch:
        raise ValueError("seq_tokens_dev needs one entry per sequence")
    check(lib().rt_sequence_pool(_dp(hidden, name="hidden"), _ip(seq_blocks_dev, name="seq_blocks_dev"),
                                 _ip(seq_tokens_dev, name="seq_tokens_dev"), batch, hidden.shape[1], mode,
                                 _dp(out), _dtype_code(hidden), _stream()))
    return out


def pooler_dense_tanh(pooled, weight_t, bias, out):
    """out = tanh(pooled @ weight_t.T + bias), weight_t as [out, in]."""
    batch, d_in = pooled.shape
    d_out = weight_t.shape[0]
    if weight_t.shape[1] != d_in or bias.numel() != d_out or tuple(out.shape) != (batch, d_out):
        raise ValueError("shape mismatch")
    for name, t in (("weight_t", weight_t), ("bias", bias), ("out", out)):
        _dp(t, pooled.dtype, None, name)
    check(lib().rt_pooler_dense_tanh(_dp(pooled), _dp(weight_t), _dp(bias), _dp(out), batch, d_in, d_out,
                                     _dtype_code(pooled), _stream()))
    return out


def embed_layernorm(input_ids, position_ids, token_type_ids, word, position, token_type, gamma, beta, out, eps=1e-12):
    """out[t] = LN(word[ids[t]] + position[pos[t]] + token_type[type[t]]) * gamma + beta; ids are int32 device
    tensors, the tables / gamma / beta share one dtype, out has the encoder's."""
    import torch
    for t in (input_ids, position_ids, token_type_ids):
        if t.dtype != torch.int32 or not t.is_cuda or not t.is_contiguous() or t.numel() != out.shape[0]:
            raise ValueError("ids must be contiguous int32 device tensors with one entry per output row")
    for t in (position, token_type, gamma, beta):
        if t.dtype != word.dtype:
            raise ValueError("tables, gamma and beta must share one dtype")
    rows, hidden = out.shape
    check(lib().rt_embed_layernorm(_dp(input_ids), _dp(position_ids), _dp(token_type_ids), _dp(word), _dp(position),
                                   _dp(token_type), _dp(gamma), _dp(beta), _dp(out), rows, hidden, word.shape[0],
                                   position.shape[0], token_type.shape[0], eps, _dtype_code(word), _dtype_code(out),
                                   _stream()))
    return out


class Gemm:
    """Owner of one rt_gemm_ctx."""

    def __init__(self):
        self._h = ctypes.c_void_p()
        check(lib().rt_gemm_create(ctypes.byref(self._h)))

    def set_tuning(self, candidates):
        check(lib().rt_gemm_set_tuning(self._h, candidates))

    def set_retuning(self, candidates):
        """How many of a kind's best solutions the first call with a new M times (0 / 1: none)."""
        check(lib().rt_gemm_set_retuning(self._h, candidates))

    @staticmethod
    def _operands(a, b, c, m, n, k, bias=None):
        _dp(a, name="a"), _dp(b, a.dtype, k * n, "b"), _dp(c, a.dtype, m * n, "c"), _dp(bias, a.dtype, n, "bias")

    def __call__(self, a, b, c):
        m, k = a.shape
        n = b.shape[1]
        self._operands(a, b, c, m, n, k)
        check(lib().rt_gemm(self._h, _dp(a), _dp(b), _dp(c), m, n, k, _dtype_code(a), _stream()))
        return c

    def bias_act(self, a, b, bias, c, epilogue=RT_EPILOGUE_BIAS_GELU):
        """c = a @ b + bias, through the tanh GELU when epilogue is RT_EPILOGUE_BIAS_GELU, in one kernel."""
        m, k = a.shape
        n = b.shape[1]
        self._operands(a, b, c, m, n, k, bias)
        check(lib().rt_gemm_bias_act(self._h, _dp(a), _dp(b), _dp(bias), _dp(c), m, n, k, epilogue, _dtype_code(a),
                                     _stream()))
        return c

    def bt(self, a, bt, c, bias=None, epilogue=RT_EPILOGUE_NONE):
        """c = a @ bt.T (+ bias, + GELU as `epilogue` says) with the weights kept as bt[N, K]."""
        m, k = a.shape
        n = bt.shape[0]
        self._operands(a, bt, c, m, n, k, bias)
        check(lib().rt_gemm_bt(self._h, _dp(a), _dp(bt), None if bias is None else _dp(bias), _dp(c), m, n, k, epilogue,
                               _dtype_code(a), _stream()))
        return c

    def close(self):
        if self._h:
            lib().rt_gemm_destroy(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Pipeline:
    """Owner of one rt_pipeline (device < 0: host only)."""

    def __init__(self, n_layers, heads, plan_mode=RT_PLAN_HF, max_pos=4096, policy=RT_POLICY_REFERENCE_PATCHED,
                 async_=True, device=0):
        self._h = ctypes.c_void_p()
        self.device = device
        check(lib().rt_pipeline_create(ctypes.byref(self._h), n_layers, heads, plan_mode, max_pos, policy,
                                       1 if async_ else 0, device))

    def publish(self, seq_blocks):
        sb = _i32(seq_blocks)
        check(lib().rt_pipeline_publish(self._h, _p(sb), len(sb) - 1))

    def acquire(self, layer, stream=None):
        idx, pos = ctypes.c_void_p(), ctypes.c_void_p()
        ph, wait = ctypes.c_int(), ctypes.c_double()
        st = ctypes.c_void_p(0) if self.device < 0 else (stream if stream is not None else _stream())
        check(lib().rt_pipeline_acquire(self._h, layer, st, ctypes.byref(idx), ctypes.byref(pos), ctypes.byref(ph),
                                        ctypes.byref(wait)))
        return idx.value, pos.value, ph.value, wait.value

    def release(self, layer, stream=None):
        st = ctypes.c_void_p(0) if self.device < 0 else (stream if stream is not None else _stream())
        check(lib().rt_pipeline_release(self._h, layer, st))

    def set_index_check(self, on):
        check(lib().rt_pipeline_set_index_check(self._h, 1 if on else 0))

    def close(self):
        if self._h:
            lib().rt_pipeline_destroy(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
