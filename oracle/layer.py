"""Encoder-layer glue and the memory-bound epilogues, restated in PyTorch-CPU fp32.

Test infrastructure (see oracle/__init__.py).  Follows
  * layers/kernels/add_bias_and_transpose.cu:118-195   bias + Q scale + head split
  * layers/kernels/add_bias_and_layernorm.cu:191-266   LN(out + bias + residual) * gamma + beta
  * layers/kernels/add_bias_act.cu:41-48, :86-105      tanh-form GELU of (out + bias)
  * layers/multi_headed_attention.cpp:154-216, layers/bert_intermediate.cpp:7-29,
    layers/bert_output.cpp:7-44                        call order and buffer roles
  * python/modeling_big_bird.py:1318-1329, :1424-1451, :1564-1567  the same glue in the
    reference's oracle (SelfOutput, Intermediate, Output, feed_forward_chunk)
  * python/modeling_bert.py:47-63                      embedding sum + LayerNorm(eps 1e-12)
Weights are stored `[in, out]` as the reference stores them
(python/modeling_bert.py:84-91, :107-113, :137-163); the fused QKV weight is Q|K|V.
"""
import math

import torch
import torch.nn.functional as F

from . import attention

GELU_C0 = 0.7978845608028654     # sqrt(2/pi), layers/kernels/add_bias_act.cu:44
GELU_C1 = 0.044715


def bias_residual_layernorm(x, residual, bias, gamma, beta, eps):
    h = x.float() + bias.float() + residual.float()
    return F.layer_norm(h, (h.shape[-1],), gamma.float(), beta.float(), eps)


def embeddings_layernorm(input_ids, position_ids, token_type_ids, word, position, token_type, gamma, beta,
                         eps=1e-12):
    """Packed-input front end of the reference (python/modeling_bert.py:53-62): rows of the three tables
    are gathered and summed in the order word + token_type + position, then LayerNorm.  Written out with
    explicit indexing and moments (not nn.Embedding / F.layer_norm, which the tests pin it against)."""
    x = (word.double()[input_ids.long()] + token_type.double()[token_type_ids.long()]
         + position.double()[position_ids.long()])
    mean = x.mean(dim=-1, keepdim=True)
    var = ((x - mean) ** 2).mean(dim=-1, keepdim=True)            # biased, as LayerNorm defines it
    return ((x - mean) / torch.sqrt(var + eps) * gamma.double() + beta.double()).float()


def bias_gelu(x, bias):
    return F.gelu(x.float() + bias.float(), approximate="tanh")


def qkv_bias_split(qkv, bias, heads, scale=None):
    """[T, 3D] -> q, k, v [T, H, d] with the bias added and q multiplied by `scale`
    (default 1/sqrt(d), layers/kernels/add_bias_and_transpose.cu:183, :214)."""
    t, d3 = qkv.shape
    dm = d3 // 3
    d = dm // heads
    scale = 1.0 / math.sqrt(d) if scale is None else scale
    x = qkv.float() + bias.float()
    q = (x[:, :dm] * scale).view(t, heads, d)
    k = x[:, dm:2 * dm].view(t, heads, d)
    v = x[:, 2 * dm:].view(t, heads, d)
    return q, k, v


def _stored(x, store_dtype):
    """A tensor as it reads back after a kernel has written it to memory in `store_dtype` (None: kept in fp32).
    The reference keeps every tensor between two kernels in the model's dtype (fp16: python/modeling_bert.py:63,
    the buffers of layers/multi_headed_attention.cpp:154-216), so its arithmetic sees these roundings too."""
    return x if store_dtype is None else x.to(store_dtype).float()


def attention_sublayer(hidden, w, heads, seq_blocks, to_idx, to_pos, plan_heads, eps, block=64, store_dtype=None,
                       bias_in_projection=False):
    """QKV projection -> split -> block-sparse attention -> out-proj -> bias+residual+LN
    (layers/multi_headed_attention.cpp:154-216).  bias_in_projection only matters with a store_dtype: the
    projection's output is then stored once, with its bias (what a GEMM with a bias epilogue writes), instead of
    being stored without it and again after the bias kernel, which is the reference's sequence."""
    st = lambda x: _stored(x, store_dtype)
    if bias_in_projection:
        rows = st(hidden.float() @ w["qkv_weight"].float() + w["qkv_bias"].float())
        q, k, v = qkv_bias_split(rows, torch.zeros_like(w["qkv_bias"]), heads)
        q = st(q)                                   # K and V are copies of what is stored; Q is scaled and stored again
    else:
        qkv = st(hidden.float() @ w["qkv_weight"].float())
        q, k, v = (st(x) for x in qkv_bias_split(qkv, w["qkv_bias"], heads))
    ctx = st(attention.csr_attention(q, k, v, seq_blocks, to_idx, to_pos, plan_heads, block, scale=1.0))
    t = ctx.shape[0]
    proj = st(ctx.reshape(t, -1) @ w["attn_out_weight"].float())
    return st(bias_residual_layernorm(proj, hidden, w["attn_out_bias"], w["attn_ln_weight"],
                                      w["attn_ln_bias"], eps))


def encoder_layer(hidden, w, heads, seq_blocks, to_idx, to_pos, plan_heads, eps=1e-5, block=64, store_dtype=None,
                  bias_in_projection=False):
    """One layer: attention sub-layer, FFN up + GELU, FFN down + bias+residual+LN with the
    attention output as the residual (python/modeling_bert.py:172-210).  store_dtype: the dtype every tensor
    that passes from one kernel to the next is rounded to (None: all fp32, the plain mathematical layer);
    bias_in_projection: see attention_sublayer."""
    st = lambda x: _stored(x, store_dtype)
    attn = attention_sublayer(hidden, w, heads, seq_blocks, to_idx, to_pos, plan_heads, eps, block, store_dtype,
                              bias_in_projection)
    inter = st(bias_gelu(attn @ w["inter_weight"].float(), w["inter_bias"]))
    out = st(inter @ w["out_weight"].float())
    return st(bias_residual_layernorm(out, attn, w["out_bias"], w["out_ln_weight"], w["out_ln_bias"], eps))


def random_layer_weights(hidden, ffn, generator, std=0.02, dtype=torch.float32):
    """N(0, 0.02) weights and biases, gamma = 1, beta = 0."""
    def n(*shape):
        return (torch.randn(*shape, generator=generator) * std).to(dtype)
    return {
        "qkv_weight": n(hidden, 3 * hidden), "qkv_bias": n(3 * hidden),
        "attn_out_weight": n(hidden, hidden), "attn_out_bias": n(hidden),
        "attn_ln_weight": torch.ones(hidden, dtype=dtype), "attn_ln_bias": torch.zeros(hidden, dtype=dtype),
        "inter_weight": n(hidden, ffn), "inter_bias": n(ffn),
        "out_weight": n(ffn, hidden), "out_bias": n(hidden),
        "out_ln_weight": torch.ones(hidden, dtype=dtype), "out_ln_bias": torch.zeros(hidden, dtype=dtype),
    }


def sequence_pool(hidden, seq_blocks, mode, seq_tokens=None, block=64):
    """SequencePool of the reference (python/modeling_bert.py:270-277 is a stub; modes = PoolingType,
    :298-314) for a packed batch: per sequence the first / last token's row, or the mean / max over
    its tokens.  hidden [T, D]; seq_tokens = true token counts when the last block ends in padding."""
    hidden = hidden.double()
    rows = []
    for s in range(len(seq_blocks) - 1):
        t0 = seq_blocks[s] * block
        count = (seq_blocks[s + 1] - seq_blocks[s]) * block
        if seq_tokens is not None:
            count = max(1, min(int(seq_tokens[s]), count))
        x = hidden[t0:t0 + count]
        if mode == "First":
            rows.append(x[0])
        elif mode == "Last":
            rows.append(x[-1])
        elif mode == "Mean":
            rows.append(x.sum(0) / count)
        elif mode == "Max":
            rows.append(x.max(0).values)
        else:
            raise ValueError("unknown pooling mode %r" % (mode,))
    return torch.stack(rows).float()


def pooler(pooled, weight, bias):
    """BertPooler (python/modeling_bert.py:279-296, commented out there; HuggingFace
    BigBirdModel: `activation(pooler(sequence_output[:, 0]))`, modeling_big_bird.py): tanh of a dense
    layer; weight is [in, out] as every weight of the layers."""
    return torch.tanh(pooled.double() @ weight.double() + bias.double()).float()
