"""Python callers of the `raptor_t` layer functors.

Mirrors python/modeling_bert.py of the reference: the same classes (`BertEmbeddings`,
`BertIntermediate`, `BertOutput`, `BertAttention`, `BertLayer`, `BertEncoder`,
`BertModelNoPooler`), the same call order and buffer aliasing (attention writes
`attention_output`; the FFN writes back into the layer's input buffer, :204-207), the same
weight re-layout in `from_torch` (`cat(q, k, v).t()`, `dense.weight.t()`, :137-163).
Differences: sizes are read from the weights (no 768 / 3072 literals), LayerNorm eps and
the dtype are arguments, and `from_weights` builds layers from plain tensors so that a
random-init model needs no HuggingFace object.
"""
import enum
import os
import sys
from typing import Optional, Sequence

import torch
import torch.nn as nn

_LIB = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib")
if _LIB not in sys.path:
    sys.path.insert(0, _LIB)
try:
    import raptor_t as cxx          # built by raptor-t_amd/layers/build_ext.py
except ImportError as e:            # no silent fallback: the layer API is the product
    raise ImportError("the raptor_t extension is not built: run __graft_entry__.build() (%s)" % e)

from . import capi, checkpoint
from .util import generate_data_metainfo

roctx = torch.cuda.nvtx             # torch maps these ranges onto roctx on ROCm


def to_param_dict(torch_module: torch.nn.Module):
    return {k: v for k, v in torch_module.named_parameters()}


def create_empty_if_none(tensor, shape, device, dtype=torch.float16):
    if tensor is None:
        tensor = torch.zeros(shape, dtype=dtype, device=device)
    return tensor


class BertEmbeddings:
    """Word + position + token-type embeddings and LayerNorm(eps 1e-12) of the packed input
    (reference: python/modeling_bert.py:27-69, there PyTorch operators): one gather + LayerNorm
    kernel writing the packed [T, D] activations in the encoder's dtype.  The tables stay in fp32
    as the reference keeps them."""

    def __init__(self, word_embeddings_weight, position_embeddings_weight, token_type_embeddings_weight,
                 layerNorm_weight, layerNorm_bias, pad_token_id: int = 0, dtype=torch.float16, device="cuda"):
        prep = lambda w: w.detach().to(device=device, dtype=torch.float32).contiguous()
        self.word_embeddings = prep(word_embeddings_weight)
        self.position_embeddings = prep(position_embeddings_weight)
        self.token_type_embeddings = prep(token_type_embeddings_weight)
        self.gamma = prep(layerNorm_weight)
        self.beta = prep(layerNorm_bias)
        self.pad_token_id = pad_token_id          # kept for the reference's signature; a lookup needs no padding row
        self.dtype = dtype
        self.eps = 1e-12

    @torch.no_grad()
    def __call__(self, input_ids=None, position_ids=None, token_type_ids=None, output=None):
        if input_ids is None or position_ids is None or token_type_ids is None:
            raise ValueError("input_ids, position_ids and token_type_ids are all required")
        dev = self.word_embeddings.device
        ids = [t.to(device=dev, dtype=torch.int32).contiguous().view(-1) for t in (input_ids, position_ids, token_type_ids)]
        if output is None:
            output = torch.empty(ids[0].numel(), self.word_embeddings.shape[1], dtype=self.dtype, device=dev)
        capi.embed_layernorm(ids[0], ids[1], ids[2], self.word_embeddings, self.position_embeddings,
                             self.token_type_embeddings, self.gamma, self.beta, output, self.eps)
        return output

    @staticmethod
    def from_torch(bert_embedding, dtype=torch.float16):
        p = to_param_dict(bert_embedding)
        return BertEmbeddings(p["word_embeddings.weight"], p["position_embeddings.weight"],
                              p["token_type_embeddings.weight"], p["LayerNorm.weight"], p["LayerNorm.bias"],
                              dtype=dtype)


class BertIntermediate(cxx.BertIntermediate):
    def __call__(self, input_tensor, total_seq_len, output=None, kernel_fusion=True, test_info=None):
        roctx.range_push("intermediate")
        test_info = {} if test_info is None else test_info
        test_info = super().__call__(input_tensor, output, test_info, kernel_fusion)
        roctx.range_pop()
        return test_info

    @staticmethod
    def from_weights(weight_in_out, bias):
        return BertIntermediate(weight_in_out.contiguous(), bias.contiguous())

    @staticmethod
    def from_torch(intermediate, dtype=torch.float16):
        p = to_param_dict(intermediate)
        return BertIntermediate(torch.t(p["dense.weight"]).contiguous().to(dtype).cuda(), p["dense.bias"].to(dtype).cuda())


class BertOutput(cxx.BertOutput):
    def __call__(self, intermediate_output, attention_output, total_seq_len, output=None, kernel_fusion=True,
                 test_info=None):
        roctx.range_push("output")
        test_info = {} if test_info is None else test_info
        test_info = super().__call__(intermediate_output, attention_output, output, test_info, kernel_fusion)
        roctx.range_pop()
        return test_info

    @staticmethod
    def from_torch(output, dtype=torch.float16, eps=1e-5):
        p = to_param_dict(output)
        c = lambda t: t.detach().to(dtype).cuda().contiguous()
        return BertOutput(c(torch.t(p["dense.weight"])), c(p["dense.bias"]), c(p["LayerNorm.weight"]),
                          c(p["LayerNorm.bias"]), eps)


class BertAttention(cxx.BertAttention):
    def __call__(self, input_tensor, seq_position_info, seq_position_info_tensor, partition_part_index_tensor,
                 partition_part_tensor, context_layer, block_limit, attention_mask=None, head_mask=None,
                 output_attentions=False, is_trans_weight=False, kernel_fusion=True, test_info=None, balanced=True):
        roctx.range_push("attention")
        test_info = {} if test_info is None else test_info
        if attention_mask is None:
            attention_mask = torch.empty(0)
        test_info = super().__call__(input_tensor, attention_mask, context_layer, seq_position_info,
                                     seq_position_info_tensor, partition_part_index_tensor, partition_part_tensor,
                                     block_limit, test_info, kernel_fusion, balanced)
        roctx.range_pop()
        return test_info

    @staticmethod
    def from_torch(attention, layer_idx: int, async_: bool, dtype=torch.float16, eps=1e-5):
        p = {k: v for k, v in attention.named_parameters()}
        c = lambda t: t.detach().to(dtype).cuda().contiguous()
        with torch.no_grad():
            qkv_weight = torch.t(torch.cat((p["self.query.weight"], p["self.key.weight"], p["self.value.weight"]), 0))
            qkv_bias = torch.cat((p["self.query.bias"], p["self.key.bias"], p["self.value.bias"]), 0)
            return BertAttention(c(qkv_weight), c(qkv_bias), c(torch.t(p["output.dense.weight"])),
                                 c(p["output.dense.bias"]), c(p["output.LayerNorm.weight"]),
                                 c(p["output.LayerNorm.bias"]), attention.self.num_attention_heads, layer_idx, async_, eps)


class BertLayer:
    def __init__(self, attention: BertAttention, intermediate: BertIntermediate, output: BertOutput):
        self.attention = attention
        self.intermediate = intermediate
        self.output = output

    def __call__(self, hidden_states, seq_position_info, seq_position_info_tensor, partition_part_index_tensor,
                 partition_part_tensor, intermediate_temp, output_layer_temp, attention_output, block_limit,
                 attention_mask=None, head_mask=None, output_attentions=False, kernel_fusion=True, test_info=None,
                 balanced=True):
        roctx.range_push("layer")
        total = seq_position_info[-1] * 64
        test_info = self.attention(hidden_states, seq_position_info, seq_position_info_tensor,
                                   partition_part_index_tensor, partition_part_tensor, attention_output, block_limit,
                                   attention_mask, head_mask, output_attentions=output_attentions, test_info=test_info,
                                   kernel_fusion=kernel_fusion, balanced=balanced)
        test_info = self.intermediate(attention_output, total, intermediate_temp, test_info=test_info,
                                      kernel_fusion=kernel_fusion)
        test_info = self.output(intermediate_temp, attention_output, total, hidden_states, test_info=test_info,
                                kernel_fusion=kernel_fusion)
        roctx.range_pop()
        return hidden_states, test_info

    @staticmethod
    def from_weights(w, heads, layer_idx, async_=True, eps=1e-5):
        """`w`: the twelve tensors of one layer in the `[in, out]` layout (keys as
        produced by `random_layer_weights`)."""
        att = BertAttention(w["qkv_weight"], w["qkv_bias"], w["attn_out_weight"], w["attn_out_bias"],
                            w["attn_ln_weight"], w["attn_ln_bias"], heads, layer_idx, async_, eps)
        inter = BertIntermediate(w["inter_weight"], w["inter_bias"])
        out = BertOutput(w["out_weight"], w["out_bias"], w["out_ln_weight"], w["out_ln_bias"], eps)
        return BertLayer(att, inter, out)

    @staticmethod
    def from_torch(layer, layer_idx: int, async_: bool, dtype=torch.float16, eps=1e-5):
        return BertLayer(BertAttention.from_torch(layer.attention, layer_idx, async_, dtype, eps),
                         BertIntermediate.from_torch(layer.intermediate, dtype),
                         BertOutput.from_torch(layer.output, dtype, eps))


class BertEncoder:
    def __init__(self, layer: Sequence[BertLayer]):
        self.layer = layer

    def __call__(self, hidden_states, total_seq_len, thread_block_limit, seq_position_info, seq_position_info_tensor,
                 partition_part_index_tensor, partition_part_tensor, output_layer_temp, intermediate_temp,
                 attention_output, test_info=None, kernel_fusion=True, balanced=True, attention_mask=None,
                 head_mask=None, output_attentions=False, output_hidden_states=False):
        for l in self.layer:
            hidden_states, test_info = l(hidden_states=hidden_states, block_limit=thread_block_limit,
                                         seq_position_info=seq_position_info,
                                         seq_position_info_tensor=seq_position_info_tensor,
                                         partition_part_index_tensor=partition_part_index_tensor,
                                         partition_part_tensor=partition_part_tensor,
                                         output_layer_temp=output_layer_temp, intermediate_temp=intermediate_temp,
                                         attention_output=attention_output, attention_mask=attention_mask,
                                         test_info=test_info, kernel_fusion=kernel_fusion,
                                         output_attentions=output_attentions, balanced=balanced)
        return hidden_states, test_info

    def call_two_streams(self, hidden_states, seq_lens, thread_block_limit, head_num, output_layer_temp,
                         intermediate_temp, attention_output, test_info=None, kernel_fusion=True, balanced=True):
        """The same forward pass with the batch cut in two micro-batches, each on a HIP stream of its own (equal
        priority), so that one micro-batch's attention kernel runs beside the other's projection and FFN GEMMs
        instead of between them.  The reference overlaps only the host's index generation with the GPU
        (layers/multi_headed_attention.cpp:131-132, :179-185); its launches are serial on one stream.

        `seq_lens`: token count of every sequence of the packed batch (multiples of 64).  The cut is the sequence
        boundary nearest to half the tokens, so both micro-batches are row ranges of the caller's buffers and
        nothing is copied.  The batch metadata of both halves is made here (cached per geometry) and published
        on the two micro-batch lanes of the extension; the caller does not call MetaData.update_meta_data.
        Returns when everything is queued; the caller's current stream waits for both streams."""
        seq_lens = [int(n) for n in seq_lens]
        key = (tuple(seq_lens), int(thread_block_limit), int(head_num))
        if getattr(self, "_two_key", None) != key:
            total, run, cut, best = sum(seq_lens), 0, 1, None
            for i, n in enumerate(seq_lens[:-1]):
                run += n
                if best is None or abs(2 * run - total) < best:
                    best, cut = abs(2 * run - total), i + 1
            halves = [seq_lens] if len(seq_lens) < 2 else [seq_lens[:cut], seq_lens[cut:]]
            self._two_parts, t0 = [], 0
            for lens in halves:
                info = generate_data_metainfo(lens, 64, thread_block_limit, head_num)
                self._two_parts.append((slice(t0, t0 + sum(lens)), sum(lens), info))
                t0 += sum(lens)
            self._two_key = key
        if not hasattr(self, "_two_streams"):
            self._two_streams = [torch.cuda.Stream(), torch.cuda.Stream()]
            self._two_meta = cxx.MetaData()
        test_info = {} if test_info is None else test_info
        cur = torch.cuda.current_stream()
        try:
            for lane, (rows, t, (spi, spi_t, comp, ppi_t, pp_t)) in enumerate(self._two_parts):
                cxx.set_micro_batch_lane(lane)
                self._two_streams[lane].wait_stream(cur)
                with torch.cuda.stream(self._two_streams[lane]):
                    self._two_meta.update_meta_data(t, spi[-1] + 1, comp, spi)
            for l in self.layer:                       # issue order: the two lanes' layers alternate
                for lane, (rows, t, (spi, spi_t, comp, ppi_t, pp_t)) in enumerate(self._two_parts):
                    cxx.set_micro_batch_lane(lane)
                    with torch.cuda.stream(self._two_streams[lane]):
                        _, test_info = l(hidden_states=hidden_states[rows], block_limit=thread_block_limit,
                                         seq_position_info=spi, seq_position_info_tensor=spi_t,
                                         partition_part_index_tensor=ppi_t, partition_part_tensor=pp_t,
                                         output_layer_temp=output_layer_temp[rows],
                                         intermediate_temp=intermediate_temp[rows],
                                         attention_output=attention_output[rows], test_info=test_info,
                                         kernel_fusion=kernel_fusion, balanced=balanced)
        finally:
            cxx.set_micro_batch_lane(0)
        for lane in range(len(self._two_parts)):
            cur.wait_stream(self._two_streams[lane])
        return hidden_states, test_info

    @staticmethod
    def from_weights(layers_w, heads, async_=True, eps=1e-5):
        return BertEncoder([BertLayer.from_weights(w, heads, i, async_, eps) for i, w in enumerate(layers_w)])

    @staticmethod
    def from_torch(encoder, async_: bool, dtype=torch.float16, eps=1e-5):
        return BertEncoder([BertLayer.from_torch(l, i, async_, dtype, eps) for i, l in enumerate(encoder.layer)])


class BertModelNoPooler:
    def __init__(self, embeddings: BertEmbeddings, encoder: BertEncoder):
        self.embeddings = embeddings
        self.encoder = encoder

    def __call__(self, inputs, total_seq_len, thread_block_limit, seq_position_info, seq_position_info_tensor,
                 partition_part_index_tensor, partition_part_tensor, attention_masks=None, token_type_ids=None,
                 position_ids=None, output_layer_temp=None, intermediate_temp=None, attention_output=None,
                 test_info=None, kernel_fusion=True, balanced=True, **unused):
        roctx.range_push("embeddings")
        hidden = self.embeddings(inputs, position_ids=position_ids, token_type_ids=token_type_ids)
        roctx.range_pop()
        d = hidden.shape[1]
        dev, dt = hidden.device, hidden.dtype
        output_layer_temp = create_empty_if_none(output_layer_temp, (total_seq_len, d), dev, dt)
        attention_output = create_empty_if_none(attention_output, (total_seq_len, d), dev, dt)
        if intermediate_temp is None:
            raise ValueError("intermediate_temp [T, F] must be provided (its width defines the FFN size)")
        roctx.range_push("encoder")
        out, test_info = self.encoder(hidden_states=hidden, total_seq_len=total_seq_len,
                                      thread_block_limit=thread_block_limit, seq_position_info=seq_position_info,
                                      seq_position_info_tensor=seq_position_info_tensor,
                                      partition_part_index_tensor=partition_part_index_tensor,
                                      partition_part_tensor=partition_part_tensor, output_layer_temp=output_layer_temp,
                                      intermediate_temp=intermediate_temp, attention_output=attention_output,
                                      test_info={} if test_info is None else test_info, kernel_fusion=kernel_fusion,
                                      balanced=balanced, attention_mask=attention_masks)
        roctx.range_pop()
        return out, test_info

    @staticmethod
    def from_torch(model, async_: bool = True, dtype=torch.float16, eps=None):
        eps = model.config.layer_norm_eps if eps is None else eps
        return BertModelNoPooler(BertEmbeddings.from_torch(model.embeddings, dtype),
                                 BertEncoder.from_torch(model.encoder, async_, dtype, eps))


class PoolingType(enum.Enum):
    FIRST = "First"
    LAST = "Last"
    MEAN = "Mean"
    MAX = "Max"


PoolingMap = {PoolingType.FIRST: "First", PoolingType.LAST: "Last", PoolingType.MEAN: "Mean", PoolingType.MAX: "Max"}
_POOL_CODE = {"First": capi.RT_POOL_FIRST, "Last": capi.RT_POOL_LAST, "Mean": capi.RT_POOL_MEAN, "Max": capi.RT_POOL_MAX}


class SequencePool:
    """One row per sequence of a packed batch: the first / last token's hidden state, or the mean / maximum over
    the sequence's tokens.  The reference's class is a stub that returns its output argument
    (python/modeling_bert.py:270-277); the modes are its PoolingType (:298-314)."""

    def __init__(self, pooling_type="First"):
        if isinstance(pooling_type, PoolingType):
            pooling_type = PoolingMap[pooling_type]
        if pooling_type not in _POOL_CODE:
            raise ValueError("unknown pooling type %r" % (pooling_type,))
        self.mode = _POOL_CODE[pooling_type]

    def __call__(self, input_tensor, seq_position_info_tensor, output_tensor=None, seq_tokens=None):
        batch = seq_position_info_tensor.numel() - 1
        if output_tensor is None:
            output_tensor = torch.empty(batch, input_tensor.shape[1], dtype=input_tensor.dtype, device=input_tensor.device)
        return capi.sequence_pool(input_tensor, seq_position_info_tensor, self.mode, output_tensor, seq_tokens)


class BertPooler:
    """tanh(dense(pooled)): the BertPooler the reference has commented out (python/modeling_bert.py:279-296);
    weight arrives as [in, out] like every weight of the layers and is kept [out, in]."""

    def __init__(self, weight, bias):
        if weight.dim() != 2 or bias.numel() != weight.shape[1]:
            raise ValueError("BertPooler: weight must be [in, out] and bias [out]")
        self.weight_t = weight.t().contiguous().cuda()
        self.bias = bias.contiguous().cuda()

    def __call__(self, input_tensor, output=None):
        if output is None:
            output = torch.empty(input_tensor.shape[0], self.weight_t.shape[0], dtype=input_tensor.dtype,
                                 device=input_tensor.device)
        return capi.pooler_dense_tanh(input_tensor, self.weight_t, self.bias, output)

    @staticmethod
    def from_torch(pooler, bigbird: bool = True, dtype=torch.float16):
        """pooler: BigBirdModel.pooler (an nn.Linear; bigbird=True) or BertModel.pooler (with .dense)."""
        lin = pooler if bigbird else pooler.dense
        return BertPooler(torch.t(lin.weight.detach()).contiguous().to(dtype), lin.bias.detach().to(dtype))


class BertModel:
    """BertModelNoPooler + SequencePool + BertPooler (python/modeling_bert.py:398-440, whose from_torch leaves the
    pooler out): returns (sequence_output, pooler_output, test_info)."""

    def __init__(self, model_nopooler, pooler):
        self.bertmodel_nopooler = model_nopooler
        self.pooler = pooler

    def __call__(self, inputs, total_seq_len, thread_block_limit, seq_position_info, seq_position_info_tensor,
                 partition_part_index_tensor, partition_part_tensor, pooling_type=PoolingType.FIRST,
                 pooler_output=None, **kwargs):
        sequence_output, test_info = self.bertmodel_nopooler(
            inputs, total_seq_len, thread_block_limit, seq_position_info, seq_position_info_tensor,
            partition_part_index_tensor, partition_part_tensor, **kwargs)
        pooled = SequencePool(pooling_type)(sequence_output, seq_position_info_tensor,
                                            seq_tokens=kwargs.get("attention_masks"))
        return sequence_output, self.pooler(pooled, pooler_output), test_info

    @staticmethod
    def from_torch(model, async_: bool = True, dtype=torch.float16, eps=None, bigbird: bool = True):
        if getattr(model, "pooler", None) is None:
            raise ValueError("the torch model was built without a pooling layer")
        return BertModel(BertModelNoPooler.from_torch(model, async_, dtype, eps),
                         BertPooler.from_torch(model.pooler, bigbird, dtype))


def _model_from_checkpoint(path, heads=None, async_=True, dtype=torch.float16, eps=None, device="cuda"):
    emb, layers, cfg = checkpoint.load(path)
    heads = cfg.get("num_attention_heads") if heads is None else heads
    if heads is None:
        raise ValueError("no config.json beside the checkpoint: pass heads=")
    eps = cfg.get("layer_norm_eps", 1e-12) if eps is None else eps
    act = cfg.get("hidden_act", "gelu_new")
    if act not in ("gelu_new", "gelu_pytorch_tanh", "gelu_fast"):
        raise ValueError("the layer applies the tanh GELU; this checkpoint's hidden_act is %r" % act)
    embeddings = BertEmbeddings(emb["word_embeddings.weight"], emb["position_embeddings.weight"],
                                emb["token_type_embeddings.weight"], emb["LayerNorm.weight"], emb["LayerNorm.bias"],
                                pad_token_id=cfg.get("pad_token_id", 0), dtype=dtype, device=device)
    dev = lambda w: {k: v.detach().to(device=device, dtype=dtype).contiguous() for k, v in w.items()}
    return BertModelNoPooler(embeddings, BertEncoder.from_weights([dev(w) for w in layers], heads, async_, eps))


def _model_with_pooler_from_checkpoint(path, heads=None, async_=True, dtype=torch.float16, eps=None, device="cuda"):
    """BertModel from a checkpoint on disk that holds a pooling head (see BertModelNoPooler.from_local_checkpoint)."""
    sd, _ = checkpoint.read_state_dict(path)
    head = checkpoint.pooler_from_state_dict(sd)
    if head is None:
        raise KeyError("the checkpoint has no pooler.weight / pooler.dense.weight")
    weight, bias = (t.detach().to(device=device, dtype=dtype) for t in head)
    return BertModel(_model_from_checkpoint(path, heads, async_, dtype, eps, device), BertPooler(weight, bias))


BertModel.from_local_checkpoint = staticmethod(_model_with_pooler_from_checkpoint)
BertModelNoPooler.from_local_checkpoint = staticmethod(_model_from_checkpoint)
BertModelNoPooler.from_local_checkpoint.__doc__ = (
    "Builds the model from a HuggingFace BigBird / BERT checkpoint on disk (a directory with config.json and "
    "model.safetensors or pytorch_model.bin, or the weight file itself): the on-disk counterpart of from_torch "
    "(reference python/modeling_bert.py:62-69, :137-163).  Nothing is fetched over the network.")


def random_layer_weights(hidden, ffn, generator, std=0.02, dtype=torch.float16, device="cuda"):
    """N(0, std) weights and biases in the `[in, out]` layout, gamma = 1, beta = 0."""
    def n(*shape):
        return (torch.randn(*shape, generator=generator) * std).to(dtype).to(device)
    one = lambda k: torch.ones(k, dtype=dtype, device=device)
    zero = lambda k: torch.zeros(k, dtype=dtype, device=device)
    return {
        "qkv_weight": n(hidden, 3 * hidden), "qkv_bias": n(3 * hidden),
        "attn_out_weight": n(hidden, hidden), "attn_out_bias": n(hidden),
        "attn_ln_weight": one(hidden), "attn_ln_bias": zero(hidden),
        "inter_weight": n(hidden, ffn), "inter_bias": n(ffn),
        "out_weight": n(ffn, hidden), "out_bias": n(hidden),
        "out_ln_weight": one(hidden), "out_ln_bias": zero(hidden),
    }
