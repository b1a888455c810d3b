"""Layer glue and epilogues of the oracle against library routines."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import layer as ol
from oracle import metadata as md


def test_gelu_constants_and_library():
    x = torch.linspace(-6, 6, 1001)
    b = torch.zeros(1001)
    hand = 0.5 * x * (1 + torch.tanh(ol.GELU_C0 * (x + ol.GELU_C1 * x ** 3)))
    assert (ol.bias_gelu(x, b) - hand).abs().max().item() < 1e-6
    assert abs(ol.GELU_C0 - math.sqrt(2 / math.pi)) < 1e-12


def test_layernorm_by_hand():
    torch.manual_seed(0)
    x, r = torch.randn(5, 768), torch.randn(5, 768)
    b, g, be = torch.randn(768), torch.randn(768), torch.randn(768)
    h = (x + b + r).double()
    mu = h.mean(-1, keepdim=True)
    var = ((h - mu) ** 2).mean(-1, keepdim=True)
    want = (h - mu) / torch.sqrt(var + 1e-5) * g.double() + be.double()
    assert (ol.bias_residual_layernorm(x, r, b, g, be, 1e-5).double() - want).abs().max().item() < 1e-5


def test_qkv_split_is_reshape_permute():
    torch.manual_seed(0)
    qkv, bias = torch.randn(128, 3 * 768), torch.randn(3 * 768)
    q, k, v = ol.qkv_bias_split(qkv, bias, 12)
    full = (qkv + bias).view(128, 3, 12, 64)
    assert torch.equal(q, full[:, 0] * 0.125) and torch.equal(k, full[:, 1]) and torch.equal(v, full[:, 2])


def test_layer_composition_matches_plain_torch_modules():
    """One 12-block sequence forced to full attention == a textbook post-LN encoder layer."""
    torch.manual_seed(0)
    g = torch.Generator().manual_seed(0)
    hid, ffn, heads = 128, 256, 2
    w = ol.random_layer_weights(hid, ffn, g, std=0.2)
    n = 4
    x = torch.randn(n * 64, hid)
    idx, pos = md.hf_to_index([n * 64], 0, heads)          # n < 12 -> every row lists all blocks
    got = ol.encoder_layer(x, w, heads, [0, n], idx, pos, heads, eps=1e-5)
    qkv = x @ w["qkv_weight"] + w["qkv_bias"]
    q, k, v = (t.view(n * 64, heads, 64).transpose(0, 1) for t in qkv.split(hid, dim=1))
    ctx = F.scaled_dot_product_attention(q, k, v).transpose(0, 1).reshape(n * 64, hid)
    a = F.layer_norm(ctx @ w["attn_out_weight"] + w["attn_out_bias"] + x, (hid,), w["attn_ln_weight"], w["attn_ln_bias"], 1e-5)
    i = F.gelu(a @ w["inter_weight"] + w["inter_bias"], approximate="tanh")
    want = F.layer_norm(i @ w["out_weight"] + w["out_bias"] + a, (hid,), w["out_ln_weight"], w["out_ln_bias"], 1e-5)
    assert (got - want).abs().max().item() < 2e-5


def test_embeddings_layernorm_matches_torch_modules_and_hand_case():
    """The restatement indexes and normalises by hand; torch's own Embedding + LayerNorm modules (what the
    reference calls, python/modeling_bert.py:31-36,53-62) are the independent answer.  A dropped table,
    a swapped id stream or an unbiased variance each fail it."""
    g = torch.Generator().manual_seed(5)
    vocab, max_pos, types, hidden, t = 97, 33, 2, 24, 50
    word, pos, typ = (torch.randn(n, hidden, generator=g) for n in (vocab, max_pos, types))
    gamma, beta = torch.randn(hidden, generator=g), torch.randn(hidden, generator=g)
    ids = torch.randint(0, vocab, (t,), generator=g)
    pids = torch.randint(0, max_pos, (t,), generator=g)
    tids = torch.randint(0, types, (t,), generator=g)
    got = ol.embeddings_layernorm(ids, pids, tids, word, pos, typ, gamma, beta, eps=1e-12)
    ln = torch.nn.LayerNorm(hidden, eps=1e-12)
    with torch.no_grad():
        ln.weight.copy_(gamma)
        ln.bias.copy_(beta)
        want = ln(torch.nn.functional.embedding(ids, word) + torch.nn.functional.embedding(tids, typ)
                  + torch.nn.functional.embedding(pids, pos))
    assert (got - want).abs().max().item() <= 2e-5
    # hand case: rows sum to [1, 3] -> mean 2, biased variance 1 -> [-1, 1] * gamma + beta
    w = torch.tensor([[0.0, 1.0], [5.0, 5.0]]); p = torch.tensor([[1.0, 1.0]]); ty = torch.tensor([[0.0, 1.0]])
    out = ol.embeddings_layernorm(torch.tensor([0]), torch.tensor([0]), torch.tensor([0]), w, p, ty,
                                  torch.tensor([2.0, 3.0]), torch.tensor([0.5, -0.5]), eps=0.0)
    assert torch.allclose(out, torch.tensor([[-1.5, 2.5]]), atol=1e-6)


def test_sequence_pool_and_pooler_match_torch_and_hand_cases():
    """sequence_pool against per-sequence torch reductions written out here and a hand case; pooler against
    torch's own Linear + Tanh modules (HuggingFace BigBirdModel: activation(pooler(sequence_output[:, 0])))."""
    g = torch.Generator().manual_seed(8)
    seq_blocks = [0, 2, 3, 6]
    hidden = torch.randn(6 * 64, 16, generator=g)
    tokens = [100, 64, 131]
    for mode, fn in (("First", lambda x: x[0]), ("Last", lambda x: x[-1]), ("Mean", lambda x: x.mean(0)),
                     ("Max", lambda x: x.amax(0))):
        full = ol.sequence_pool(hidden, seq_blocks, mode)
        cut = ol.sequence_pool(hidden, seq_blocks, mode, seq_tokens=tokens)
        for s in range(3):
            t0, n = seq_blocks[s] * 64, (seq_blocks[s + 1] - seq_blocks[s]) * 64
            assert torch.allclose(full[s], fn(hidden[t0:t0 + n]), atol=1e-6)
            assert torch.allclose(cut[s], fn(hidden[t0:t0 + tokens[s]]), atol=1e-6)
    ramp = torch.arange(64, dtype=torch.float32)[:, None].repeat(1, 2)
    assert ol.sequence_pool(ramp, [0, 1], "Mean").tolist() == [[31.5, 31.5]]
    assert ol.sequence_pool(ramp, [0, 1], "Last", seq_tokens=[10]).tolist() == [[9.0, 9.0]]
    with pytest.raises(ValueError):
        ol.sequence_pool(ramp, [0, 1], "Median")
    lin = torch.nn.Linear(16, 12)
    x = torch.randn(5, 16, generator=g)
    with torch.no_grad():
        want = torch.tanh(lin(x))
        got = ol.pooler(x, lin.weight.t().contiguous(), lin.bias)
    assert (got - want).abs().max().item() <= 1e-6
    one = ol.pooler(torch.tensor([[1.0, 2.0]]), torch.tensor([[0.5], [0.25]]), torch.tensor([-1.0]))
    assert abs(one.item() - 0.0) < 1e-7                       # tanh(0.5 + 0.5 - 1)


def test_stored_tensors_option_rounds_between_kernels_only():
    """encoder_layer(store_dtype=...) rounds every tensor that passes from one kernel to the next and nothing else:
    with fp32 as the storage type it is the plain layer, with bf16 the output is a bf16 value everywhere and stays
    within a few bf16 ulp of the plain layer."""
    from oracle import metadata as md
    g = torch.Generator().manual_seed(0)
    hidden, heads, ffn, lens = 128, 2, 256, [832, 128]
    w = ol.random_layer_weights(hidden, ffn, g)
    x = torch.randn(sum(lens), hidden, generator=g)
    sb = md.seq_prefix_blocks(lens)
    idx, pos = md.hf_to_index(lens, 0, heads)
    plain = ol.encoder_layer(x, w, heads, sb, idx, pos, heads)
    same = ol.encoder_layer(x, w, heads, sb, idx, pos, heads, store_dtype=torch.float32)
    assert torch.equal(plain, same)
    rounded = ol.encoder_layer(x, w, heads, sb, idx, pos, heads, store_dtype=torch.bfloat16)
    assert torch.equal(rounded, rounded.to(torch.bfloat16).float())
    err = (rounded - plain).abs().max().item()
    assert 0 < err <= 0.1, err
    # the projection stored once, with its bias: the plain layer in fp32 (the sum of two fp32 roundings apart),
    # another set of bf16 roundings (not the same values, the same size of error) in bf16
    same = ol.encoder_layer(x, w, heads, sb, idx, pos, heads, store_dtype=torch.float32, bias_in_projection=True)
    assert (plain - same).abs().max().item() <= 1e-5
    once = ol.encoder_layer(x, w, heads, sb, idx, pos, heads, store_dtype=torch.bfloat16, bias_in_projection=True)
    assert torch.equal(once, once.to(torch.bfloat16).float()) and not torch.equal(once, rounded)
    assert 0 < (once - plain).abs().max().item() <= 0.1
