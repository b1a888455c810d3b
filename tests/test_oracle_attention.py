"""The three CPU statements of block-sparse attention against the HuggingFace golden
outputs, against each other, and against cases the mathematics fixes."""
import math
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import attention as oa
from oracle import metadata as md
from oracle import plans


def _inputs(length, heads, seed):
    rs = np.random.RandomState(seed)
    return [torch.from_numpy(rs.standard_normal((heads, length, 64)).astype(np.float32)) for _ in range(3)]


@pytest.mark.parametrize("name", ["L1024_H2_seed0", "L832_H2_seed3"])
def test_5part_and_csr_match_hf_golden(golden_dir, name):
    g = np.load(os.path.join(golden_dir, "hf_attention.npz"))
    length, heads, seed, in_seed = (int(x) for x in g[name + "_meta"])
    want = torch.from_numpy(g[name + "_out"])
    q, k, v = _inputs(length, heads, in_seed)
    ra = plans.rand_attn_for_length(length, seed, heads)
    got5 = oa.bigbird_5part(q, k, v, ra)
    assert (got5 - want).abs().max().item() < 2e-6
    idx, pos = md.hf_to_index([length], seed, heads)
    qt, kt, vt = (x.transpose(0, 1).contiguous() for x in (q, k, v))
    got_csr = oa.csr_attention(qt, kt, vt, [0, length // 64], idx, pos, heads)
    assert (got_csr - want).abs().max().item() < 2e-6


def test_csr_equals_bruteforce_with_duplicates():
    torch.manual_seed(1)
    lens = [768, 512, 1024]
    heads = 2
    sb = md.seq_prefix_blocks(lens)
    idx, pos = md.hf_to_index(lens, 0, heads)
    # the 1024-token max-length plan draws from blocks 1..15, block 15 is also the last global block
    dup = any(len(set(idx[pos[r]:pos[r + 1]].tolist())) < pos[r + 1] - pos[r] for r in range(len(pos) - 1))
    assert dup
    t = sb[-1] * 64
    q, k, v = (torch.randn(t, heads, 64) for _ in range(3))
    a = oa.csr_attention(q, k, v, sb, idx, pos, heads)
    b = oa.multiset_attention(q, k, v, sb, idx, pos, heads)
    assert (a.double() - b).abs().max().item() < 1e-5


def test_dense_rows_and_full_plan_reduce_to_sdpa():
    torch.manual_seed(2)
    n, heads = 13, 2
    length = n * 64
    q, k, v = (torch.randn(length, heads, 64) for _ in range(3))
    idx, pos = md.hf_to_index([length], 0, heads)
    got = oa.csr_attention(q, k, v, [0, n], idx, pos, heads).view(length, heads, 64)
    ref = F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1)).transpose(0, 1)
    assert (got[:64] - ref[:64]).abs().max().item() < 1e-5              # from-block 0
    assert (got[-64:] - ref[-64:]).abs().max().item() < 1e-5            # from-block n-1
    assert (got[64:128] - ref[64:128]).abs().max().item() > 1e-3        # a sparse row differs
    full_idx = np.tile(np.arange(n, dtype=np.int32), n)
    full_pos = np.arange(0, n * n + 1, n, dtype=np.int32)
    got_full = oa.csr_attention(q, k, v, [0, n], full_idx, full_pos, 1).view(length, heads, 64)
    assert (got_full - ref).abs().max().item() < 1e-5
    assert (oa.full_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1)).view(length, heads, 64)
            - ref).abs().max().item() < 1e-5


def test_invariants_constant_v_permutation_duplicate_mass():
    torch.manual_seed(3)
    n, heads = 12, 1
    length = n * 64
    q, k, v = (torch.randn(length, heads, 64) for _ in range(3))
    idx, pos = md.hf_to_index([length], 1, heads)
    vc = torch.ones_like(v) * 0.37
    assert (oa.csr_attention(q, k, vc, [0, n], idx, pos, 1) - 0.37).abs().max().item() < 1e-6
    # order of the key blocks inside a row does not matter
    idx2 = idx.copy()
    for r in range(n):
        idx2[pos[r]:pos[r + 1]] = idx2[pos[r]:pos[r + 1]][::-1]
    a = oa.csr_attention(q, k, v, [0, n], idx, pos, 1)
    assert (a - oa.csr_attention(q, k, v, [0, n], idx2, pos, 1)).abs().max().item() < 1e-5
    # listing a block twice doubles its probability mass: one from-block, keys {0, 0, 1}
    q1, k1, v1 = q[:128], k[:128], v[:128]
    two = oa.csr_attention(q1, k1, v1, [0, 2], np.array([0, 0, 1, 0, 1], np.int32), np.array([0, 3, 5], np.int32), 1)
    s = (q1[:64, 0] @ k1[:, 0].t()) / math.sqrt(64)
    e = torch.exp(s - s.max(-1, keepdim=True).values)
    e[:, :64] *= 2
    want = (e / e.sum(-1, keepdim=True)) @ v1[:, 0]
    assert (two[:64] - want).abs().max().item() < 1e-5


@pytest.mark.parametrize("name", ["L832_H2_seed3_len800", "L1024_H2_seed0_len961"])
def test_padded_tail_matches_hf_golden(golden_dir, name):
    """HuggingFace's own masks on a sequence whose last block is partly padding (tests/golden/
    make_hf_goldens.py) against the oracle's key masking; the padded query rows, which HuggingFace
    zeroes, are left out.  Masking the wrong side of the boundary, or by block instead of by token,
    fails this; so does ignoring the mask (checked against the unmasked golden below)."""
    g = np.load(os.path.join(golden_dir, "hf_attention.npz"))
    length, heads, seed, in_seed, tokens = (int(x) for x in g[name + "_meta"])
    want = torch.from_numpy(g[name + "_out"])
    q, k, v = _inputs(length, heads, in_seed)
    idx, pos = md.hf_to_index([length], seed, heads)
    qt, kt, vt = (x.transpose(0, 1).contiguous() for x in (q, k, v))
    got = oa.csr_attention(qt, kt, vt, [0, length // 64], idx, pos, heads, seq_tokens=[tokens])
    assert (got[:tokens] - want[:tokens]).abs().max().item() < 2e-6
    assert want[tokens:].abs().max().item() == 0.0
    unmasked = oa.csr_attention(qt, kt, vt, [0, length // 64], idx, pos, heads)
    assert (unmasked[:tokens] - want[:tokens]).abs().max().item() > 1e-3
    brute = oa.multiset_attention(qt, kt, vt, [0, length // 64], idx, pos, heads, seq_tokens=[tokens])
    assert (brute[:tokens].float() - want[:tokens]).abs().max().item() < 2e-5
