"""Block-sparse attention of one packed batch, three independent CPU statements.

Test infrastructure (see oracle/__init__.py).

  bigbird_5part      the reference oracle's own algorithm for ONE sequence
                     (python/modeling_big_bird.py:516-852): q[0], q[1], q[2:-2], q[-2],
                     q[-1] handled as five parts, random keys gathered per head
                     (:978-999), all-ones masks so every -10000 penalty vanishes.
  csr_attention      what the kernel is specified to compute: for every from-block, a
                     softmax over the concatenated key blocks its CSR row LISTS
                     (duplicates kept, layers/kernels/sparse_attention.cu:3045-3174 loop).
  multiset_attention brute force in fp64: dense [L, L] scores plus log(multiplicity)
                     where a key block is listed, -inf elsewhere, textbook softmax.
Layouts: q, k, v are token-major packed `[T, H, d]`; the result is `[T, H*d]`.
Scores are `(q . k) * scale` with scale = 1/sqrt(d) (:568).
"""
import math

import numpy as np
import torch


def _bmm_t(a, b):
    return torch.matmul(a, b.transpose(-1, -2))


def bigbird_5part(q, k, v, rand_attn, block=64):
    """q, k, v: [H, L, d] fp32 tensors of one sequence; rand_attn: [H, n-2, r] int.
    Returns [L, H*d] (python/modeling_big_bird.py:851, :495)."""
    heads, length, d = q.shape
    n = length // block
    r = rand_attn.shape[-1]
    rs = 1.0 / math.sqrt(d)
    ra = torch.as_tensor(np.asarray(rand_attn), dtype=torch.long)
    bq = q.view(heads, n, block, d)
    bk = k.view(heads, n, block, d)
    bv = v.view(heads, n, block, d)
    # gathered random blocks, [H, n-2, r*block, d]                                  (:611-618)
    gk = torch.stack([bk[h][ra[h].reshape(-1)] for h in range(heads)]).view(heads, n - 2, r * block, d)
    gv = torch.stack([bv[h][ra[h].reshape(-1)] for h in range(heads)]).view(heads, n - 2, r * block, d)

    def attend(qq, kk, vv):
        return torch.matmul(torch.softmax(_bmm_t(qq, kk) * rs, dim=-1), vv)

    # part 1: first block attends to everything                                      (:631-641)
    first = attend(bq[:, 0], k, v).unsqueeze(1)
    # part 2: second block: blocks 0,1,2,last + its random blocks                    (:649-696)
    k2 = torch.cat([bk[:, 0], bk[:, 1], bk[:, 2], bk[:, -1], gk[:, 0]], dim=1)
    v2 = torch.cat([bv[:, 0], bv[:, 1], bv[:, 2], bv[:, -1], gv[:, 0]], dim=1)
    second = attend(bq[:, 1], k2, v2).unsqueeze(1)
    # part 3: middle blocks: global first, 3-block band, random, global last         (:705-774)
    ek = torch.cat([bk[:, 1:-3], bk[:, 2:-2], bk[:, 3:-1]], dim=2)
    ev = torch.cat([bv[:, 1:-3], bv[:, 2:-2], bv[:, 3:-1]], dim=2)
    mq = bq[:, 2:-2]
    inner = _bmm_t(mq, ek) * rs
    rnd = _bmm_t(mq, gk[:, 1:-1]) * rs
    fst = torch.einsum("hlqd,hkd->hlqk", mq, bk[:, 0]) * rs
    lst = torch.einsum("hlqd,hkd->hlqk", mq, bk[:, -1]) * rs
    w = torch.softmax(torch.cat([fst, inner, rnd, lst], dim=-1), dim=-1)
    mid = torch.matmul(w[..., block:4 * block], ev)
    mid = mid + torch.matmul(w[..., 4 * block:-block], gv[:, 1:-1])
    mid = mid + torch.einsum("hlqk,hkd->hlqd", w[..., :block], bv[:, 0])
    mid = mid + torch.einsum("hlqk,hkd->hlqd", w[..., -block:], bv[:, -1])
    # part 4: second-last block: blocks 0, n-3, n-2, n-1 + random                    (:783-829)
    k4 = torch.cat([bk[:, 0], bk[:, -3], bk[:, -2], bk[:, -1], gk[:, -1]], dim=1)
    v4 = torch.cat([bv[:, 0], bv[:, -3], bv[:, -2], bv[:, -1], gv[:, -1]], dim=1)
    second_last = attend(bq[:, -2], k4, v4).unsqueeze(1)
    # part 5: last block attends to everything                                       (:836-843)
    last = attend(bq[:, -1], k, v).unsqueeze(1)
    ctx = torch.cat([first, second, mid, second_last, last], dim=1).reshape(heads, length, d)
    return ctx.transpose(0, 1).reshape(length, heads * d)


def full_attention(q, k, v):
    """Dense attention of one sequence, [H, L, d] -> [L, H*d]; what sequences of at most
    704 tokens get (python/modeling_big_bird.py:2079-2094)."""
    heads, length, d = q.shape
    w = torch.softmax(_bmm_t(q, k) / math.sqrt(d), dim=-1)
    return torch.matmul(w, v).transpose(0, 1).reshape(length, heads * d)


def csr_attention(q, k, v, seq_blocks, to_idx, to_pos, plan_heads, block=64, scale=None, seq_tokens=None):
    """q, k, v: [T, H, d] tensors (any float dtype; computed in fp32).  Row of (head h,
    global from-block g) is `(h if plan_heads > 1 else 0) * NB + g`.

    seq_tokens (optional): true token count of each sequence; the positions from there to the end of
    the sequence's last block are padding and get no attention weight as keys (what the to_mask /
    band_mask / rand_mask terms of python/modeling_big_bird.py:640-760 do with -10000).  Padded
    query rows are computed like any other (HuggingFace zeroes them afterwards, :1013)."""
    t, heads, d = q.shape
    scale = 1.0 / math.sqrt(d) if scale is None else scale
    q, k, v = q.float(), k.float(), v.float()
    nb_total = seq_blocks[-1]
    out = torch.empty(t, heads, d, dtype=torch.float32)
    to_idx = np.asarray(to_idx)
    to_pos = np.asarray(to_pos)
    for s in range(len(seq_blocks) - 1):
        t0 = seq_blocks[s] * block
        n = seq_blocks[s + 1] - seq_blocks[s]
        ks = k[t0:t0 + n * block].view(n, block, heads, d)
        vs = v[t0:t0 + n * block].view(n, block, heads, d)
        for h in range(heads):
            hp = h if plan_heads > 1 else 0
            for i in range(n):
                row = hp * nb_total + seq_blocks[s] + i
                blocks = torch.as_tensor(to_idx[to_pos[row]:to_pos[row + 1]], dtype=torch.long)
                kk = ks[blocks, :, h].reshape(-1, d)
                vv = vs[blocks, :, h].reshape(-1, d)
                qq = q[t0 + i * block: t0 + (i + 1) * block, h]
                sc = qq @ kk.t() * scale
                if seq_tokens is not None:
                    key_pos = (blocks[:, None] * block + torch.arange(block)[None, :]).reshape(-1)
                    sc = sc.masked_fill((key_pos >= int(seq_tokens[s]))[None, :], float("-inf"))
                w = torch.softmax(sc, dim=-1)
                out[t0 + i * block: t0 + (i + 1) * block, h] = w @ vv
    return out.reshape(t, heads * d)


def multiset_attention(q, k, v, seq_blocks, to_idx, to_pos, plan_heads, block=64, scale=None, seq_tokens=None):
    """Brute force in fp64 (small inputs only); seq_tokens as in csr_attention."""
    t, heads, d = q.shape
    scale = 1.0 / math.sqrt(d) if scale is None else scale
    q, k, v = q.double(), k.double(), v.double()
    nb_total = seq_blocks[-1]
    out = torch.empty(t, heads, d, dtype=torch.float64)
    for s in range(len(seq_blocks) - 1):
        t0 = seq_blocks[s] * block
        n = seq_blocks[s + 1] - seq_blocks[s]
        length = n * block
        for h in range(heads):
            hp = h if plan_heads > 1 else 0
            count = torch.zeros(n, n, dtype=torch.float64)
            for i in range(n):
                row = hp * nb_total + seq_blocks[s] + i
                for j in to_idx[to_pos[row]:to_pos[row + 1]]:
                    count[i, int(j)] += 1.0
            bias = torch.log(count).repeat_interleave(block, 0).repeat_interleave(block, 1)
            if seq_tokens is not None:
                bias[:, int(seq_tokens[s]):] = float("-inf")
            sc = q[t0:t0 + length, h] @ k[t0:t0 + length, h].t() * scale + bias
            sc = sc - sc.max(dim=-1, keepdim=True).values
            e = torch.exp(sc)
            out[t0:t0 + length, h] = (e / e.sum(dim=-1, keepdim=True)) @ v[t0:t0 + length, h]
    return out.reshape(t, heads * d)
