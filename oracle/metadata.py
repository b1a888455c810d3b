"""Host metadata of the padding-free block-sparse layer, restated in Python.

Test infrastructure (see oracle/__init__.py).  Follows
  * layers/multi_headed_attention.cpp:15-140  (to-block CSR, one row per from-block)
  * python/util.py:11-34, :36-50              (LPT work plan, batch geometry)
  * python/modeling_big_bird.py:631-836       (which key blocks each from-block reads)
"""
import heapq

import numpy as np

from . import plans

MIN_SPARSE_BLOCKS = 12   # (5 + 2*3) * 64 = 704 tokens and below run full attention
                         # (python/modeling_big_bird.py:2079-2094)


def seq_prefix_blocks(seq_lens, block=64):
    """`seq_position_info`: prefix sums of per-sequence block counts (python/util.py:37,45)."""
    out = [0]
    for length in seq_lens:
        if length % block != 0 or length <= 0:
            raise ValueError("sequence length must be a positive multiple of the block size")
        out.append(out[-1] + length // block)
    return out


def row_blocks(i, n, rand_row):
    """Key-block list of from-block i in an n-block sequence, in the reference's row
    order (layers/multi_headed_attention.cpp:44-125) with the three random entries taken
    from `rand_row` (python/modeling_big_bird.py:649-658, :705-747, :783-792)."""
    if n < MIN_SPARSE_BLOCKS or i == 0 or i == n - 1:
        return list(range(n))
    r = [int(x) for x in rand_row]
    if i == 1:
        return [0, 1, 2, n - 1] + r
    if i == 2:
        return [1, 2, 3, n - 1, 0] + r
    if i == n - 2:
        return [i - 1, i, i + 1, 0] + r
    return [i - 1, i, i + 1, 0, n - 1] + r


def to_index_from_rand_attn(seq_blocks, rand_attn_per_seq, plan_heads):
    """CSR (to_idx, to_pos) with row `hp * NB + g` for plan head hp and global from-block g.
    `rand_attn_per_seq[s]` is [plan_heads, n_s-2, 3] (ignored for n_s < 12)."""
    nb_total = seq_blocks[-1]
    idx, pos = [], [0]
    for hp in range(plan_heads):
        for s in range(len(seq_blocks) - 1):
            n = seq_blocks[s + 1] - seq_blocks[s]
            for i in range(n):
                rr = None
                if n >= MIN_SPARSE_BLOCKS and 0 < i < n - 1:
                    rr = rand_attn_per_seq[s][hp][i - 1]
                idx.extend(row_blocks(i, n, rr))
                pos.append(len(idx))
    assert len(pos) == plan_heads * nb_total + 1
    return np.array(idx, dtype=np.int32), np.array(pos, dtype=np.int32)


def hf_to_index(seq_lens, seed, heads, max_pos=4096, block=64,
                policy=plans.POLICY_REFERENCE_PATCHED):
    """The per-head CSR of the plan the reference's oracle draws for each sequence of a
    packed batch in the layer with seed `seed` (each sequence alone, batch 1)."""
    sb = seq_prefix_blocks(seq_lens, block)
    ras = []
    for length in seq_lens:
        if length // block >= MIN_SPARSE_BLOCKS:
            ras.append(plans.rand_attn_for_length(length, seed, heads, max_pos, block, 3, policy))
        else:
            ras.append(None)
    return to_index_from_rand_attn(sb, ras, heads)


def reference_random_candidates(i, n):
    """Legal random to-blocks of from-block i under the reference's own generator
    (layers/multi_headed_attention.cpp:52-123): the slice each branch shuffles."""
    if i == 1:
        return list(range(3, n - 1))
    if i == 2:
        return list(range(4, n - 1))
    if i == n - 3:
        return list(range(1, n - 4))
    if i == n - 2:
        return list(range(1, n - 3))
    return [b for b in range(1, n - 1) if b not in (i - 1, i, i + 1)]


def reference_to_index(seq_blocks, rng):
    """Head-shared CSR with the reference's generator; `rng` (numpy RandomState) replaces
    the unseeded std::mt19937 of the reference, so only the structure is comparable."""
    ras = []
    for s in range(len(seq_blocks) - 1):
        n = seq_blocks[s + 1] - seq_blocks[s]
        if n < MIN_SPARSE_BLOCKS:
            ras.append(None)
            continue
        ra = np.zeros((1, n - 2, 3), dtype=np.int32)
        for i in range(1, n - 1):
            ra[0, i - 1] = rng.permutation(reference_random_candidates(i, n))[:3]
        ras.append(ra)
    return to_index_from_rand_attn(seq_blocks, ras, 1)


def block_costs(seq_blocks):
    """Per from-block cost `[n, 7, 8 x (n-4), 7, n]` per sequence (python/util.py:38-44);
    sequences below 12 blocks run full attention, every block costs n (the reference
    never builds such a batch: its lengths start at 768 tokens)."""
    out = []
    for s in range(len(seq_blocks) - 1):
        n = seq_blocks[s + 1] - seq_blocks[s]
        if n < MIN_SPARSE_BLOCKS:
            out.extend([n] * n)
        else:
            out.extend([n, 7] + [8] * (n - 4) + [7, n])
    return out


def lpt_partition(costs, seq_blocks, n_cta, heads):
    """Longest-processing-time plan (python/util.py:11-34): blocks by descending cost
    (stable), each (block, head) unit to the least-loaded CTA; unit id =
    `blk_in_seq + head * n_seq + seq_start * heads`.  Returns (pos[n_cta+1], ids)."""
    order = sorted(range(len(costs)), key=lambda b: -costs[b])      # stable, descending
    parts = [[] for _ in range(n_cta)]
    heap = [(0, c) for c in range(n_cta)]
    starts = [(seq_blocks[s], seq_blocks[s + 1] - seq_blocks[s]) for s in range(len(seq_blocks) - 1)]
    for b in order:
        st, n = 0, 0
        for cand in starts:
            if b >= cand[0]:
                st, n = cand
            else:
                break
        for h in range(heads):
            load, cta = heapq.heappop(heap)
            parts[cta].append(b - st + h * n + st * heads)
            heapq.heappush(heap, (load + costs[b], cta))
    pos = [0]
    for p in parts:
        pos.append(pos[-1] + len(p))
    ids = [u for p in parts for u in p]
    return np.array(pos, dtype=np.int32), np.array(ids, dtype=np.int32)


def data_metainfo(seq_lens, block, n_cta, heads=12):
    """python/util.py:36-50: (seq prefix blocks, total cost, plan pos, plan ids)."""
    sb = seq_prefix_blocks(seq_lens, block)
    costs = block_costs(sb)
    pos, ids = lpt_partition(costs, sb, n_cta, heads)
    return sb, int(sum(costs)), pos, ids


def decode_unit(unit, seq_blocks, heads):
    """(seq, head, block-in-seq) of a flat unit id."""
    for s in range(len(seq_blocks) - 1):
        if seq_blocks[s] * heads <= unit < seq_blocks[s + 1] * heads:
            n = seq_blocks[s + 1] - seq_blocks[s]
            rem = unit - seq_blocks[s] * heads
            return s, rem // n, rem % n
    raise ValueError("unit id out of range")
