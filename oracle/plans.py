"""Random-block plans of BigBird attention, restated with numpy's legacy RNG.

Test infrastructure (see oracle/__init__.py).  Follows the reference's patched
HuggingFace copy, python/modeling_big_bird.py:
  * plan selection                     :573-597
  * `_get_rand_attn_plan`              :1039-1069
  * `_bigbird_block_rand_mask`         :1072-1125
  * `_bigbird_block_rand_mask_with_head` :1127-1258
  * `_get_single_block_row_attention`  :1261-1314
The global numpy RNG is consumed exactly as the reference consumes it
(`np.random.seed(seed)` once, then one `np.random.permutation` per row/head in
the reference's loop order), so a plan is a pure function of (length, seed).
"""
import numpy as np

BLOCK = 64
NUM_RAND = 3


def rand_attn_max_plan(max_len, block=BLOCK, r=NUM_RAND, last_idx=-1):
    """One head's plan for a `max_len`-token sequence; rows for from-blocks
    1..nb-2, `r` random to-blocks each (python/modeling_big_bird.py:1072-1125).
    With `last_idx` > 2*block the candidates stop before block last_idx//block-1."""
    nb = max_len // block
    out = np.zeros((nb - 2, r), dtype=np.int32)
    mid = np.arange(1, nb - 1, dtype=np.int32)
    last = nb - 1
    if last_idx > 2 * block:
        last = last_idx // block - 1
    for i in range(1, nb - 1):
        lo, hi = i - 2, i
        if i == 1:
            cand = mid[2:last]
        elif i == 2:
            cand = mid[3:last]
        elif i == nb - 3 or i == nb - 2:
            cand = mid[:last]
        elif lo > last:
            cand = mid[:last]
        elif hi + 1 == last:
            cand = mid[:lo]
        else:
            cand = np.concatenate((mid[:lo], mid[hi + 1:last]))
        out[i - 1, :] = np.random.permutation(cand)[:r]
    return out


def rand_attn_plan(length, block=BLOCK, r=NUM_RAND):
    """(plan_from_length, plan_num_rand_blocks), python/modeling_big_bird.py:1039-1069."""
    nb = length // block
    if 2 * r + 5 < nb:
        return [int((2 * r + 5) * block), length], [r, 0]
    if r + 5 < nb:
        return [int((r + 5) * block), length], [r // 2, r - r // 2]
    return [length], [r]


def single_block_row_attention(block_id, to_start, to_end, num_rand,
                               win_left=1, win_right=1, glob_left=1, glob_right=1):
    """Random to-blocks of one from-block row: the first `num_rand` legal entries
    of a permutation of [to_start, to_end) (python/modeling_big_bird.py:1261-1314)."""
    perm = np.random.permutation(np.arange(to_start, to_end, dtype=np.int32))
    illegal = set(range(block_id - win_left, block_id + win_right + 1))
    illegal.update(range(glob_left))
    illegal.update(range(to_end - glob_right, to_end))
    if block_id == 1:
        illegal.add(to_end - 2)
    if block_id == to_end - 2:
        illegal.add(1)
    picked = []
    for b in perm[: to_end - to_start]:
        if int(b) not in illegal:
            picked.append(int(b))
        if len(picked) == num_rand:
            break
    return np.array(picked, dtype=np.int32)


def rand_attn_with_head(length, heads, plan_from_length, plan_num_rand, block=BLOCK,
                        glob_top=1, glob_bottom=1):
    """Per-head planned variant, python/modeling_big_bird.py:1127-1258.
    Returns a list of `heads` arrays [nb-2, sum(plan_num_rand)]."""
    nb = length // block
    plan_blocks = [p // block for p in plan_from_length]
    max_plan = plan_from_length.index(length)
    width = int(np.sum(plan_num_rand[: max_plan + 1]))
    rand = [np.zeros((nb, width), dtype=np.int32) for _ in range(heads)]

    def fill(row, c0, c1, to_start, to_end, count):
        for h in range(heads):
            rand[h][row, c0:c1] = single_block_row_attention(row, to_start, to_end, count)

    for p in range(max_plan + 1):
        c0 = 0
        if p > 0:
            if plan_num_rand[p] > 0:
                c0 = int(np.sum(plan_num_rand[:p]))
                c1 = int(np.sum(plan_num_rand[: p + 1]))
                for row in range(glob_top, plan_blocks[p - 1]):
                    fill(row, c0, c1, plan_blocks[p - 1], plan_blocks[p], plan_num_rand[p])
            for q in range(p):
                if plan_num_rand[q] == 0:
                    continue
                for row in range(plan_blocks[p - 1], plan_blocks[p]):
                    c0, to_start = 0, 0
                    if q > 0:
                        c0 = int(np.sum(plan_num_rand[:q]))
                        to_start = plan_blocks[q - 1]
                    c1 = int(np.sum(plan_num_rand[: q + 1]))
                    fill(row, c0, c1, to_start, plan_blocks[q], plan_num_rand[q])
        if plan_num_rand[p] == 0:
            continue
        c1 = int(np.sum(plan_num_rand[: p + 1]))
        from_start, to_start = glob_top, 0
        if p > 0:
            c0 = int(np.sum(plan_num_rand[:p]))
            from_start = plan_blocks[p - 1]
            to_start = plan_blocks[p - 1]
        for row in range(from_start, plan_blocks[p]):
            fill(row, c0, c1, to_start, plan_blocks[p], plan_num_rand[p])
    return [a[glob_top: nb - glob_bottom, :] for a in rand]


POLICY_REFERENCE_PATCHED = "reference_patched"
POLICY_HF_UPSTREAM = "hf_upstream"


def uses_max_plan(length, policy=POLICY_REFERENCE_PATCHED):
    """Which generator a length selects.  The reference patched the upstream test
    `length in [1024, 3072, 4096]` into `length % 256 == 0`
    (python/modeling_big_bird.py:574); below 1024 tokens that plan would name
    blocks past the end of the sequence, so it is only honoured from 1024 up."""
    if policy == POLICY_HF_UPSTREAM:
        return length in (1024, 3072, 4096)
    return length % 256 == 0 and length >= 1024


def rand_attn_for_length(length, seed, heads, max_pos=4096, block=BLOCK, r=NUM_RAND,
                         policy=POLICY_REFERENCE_PATCHED):
    """The [heads, nb-2, r] plan the reference's oracle draws for one sequence of
    `length` tokens in the layer whose seed is `seed` (= layer index,
    python/modeling_big_bird.py:573-597, :1577)."""
    np.random.seed(seed)
    nb = length // block
    if uses_max_plan(length, policy):
        per_head = [rand_attn_max_plan(max_pos, block, r, last_idx=1024)[: nb - 2]
                    for _ in range(heads)]
    else:
        pfl, pnr = rand_attn_plan(length, block, r)
        per_head = rand_attn_with_head(length, heads, pfl, pnr, block)
    return np.stack(per_head, axis=0).astype(np.int32)
