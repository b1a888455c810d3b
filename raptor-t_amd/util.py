"""Host-side batch planning for the padding-free encoder.

Mirrors python/util.py of the reference: `generate_data_metainfo` (:36-50) and
`generate_parition_plan` (:11-34) keep their names, arguments and return order; the work
is done by the C-ABI library (`rt_meta_*`) instead of Python heapq loops, and the head
count is an argument instead of the literal 12.  `generate_array_with_avg` (:78-112) and
`generate_input_data` (:114-123) produce the synthetic variable-length batches of the
reference's benchmarks.
"""
import random

import numpy as np
import torch

from . import capi


def generate_parition_plan(block_num_array, seq_start_index, thread_block_num, head_num, device="cuda"):
    """LPT plan as (partition_part_index_tensor, partition_part_tensor).  `block_num_array` is
    accepted for signature compatibility; costs are derived from the geometry."""
    seq_blocks = [0]
    for start, count in seq_start_index:
        if start != seq_blocks[-1]:
            raise ValueError("seq_start_index must be contiguous")
        seq_blocks.append(start + count)
    pos, ids = capi.partition_lpt(seq_blocks, head_num, thread_block_num)
    return torch.from_numpy(pos).to(device), torch.from_numpy(ids).to(device)


def generate_data_metainfo(input_datas, block_size, thread_block_limit, head_num=12, device="cuda"):
    """(seq_position_info, seq_position_info_tensor, total_comp_block_num,
    partition_part_index_tensor, partition_part_tensor) for a list of token sequences (or
    of sequence lengths)."""
    if block_size != 64:
        raise ValueError("the kernels are built for 64-token blocks")
    lens = [int(x) if np.isscalar(x) else len(x) for x in input_datas]
    sb = capi.seq_prefix_blocks(lens)
    _, total = capi.block_costs(sb)
    pos, ids = capi.partition_lpt(sb, head_num, thread_block_limit)
    return (sb.tolist(), torch.from_numpy(sb).to(device), int(total),
            torch.from_numpy(pos).to(device), torch.from_numpy(ids).to(device))


def generate_array_with_avg(seq_len, batch_size, max_len, rng=None):
    """Variable lengths with a given average, floored at 768, rounded to 64, capped at
    `max_len` (python/util.py:78-112)."""
    rng = rng or random
    lens = [float(rng.randint(768, max_len + 1)) for _ in range(batch_size)]
    cur = sum(lens) / batch_size
    for i in range(batch_size):
        diff = seq_len - cur
        if lens[i] + diff > max_len:
            diff = lens[i] - max_len
        elif lens[i] + diff < 768:
            diff = lens[i] - 768
        lens[i] += diff
        cur = sum(lens) / batch_size
    diff_sum = (seq_len - cur) * batch_size
    lens.sort(reverse=diff_sum >= 0)
    for i in range(batch_size):
        diff = diff_sum / (batch_size - i)
        if lens[i] + diff > max_len:
            diff = max_len - lens[i]
        elif lens[i] + diff < 768:
            diff = 768 - lens[i]
        lens[i] += diff
        diff_sum -= diff
    return [min(max(int(round(v / 64)) * 64, 64), max_len) for v in lens]


def generate_input_data(batch_size, seq_lens, vocab=30000, rng=None):
    rng = rng or np.random
    return [rng.randint(0, vocab, (seq_lens[i],)).tolist() for i in range(batch_size)]


def uniform_lengths(batch, lo, hi, seed=0, block=64):
    """`batch` lengths uniform in [lo, hi], multiples of 64 (BASELINE configs 3 and 5)."""
    rng = np.random.default_rng(seed)
    return (block * rng.integers(lo // block, hi // block + 1, size=batch)).tolist()
