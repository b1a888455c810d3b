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
    # pinned staging + asynchronous copies: a pageable copy is ordered behind everything already on the
    # stream and would make the host wait for the previous batch's layers
    up = lambda a: torch.from_numpy(a).pin_memory().to(device, non_blocking=True)
    if not str(device).startswith("cuda"):
        up = lambda a: torch.from_numpy(a).to(device)
    return sb.tolist(), up(sb), int(total), up(pos), up(ids)


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
    """`batch` lengths uniform in [lo, hi], multiples of 64 (benchmark configs 3 and 5)."""
    rng = np.random.default_rng(seed)
    return (block * rng.integers(lo // block, hi // block + 1, size=batch)).tolist()


def pack_padded_batch(input_ids, attention_mask, token_type_ids=None, block_size=64, keep_width=False):
    """Padded HuggingFace-style batch -> the packed batch the encoder takes.

    input_ids, attention_mask: [B, L] (mask 1 on real tokens, which must be a prefix of each row).  Every
    sequence keeps its real tokens plus the padding needed to fill its own last 64-token block (the
    reference only takes lengths that are multiples of 64, python/util.py:36-46): the cheapest batch, in which
    every sequence gets the attention plan of its own length.  keep_width=True keeps every sequence at the
    batch's width L (rounded up to a block) instead, whole blocks of padding included: the plan of every
    sequence is then the one HuggingFace BigBird draws for the padded batch (python/modeling_big_bird.py:573-597
    chooses it by the padded length), so the real rows equal HuggingFace run on the padded batch itself, at the
    price of computing the padding.  Returns a dict:
      input_ids, position_ids, token_type_ids : int32 [T] packed, T = sum(seq_lens)
      seq_lens   : per-sequence packed length, a multiple of block_size
      seq_tokens : per-sequence true token count (list) and `seq_tokens_tensor` (int32, on the ids' device):
                   what the layers take as `attention_mask` so that the padded keys get no weight
    """
    if input_ids.dim() != 2 or attention_mask.shape != input_ids.shape:
        raise ValueError("input_ids and attention_mask must both be [batch, length]")
    mask = attention_mask.to(torch.int64)
    tokens = mask.sum(dim=1)
    b, length = input_ids.shape
    prefix = (torch.arange(length, device=mask.device)[None, :] < tokens[:, None]).to(torch.int64)
    if not torch.equal(prefix, (mask != 0).to(torch.int64)):
        raise ValueError("attention_mask must be 1 on a prefix of each row (right padding)")
    seq_tokens = [int(x) for x in tokens.tolist()]
    if min(seq_tokens) < 1:
        raise ValueError("every sequence needs at least one token")
    seq_lens = [(n + block_size - 1) // block_size * block_size for n in seq_tokens]
    if keep_width:
        seq_lens = [(length + block_size - 1) // block_size * block_size] * b
    pad_to = max(seq_lens)
    if pad_to > length:                                   # the padded width is not a block multiple itself
        extra = pad_to - length
        input_ids = torch.nn.functional.pad(input_ids, (0, extra))
        if token_type_ids is not None:
            token_type_ids = torch.nn.functional.pad(token_type_ids, (0, extra))
    ids, pos, typ = [], [], []
    for s, n in enumerate(seq_lens):
        ids.append(input_ids[s, :n])
        pos.append(torch.arange(n, device=input_ids.device))
        typ.append(token_type_ids[s, :n] if token_type_ids is not None else torch.zeros_like(ids[-1]))
    cat = lambda xs: torch.cat(xs).to(torch.int32).contiguous()
    return {"input_ids": cat(ids), "position_ids": cat(pos), "token_type_ids": cat(typ), "seq_lens": seq_lens,
            "seq_tokens": seq_tokens,
            "seq_tokens_tensor": torch.tensor(seq_tokens, dtype=torch.int32, device=input_ids.device)}


def unpack_to_padded(packed, seq_lens, seq_tokens, length):
    """[T, D] packed encoder output -> [B, length, D] with zeros on the padded positions (the padded rows of
    the packed output are whatever the layers computed for padding tokens and are dropped here)."""
    out = packed.new_zeros(len(seq_lens), length, packed.shape[1])
    start = 0
    for s, (n, real) in enumerate(zip(seq_lens, seq_tokens)):
        out[s, :real] = packed[start:start + real]
        start += n
    return out
