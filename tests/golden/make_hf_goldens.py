"""Write golden vectors from the HuggingFace BigBird code installed in the
authoring container (the `transformers` package; the reference's
python/modeling_big_bird.py is a patched copy of the same file and is not
importable on its own).  Run once, by hand, in the authoring container:

    python tests/golden/make_hf_goldens.py

Outputs (committed, small):
  hf_plans.json           random-block plans rand_attn[H][n-2][3] for several
                          (length, seed): the per-head planned generator
                          (lengths with L % 256 != 0) and the truncated
                          max-length generator (last_idx=1024), drawn in the
                          order python/modeling_big_bird.py:573-597 draws them.
  hf_attention.npz        fp32 outputs of `bigbird_block_sparse_attention` for
                          two tiny single-sequence cases with all-ones masks;
                          the inputs are regenerated from numpy RandomState
                          seeds recorded in the file.  Two more cases carry a padded
                          tail (attention mask 0 on the last positions).
The module is put in train() mode because upstream returns an all-zero plan in
eval mode, a guard the reference deleted.
"""
import json
import os

import numpy as np
import torch
from transformers import BigBirdConfig
from transformers.models.big_bird.modeling_big_bird import (
    BigBirdBlockSparseAttention, BigBirdModel)

HERE = os.path.dirname(os.path.abspath(__file__))


def make_attn(heads, max_pos=4096, seed=0):
    cfg = BigBirdConfig(hidden_size=64 * heads, num_attention_heads=heads, block_size=64,
                        num_random_blocks=3, max_position_embeddings=max_pos,
                        attention_type="block_sparse")
    m = BigBirdBlockSparseAttention(cfg, seed=seed)
    m.train()
    return m


def hf_plan(length, seed, heads, max_pos, use_max_plan):
    m = make_attn(heads, max_pos, seed)
    np.random.seed(seed)
    if use_max_plan:
        ra = [m._bigbird_block_rand_mask(max_pos, max_pos, 64, 64, 3, last_idx=1024)[: length // 64 - 2]
              for _ in range(heads)]
    else:
        pfl, pnr = m._get_rand_attn_plan(length, 64, 3)
        ra = m._bigbird_block_rand_mask_with_head(
            from_seq_length=length, to_seq_length=length, from_block_size=64, to_block_size=64,
            num_heads=heads, plan_from_length=pfl, plan_num_rand_blocks=pnr)
    return np.stack(ra, axis=0)


def inputs(length, heads, seed):
    rs = np.random.RandomState(seed)
    q, k, v = (rs.standard_normal((heads, length, 64)).astype(np.float32) for _ in range(3))
    return q, k, v


def hf_attention(length, heads, seed, in_seed, tokens=None):
    """tokens: true length of the sequence; positions from there to `length` are padding (attention mask 0)."""
    m = make_attn(heads, 4096, seed)
    q, k, v = (torch.from_numpy(a)[None] for a in inputs(length, heads, in_seed))
    mask = torch.ones(1, length)
    if tokens is not None:
        mask[:, tokens:] = 0.0
    blocked, band, fmask, tmask = BigBirdModel.create_masks_for_block_sparse_attn(mask, 64)
    with torch.no_grad():
        out, _ = m.bigbird_block_sparse_attention(
            q, k, v, band, fmask, tmask, blocked, blocked, heads, 3, 64, 64, 64, 1, length, length,
            seed=seed, plan_from_length=None, plan_num_rand_blocks=None)
    return out.reshape(length, heads * 64).numpy()      # token-major [L, H*d]


def main():
    plans = []
    for length, seed, heads in [(768, 0, 2), (832, 0, 12), (832, 5, 3), (1088, 0, 2), (2112, 1, 2),
                                (4032, 5, 2), (960, 11, 4), (704 + 64, 3, 1)]:
        plans.append({"kind": "with_head", "length": length, "seed": seed, "heads": heads, "max_pos": 4096,
                      "rand_attn": hf_plan(length, seed, heads, 4096, False).tolist()})
    for length, seed, heads, max_pos in [(1024, 0, 12, 4096), (4096, 0, 3, 4096), (2048, 7, 2, 4096),
                                         (3072, 2, 2, 4096), (4096, 3, 2, 16384), (8192, 1, 1, 16384)]:
        plans.append({"kind": "max_plan", "length": length, "seed": seed, "heads": heads, "max_pos": max_pos,
                      "rand_attn": hf_plan(length, seed, heads, max_pos, True).tolist()})
    with open(os.path.join(HERE, "hf_plans.json"), "w") as f:
        json.dump(plans, f, separators=(",", ":"))

    cases = {}
    for name, length, heads, seed, in_seed in [("L1024_H2_seed0", 1024, 2, 0, 100),
                                               ("L832_H2_seed3", 832, 2, 3, 101)]:
        cases[name + "_out"] = hf_attention(length, heads, seed, in_seed)
        cases[name + "_meta"] = np.array([length, heads, seed, in_seed], dtype=np.int64)
    # a padded tail: 832 positions of which 800 / 769 are tokens (HuggingFace zeroes the padded query rows)
    for name, length, heads, seed, in_seed, tokens in [("L832_H2_seed3_len800", 832, 2, 3, 101, 800),
                                                       ("L1024_H2_seed0_len961", 1024, 2, 0, 100, 961)]:
        cases[name + "_out"] = hf_attention(length, heads, seed, in_seed, tokens)
        cases[name + "_meta"] = np.array([length, heads, seed, in_seed, tokens], dtype=np.int64)
    np.savez(os.path.join(HERE, "hf_attention.npz"), **cases)
    print("plans:", len(plans), "attention cases:", [k for k in cases if k.endswith("_out")])


if __name__ == "__main__":
    main()
