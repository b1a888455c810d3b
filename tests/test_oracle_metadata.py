"""The oracle's CSR and LPT plan against the reference's golden vectors and invariants."""
import json
import os

import numpy as np
import pytest

from oracle import metadata as md


@pytest.fixture(scope="module")
def fx(golden_dir):
    with open(os.path.join(golden_dir, "layers_test_n64_h12_cta160.json")) as f:
        return json.load(f)


def test_lpt_plan_is_bit_exact(fx):
    sb, total, pos, ids = md.data_metainfo([4096], 64, 160, 12)
    assert sb == [0, 64] and total == 622
    assert pos.tolist() == fx["from_select_index_position"]
    assert ids.tolist() == fx["from_select_index"]


def test_golden_csr_structure(fx):
    pos, idx = fx["to_select_index_position"], fx["to_select_index"]
    n = 64
    assert pos == np.concatenate([[0], np.cumsum(md.block_costs([0, n]))]).tolist()
    assert pos[-1] == 10 * n - 18 == len(idx)
    for i in range(n):
        row = idx[pos[i]:pos[i + 1]]
        want = md.row_blocks(i, n, row[-3:])
        assert row == want, i
        if 0 < i < n - 1:
            cand = md.reference_random_candidates(i, n)
            assert len(set(row[-3:])) == 3 and all(b in cand for b in row[-3:]), i


def test_reference_generator_structure():
    rng = np.random.RandomState(0)
    sb = md.seq_prefix_blocks([768, 4096, 1280])
    idx, pos = md.reference_to_index(sb, rng)
    assert len(pos) == sb[-1] + 1
    assert pos[-1] == sum(10 * (sb[s + 1] - sb[s]) - 18 for s in range(3))
    g = 0
    for s in range(3):
        n = sb[s + 1] - sb[s]
        for i in range(n):
            row = idx[pos[g]:pos[g + 1]].tolist()
            assert max(row) < n and min(row) >= 0
            if 0 < i < n - 1:
                assert len(row) == (7 if i in (1, n - 2) else 8)
                assert len(set(row)) == len(row)          # this generator never repeats a block
            g += 1


def test_short_sequences_are_full_attention():
    sb = md.seq_prefix_blocks([512, 704])
    idx, pos = md.hf_to_index([512, 704], 0, 2)
    assert pos[-1] == 2 * (8 * 8 + 11 * 11)
    assert idx[:8].tolist() == list(range(8))
    assert md.block_costs(sb) == [8] * 8 + [11] * 11


def test_hf_csr_matches_key_multiset():
    from oracle import plans
    lens = [1024, 832]
    idx, pos = md.hf_to_index(lens, 3, 2)
    sb = md.seq_prefix_blocks(lens)
    nb = sb[-1]
    for s, length in enumerate(lens):
        n = length // 64
        ra = plans.rand_attn_for_length(length, 3, 2)
        for h in range(2):
            for i in range(n):
                row = sorted(idx[pos[h * nb + sb[s] + i]: pos[h * nb + sb[s] + i + 1]].tolist())
                if i in (0, n - 1):
                    want = list(range(n))
                elif i == 1:
                    want = [0, 1, 2, n - 1] + ra[h, 0].tolist()
                elif i == n - 2:
                    want = [0, n - 3, n - 2, n - 1] + ra[h, n - 3].tolist()
                else:
                    want = [0, i - 1, i, i + 1, n - 1] + ra[h, i - 1].tolist()
                assert row == sorted(want)


def test_lpt_invariants_and_tiny_textbook_case():
    lens = [768, 2048, 1024, 4096]
    sb, total, pos, ids = md.data_metainfo(lens, 64, 37, 5)
    assert sorted(ids.tolist()) == list(range(sb[-1] * 5))          # every unit exactly once
    costs = md.block_costs(sb)
    load = []
    for c in range(37):
        tot = 0
        for u in ids[pos[c]:pos[c + 1]]:
            s, h, b = md.decode_unit(int(u), sb, 5)
            tot += costs[sb[s] + b]
        load.append(tot)
    assert max(load) - min(load) <= max(costs)
    # textbook LPT by hand: jobs 3,5,3,4,3 on 2 machines
    pos2, ids2 = md.lpt_partition([3, 5, 3, 4, 3], [0, 5], 2, 1)
    # order 5(b1),4(b3),3(b0),3(b2),3(b4): m0:5, m1:4, m1:+3=7, m0:+3=8, m1:+3=10
    assert ids2[pos2[0]:pos2[1]].tolist() == [1, 2] and ids2[pos2[1]:pos2[2]].tolist() == [3, 0, 4]


def test_bad_lengths_rejected():
    with pytest.raises(ValueError):
        md.seq_prefix_blocks([100])
    with pytest.raises(ValueError):
        md.seq_prefix_blocks([0])
