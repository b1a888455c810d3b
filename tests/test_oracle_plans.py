"""The oracle's random-block plans against the HuggingFace goldens and invariants."""
import json
import os

import numpy as np
import pytest

from oracle import plans


def _load(golden_dir):
    with open(os.path.join(golden_dir, "hf_plans.json")) as f:
        return json.load(f)


def test_plans_match_hf_goldens(golden_dir):
    for p in _load(golden_dir):
        np.random.seed(p["seed"])
        nb = p["length"] // 64
        if p["kind"] == "with_head":
            pfl, pnr = plans.rand_attn_plan(p["length"])
            got = np.stack(plans.rand_attn_with_head(p["length"], p["heads"], pfl, pnr))
        else:
            got = np.stack([plans.rand_attn_max_plan(p["max_pos"], last_idx=1024)[: nb - 2]
                            for _ in range(p["heads"])])
        assert np.array_equal(got, np.array(p["rand_attn"], dtype=np.int32)), (p["kind"], p["length"], p["seed"])


def test_rand_attn_for_length_selects_the_reference_generator(golden_dir):
    for p in _load(golden_dir):
        if p["max_pos"] != 4096:
            continue
        got = plans.rand_attn_for_length(p["length"], p["seed"], p["heads"], 4096)
        if p["kind"] == "max_plan" or p["length"] % 256 != 0:
            assert np.array_equal(got, np.array(p["rand_attn"], dtype=np.int32)), (p["length"], p["seed"])


def test_policy_switch():
    assert plans.uses_max_plan(2048) and not plans.uses_max_plan(2048, plans.POLICY_HF_UPSTREAM)
    assert plans.uses_max_plan(4096, plans.POLICY_HF_UPSTREAM)
    assert not plans.uses_max_plan(768) and not plans.uses_max_plan(832)


def test_rand_attn_plan_table():
    assert plans.rand_attn_plan(4032) == ([704, 4032], [3, 0])
    assert plans.rand_attn_plan(640) == ([512, 640], [1, 2])
    assert plans.rand_attn_plan(512) == ([512], [3])


@pytest.mark.parametrize("length", [768, 832, 1984, 4032])
def test_with_head_plan_is_legal(length):
    n = length // 64
    ra = plans.rand_attn_for_length(length, 4, 3)
    assert ra.shape == (3, n - 2, 3)
    for h in range(3):
        for i in range(1, n - 1):
            row = ra[h, i - 1]
            assert len(set(row.tolist())) == 3
            for b in row:
                assert 1 <= b <= 9 and b not in (i - 1, i, i + 1)


def test_max_plan_values_and_truncation():
    np.random.seed(9)
    full = plans.rand_attn_max_plan(4096, last_idx=1024)
    assert full.shape == (62, 3) and full.min() >= 1 and full.max() <= 15
    for i in range(1, 63):
        assert len(set(full[i - 1].tolist())) == 3
        if 3 <= i <= 13:
            assert not set(full[i - 1].tolist()) & {i - 1, i, i + 1}
