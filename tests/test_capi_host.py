"""CPU-side tests of the C-ABI library: it loads, exports every declared symbol, and its
host metadata (RNG, plans, CSR, LPT) is bit-exact against numpy, the oracle and the
golden vectors.  No GPU compute is called here."""
import ctypes
import json
import os
import re
import threading
import time

import numpy as np
import pytest

import __graft_entry__ as graft
from oracle import metadata as md
from oracle import plans


@pytest.fixture(scope="module")
def capi():
    return graft.load_package().capi


def test_library_exports_every_declared_symbol(capi):
    header = open(os.path.join(graft.ROOT, "include", "raptor_t_hip.h")).read()
    declared = sorted(set(re.findall(r"\b(rt_[a-z0-9_]+)\s*\(", header)))
    assert declared == sorted(capi.EXPORTS)
    L = capi.lib()
    for name in declared:
        assert hasattr(L, name), name
    assert L.rt_abi_version() == 1


def test_rng_matches_numpy(capi):
    for seed in [0, 1, 5, 11, 12345, 2 ** 31 + 7]:
        sizes = [13, 3, 60, 12, 1, 2, 57, 0, 100, 1000]
        np.random.seed(seed)
        want = np.concatenate([np.random.permutation(n) for n in sizes])
        assert np.array_equal(capi.np_permutations(seed, sizes), want), seed


def test_plans_match_hf_goldens(capi, golden_dir):
    for p in json.load(open(os.path.join(golden_dir, "hf_plans.json"))):
        if p["kind"] == "with_head" and p["length"] % 256 == 0:
            continue        # 768 tokens: the patched reference would use the other generator
        got = capi.rand_attn(p["length"], p["seed"], p["heads"], p["max_pos"])
        assert np.array_equal(got, np.array(p["rand_attn"], dtype=np.int32)), (p["kind"], p["length"])


def test_plans_match_oracle_over_many_lengths(capi):
    for length in list(range(768, 4097, 192)) + [8192, 16384 - 64]:
        for seed in (0, 7):
            max_pos = 4096 if length <= 4096 else 16384
            want = plans.rand_attn_for_length(length, seed, 3, max_pos)
            assert np.array_equal(capi.rand_attn(length, seed, 3, max_pos), want), (length, seed)
    want = plans.rand_attn_for_length(2048, 1, 2, policy=plans.POLICY_HF_UPSTREAM)
    assert np.array_equal(capi.rand_attn(2048, 1, 2, policy=capi.RT_POLICY_HF_UPSTREAM), want)


def test_lpt_plan_bit_exact_vs_golden_and_oracle(capi, golden_dir):
    fx = json.load(open(os.path.join(golden_dir, "layers_test_n64_h12_cta160.json")))
    pos, ids = capi.partition_lpt([0, 64], 12, 160)
    assert pos.tolist() == fx["from_select_index_position"] and ids.tolist() == fx["from_select_index"]
    rng = np.random.default_rng(0)
    for _ in range(5):
        lens = (64 * rng.integers(1, 65, size=int(rng.integers(1, 17)))).tolist()
        heads, n_wg = int(rng.integers(1, 17)), int(rng.integers(1, 700))
        sb, total, opos, oids = md.data_metainfo(lens, 64, n_wg, heads)
        pos, ids = capi.partition_lpt(sb, heads, n_wg)
        assert np.array_equal(pos, opos) and np.array_equal(ids, oids)
        costs, tot = capi.block_costs(sb)
        assert costs.tolist() == md.block_costs(sb) and tot == total


def test_csr_bit_exact_vs_oracle_and_golden_structure(capi, golden_dir):
    fx = json.load(open(os.path.join(golden_dir, "layers_test_n64_h12_cta160.json")))
    lens = [768, 4096, 1024, 512, 832, 64]
    sb = capi.seq_prefix_blocks(lens)
    assert sb.tolist() == md.seq_prefix_blocks(lens)
    for seed in (0, 3, 11):
        idx, pos = capi.build_to_index(sb, 12, seed=seed)
        oi, op = md.hf_to_index(lens, seed, 12)
        assert np.array_equal(idx, oi) and np.array_equal(pos, op)
    # head-shared reference plan: same positions as the golden CSR for n = 64, legal rows
    idx, pos = capi.build_to_index([0, 64], 1, mode=capi.RT_PLAN_REFERENCE, seed=9)
    assert pos.tolist() == fx["to_select_index_position"]
    for i in range(64):
        row = idx[pos[i]:pos[i + 1]].tolist()
        assert row == md.row_blocks(i, 64, row[-3:])
        if 0 < i < 63:
            cand = md.reference_random_candidates(i, 64)
            assert len(set(row[-3:])) == 3 and all(b in cand for b in row[-3:])
    # explicit plan == the golden CSR itself
    gi, gp = fx["to_select_index"], fx["to_select_index_position"]
    ra = np.array([gi[gp[i + 1] - 3: gp[i + 1]] for i in range(1, 63)], dtype=np.int32)
    idx, pos = capi.build_to_index([0, 64], 1, mode=capi.RT_PLAN_EXPLICIT, rand_attn=ra)
    assert idx.tolist() == gi and pos.tolist() == gp


def test_error_paths_return_codes_not_exits(capi):
    with pytest.raises(capi.RaptorError) as e:
        capi.seq_prefix_blocks([100])
    assert e.value.code == capi.RT_EINVAL and "multiple of 64" in str(e.value)
    with pytest.raises(capi.RaptorError):
        capi.seq_prefix_blocks([])
    with pytest.raises(capi.RaptorError):
        capi.build_to_index([0, 5, 5], 1)
    with pytest.raises(capi.RaptorError):
        capi.build_to_index([0, 64], 2, mode=capi.RT_PLAN_REFERENCE)
    with pytest.raises(capi.RaptorError):
        capi.rand_attn(512, 0, 2)
    with pytest.raises(capi.RaptorError):
        capi.build_to_index([0, 64], 1, mode=capi.RT_PLAN_EXPLICIT, rand_attn=np.full((62, 3), 64))
    sb = np.array([0, 64], dtype=np.int32)
    idx = np.empty(10, dtype=np.int32)
    pos = np.empty(65, dtype=np.int32)
    rc = capi.lib().rt_meta_build_to_index(sb.ctypes.data_as(ctypes.POINTER(ctypes.c_int)), 1, 1, 0, 0, 4096, 0, None,
                                           idx.ctypes.data_as(ctypes.POINTER(ctypes.c_int)), 10,
                                           pos.ctypes.data_as(ctypes.POINTER(ctypes.c_int)), 65)
    assert rc == capi.RT_ENOMEM
    # kernels validate their arguments on the host before any launch
    assert capi.lib().rt_bias_gelu(None, None, 1, 8, 0, None) == capi.RT_EINVAL
    assert capi.lib().rt_bias_residual_layernorm(ctypes.c_void_p(16), ctypes.c_void_p(16), ctypes.c_void_p(16),
                                                 ctypes.c_void_p(16), ctypes.c_void_p(16), 4, 7, 1e-5, 0, None) == capi.RT_EINVAL


def test_launch_event_pair_is_per_thread_and_withdrawable(capi):
    """rt_time_next_launch only stores the pair (no GPU call): a second call reports the pair that no launch took,
    and another thread neither sees nor disturbs it."""
    import threading
    assert capi.time_next_launch(None, None) == 0
    assert capi.time_next_launch(ctypes.c_void_p(8), ctypes.c_void_p(16)) == 0
    seen = []
    th = threading.Thread(target=lambda: seen.append(capi.time_next_launch(None, None)))
    th.start()
    th.join()
    assert seen == [0]
    assert capi.time_next_launch(None, None) == 1          # still there: withdrawn now
    assert capi.time_next_launch(None, None) == 0


def test_plan_memo_table_returns_what_a_fresh_draw_returns(capi):
    """The memo table of plans changes nothing but the time: every index built with it equals the index built with
    the table off, for both plan families, several seeds and position counts; look-ups are counted; a bound of zero
    forgets everything."""
    lens = [832, 1024, 64, 2048, 1088, 4096, 1024]
    sb = capi.seq_prefix_blocks(lens)
    try:
        capi.plan_cache(0)
        fresh = {(seed, mp): capi.build_to_index(sb, 3, seed=seed, max_pos=mp) for seed in (0, 5) for mp in (4096, 8192)}
        capi.plan_cache(1 << 20)
        h0, m0 = capi.plan_cache()
        for rnd in range(2):
            for (seed, mp), (idx, pos) in fresh.items():
                got_idx, got_pos = capi.build_to_index(sb, 3, seed=seed, max_pos=mp)
                assert np.array_equal(got_idx, idx) and np.array_equal(got_pos, pos)
        h1, m1 = capi.plan_cache()
        sparse = sum(1 for n in lens if n >= 768)
        assert m1 - m0 == 4 * (sparse - 1)                   # the two 1024-token sequences share a plan
        assert h1 - h0 == 4 * (sparse + 1)
        assert np.array_equal(capi.rand_attn(1088, 5, 3), capi.rand_attn(1088, 5, 3))
        capi.plan_cache(0)                                    # forget, then a tiny bound: nothing fits, results unchanged
        capi.plan_cache(16)
        idx, pos = capi.build_to_index(sb, 3, seed=0, max_pos=4096)
        assert np.array_equal(idx, fresh[(0, 4096)][0])
    finally:
        capi.plan_cache(64 << 20)


def _host_csr(ptr, n):
    return np.ctypeslib.as_array(ctypes.cast(ptr, ctypes.POINTER(ctypes.c_int)), shape=(n,)).copy()


@pytest.mark.parametrize("async_", [True, False])
def test_pipeline_host_mode_builds_every_layer(capi, async_):
    heads, layers = 4, 6
    pipe = capi.Pipeline(layers, heads, async_=async_, device=-1)
    pipe.set_index_check(True)                    # every CSR the pipeline builds passes rt_meta_check_to_index
    try:
        for lens in ([768, 1024], [4096], [64, 832, 2048, 128]):
            sb = capi.seq_prefix_blocks(lens)
            pipe.publish(sb)
            for layer in reversed(range(layers)):
                ip, pp, ph, wait = pipe.acquire(layer)
                assert ph == heads and wait >= 0
                n_idx, n_pos = capi.to_index_size(sb, ph)
                want_idx, want_pos = capi.build_to_index(sb, ph, seed=layer)
                assert np.array_equal(_host_csr(ip, n_idx), want_idx)
                assert np.array_equal(_host_csr(pp, n_pos), want_pos)
                pipe.release(layer)
    finally:
        pipe.close()


def test_pipeline_ordering_and_termination(capi):
    pipe = capi.Pipeline(3, 2, device=-1)
    with pytest.raises(capi.RaptorError):          # nothing published yet
        pipe.acquire(0)
    with pytest.raises(capi.RaptorError):
        pipe.acquire(7)
    with pytest.raises(capi.RaptorError):
        pipe.publish([0, 0])
    # two publishes back to back: acquire sees the latest batch
    pipe.publish([0, 12])
    pipe.publish([0, 20])
    ip, pp, ph, _ = pipe.acquire(1)
    assert _host_csr(pp, 2 * 20 + 1)[-1] == 2 * (10 * 20 - 18)
    # a waiter blocked in acquire is released by a publish from another thread
    pipe2 = capi.Pipeline(2, 2, device=-1)
    pipe2.publish([0, 16])
    pipe2.acquire(0)
    got = {}

    def late_publish():
        time.sleep(0.05)
        pipe2.publish([0, 32])
    th = threading.Thread(target=late_publish)
    th.start()
    th.join()
    ip, pp, ph, _ = pipe2.acquire(1)
    assert _host_csr(pp, 2 * 32 + 1)[-1] == 2 * (10 * 32 - 18)
    pipe2.close()
    pipe.close()            # terminate with idle workers: must join, not hang
    pipe.close()            # idempotent


def test_pipeline_is_race_free_under_thread_sanitizer():
    """Builds the host pipeline with -fsanitize=thread and runs the stress driver
    (tests/host/pipeline_stress.cpp): publish / acquire / release orders, double signals,
    destruction right after a publish.  Any data race makes the run fail."""
    import subprocess
    csrc = os.path.join(graft.ROOT, "raptor-t_amd", "csrc")
    subprocess.check_call(["make", "-C", csrc, "tsan_test"], stdout=subprocess.DEVNULL, stderr=subprocess.STDOUT)
    exe = os.path.join(graft.ROOT, "raptor-t_amd", "build", "pipeline_stress_tsan")
    env = dict(os.environ, TSAN_OPTIONS="halt_on_error=1 exitcode=66")
    res = subprocess.run([exe], capture_output=True, text=True, timeout=300, env=env)
    assert res.returncode == 0, res.stdout[-2000:] + res.stderr[-4000:]
    assert "pipeline_stress OK" in res.stdout and "ThreadSanitizer" not in res.stderr


def test_host_metadata_under_address_and_ub_sanitizers():
    """meta.cpp built with AddressSanitizer + UndefinedBehaviorSanitizer and driven over random batch
    geometries with exact-size heap buffers, short capacities and malformed arguments: an out-of-bounds
    write, a signed overflow or an accepted bad argument makes the run fail."""
    import subprocess
    csrc = os.path.join(graft.ROOT, "raptor-t_amd", "csrc")
    subprocess.check_call(["make", "-C", csrc, "asan_test"], stdout=subprocess.DEVNULL, stderr=subprocess.STDOUT)
    exe = os.path.join(graft.ROOT, "raptor-t_amd", "build", "meta_fuzz_asan")
    # the harness preloads a library of its own: AddressSanitizer only checks that its runtime comes first
    env = dict(os.environ, ASAN_OPTIONS="verify_asan_link_order=0:detect_leaks=1:exitcode=67",
               UBSAN_OPTIONS="halt_on_error=1:print_stacktrace=1")
    res = subprocess.run([exe], capture_output=True, text=True, timeout=300, env=env)
    assert res.returncode == 0, res.stdout[-2000:] + res.stderr[-4000:]
    assert "meta_fuzz OK" in res.stdout and "Sanitizer" not in res.stderr


def test_padded_batch_adapters_round_trip():
    """pack_padded_batch keeps each sequence's tokens plus the padding that fills its last block, and
    unpack_to_padded puts rows back where they came from."""
    import importlib
    import torch
    graft.load_package()
    ut = importlib.import_module("raptor_t_amd.util")
    lens = [130, 64, 1]
    width = 150                                           # not a multiple of 64: rows are widened as needed
    ids = torch.arange(3 * width).view(3, width) + 1
    mask = (torch.arange(width)[None, :] < torch.tensor(lens)[:, None]).long()
    p = ut.pack_padded_batch(ids, mask)
    assert p["seq_lens"] == [192, 64, 64] and p["seq_tokens"] == lens
    assert p["input_ids"].dtype == torch.int32 and p["input_ids"].numel() == 320
    assert p["position_ids"][:192].tolist() == list(range(192)) and p["position_ids"][192] == 0
    assert p["input_ids"][:130].tolist() == ids[0, :130].tolist()
    assert p["input_ids"][192:256].tolist() == ids[1, :64].tolist()
    assert p["seq_tokens_tensor"].tolist() == lens
    hidden = torch.arange(320 * 2, dtype=torch.float32).view(320, 2)
    back = ut.unpack_to_padded(hidden, p["seq_lens"], p["seq_tokens"], width)
    assert back.shape == (3, width, 2)
    assert torch.equal(back[0, :130], hidden[:130]) and torch.equal(back[2, 0], hidden[256])
    assert back[0, 130:].abs().sum() == 0 and back[2, 1:].abs().sum() == 0
    # every sequence kept at the batch's width (rounded up to a block): whole blocks of padding stay
    w = ut.pack_padded_batch(ids, mask, keep_width=True)
    assert w["seq_lens"] == [192, 192, 192] and w["seq_tokens"] == lens and w["input_ids"].numel() == 576
    assert w["input_ids"][192:192 + 150].tolist() == ids[1].tolist() and w["input_ids"][192 + 150:384].abs().sum() == 0
    assert w["position_ids"][384:576].tolist() == list(range(192))
    back = ut.unpack_to_padded(torch.arange(576 * 2, dtype=torch.float32).view(576, 2), w["seq_lens"], w["seq_tokens"], width)
    assert back.shape == (3, width, 2) and back[1, 64:].abs().sum() == 0 and back[1, 63, 0] == 2 * (192 + 63)
    with pytest.raises(ValueError):
        ut.pack_padded_batch(ids, torch.tensor([[1, 0, 1]]).expand(3, 3)[:, :3].repeat(1, 50))   # holes in the mask
    with pytest.raises(ValueError):
        ut.pack_padded_batch(ids, torch.zeros_like(mask))
