"""Host-side checks of bench.py that need no GPU: the one-GPU rule, the pair count behind the attention FLOPs
and the roofline helpers."""
import importlib.util
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench():
    spec = importlib.util.spec_from_file_location("rt_bench", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0
    assert "one gpu" in (r.stdout + r.stderr).lower()


def test_block_pairs_follow_the_bigbird_row_rules():
    """10n - 18 key blocks per (sequence, head) for a sparse sequence (two dense rows of n, two rows of 7, the
    others 8), n*n below twelve blocks: the figure the attention FLOPs are derived from."""
    b = _bench()
    for n in (12, 13, 64):
        rows = [n, 7] + [8] * (n - 4) + [7, n]
        assert sum(rows) == 10 * n - 18
        assert b.block_pairs([0, n], 3) == 3 * (10 * n - 18)
    assert b.block_pairs([0, 5, 16], 2) == 2 * (25 + 11 * 11)
    assert b.block_pairs([0, 64] + [64 * i for i in range(2, 9)], 12) == 59712        # config 2
    assert b.PAIR_FLOP == 4 * 64 * 64 * 64


def test_hbm_roofline_arithmetic():
    b = _bench()
    r = b.hbm_roofline("k", 8_000_000, 2.0, traffic=9e6)
    assert r["bound"] == "hbm" and r["unit"] == "GB/s" and r["peak"] == 8000.0
    assert abs(r["achieved"] - 4000.0) < 1e-9 and abs(r["frac"] - 0.5) < 1e-12
    assert r["traffic"] == 9e6 and r["bytes_per_launch"] == 8_000_000
    json.dumps(r)


def test_cpu_baseline_helpers():
    """The thread count of the CPU baselines never exceeds what the job may use, and the bounded timer stops at its
    budget but not before three runs."""
    b = _bench()
    n = b.host_cores()
    assert 1 <= n <= (os.cpu_count() or 1)
    old = os.environ.get("OMP_NUM_THREADS")
    os.environ["OMP_NUM_THREADS"] = "1"
    try:
        assert b.host_cores() == 1
    finally:
        if old is None:
            del os.environ["OMP_NUM_THREADS"]
        else:
            os.environ["OMP_NUM_THREADS"] = old
    calls = []
    med, runs = b.timed_median(lambda: calls.append(1), warmup=2, reps=50, budget_s=0.0)
    assert runs == 3 and len(calls) == 5 and med >= 0.0
    med, runs = b.timed_median(lambda: None, warmup=0, reps=4, budget_s=60.0)
    assert runs == 4


def test_traffic_figures_come_from_the_committed_profile():
    """bench.py's `traffic` fields are read from the table of profiles/memory_kernels_c3_traffic.txt: every
    hand-written kernel of the default line has a row, the memory-bound ones at their algorithmic bytes."""
    b = _bench()
    t = b.measured_traffic_c3()
    assert set(t) >= {"bs_attention_kernel", "bias_residual_layernorm_kernel", "bias_gelu_kernel", "qkv_bias_split_kernel"}
    tokens, hidden, ffn = 37184, 768, 3072
    assert abs(t["bias_residual_layernorm_kernel"] / (3 * tokens * hidden * 2) - 1) < 0.01
    assert abs(t["bias_gelu_kernel"] / (2 * tokens * ffn * 2) - 1) < 0.01
    assert abs(t["qkv_bias_split_kernel"] / (2 * tokens * 2 * hidden * 2) - 1) < 0.01
    assert 4 * tokens * hidden * 2 <= t["bs_attention_kernel"] <= 3 * 4 * tokens * hidden * 2
