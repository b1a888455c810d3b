"""Benchmark of the block-sparse encoder hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c3|c1|c2|c4|c5|ref_e2e|stream|overlap|mfma_mix]

Default workload `c3` is the headline configuration (benchmark config 3): the 12-layer BigBird-base fp16 encoder
on a padding-free batch of 16 sequences with lengths uniform in [512, 4096] (multiples of
64, numpy default_rng(0)), random-init N(0, 0.02) weights, N(0, 1) inputs, driven through
the drop-in layer API (`raptor_t` pybind module) with the asynchronous metadata pipeline.
One step = MetaData.update_meta_data + one 12-layer forward; inputs are resident in HBM.
Prints ONE JSON line: seqs/s (value), ms/step, ms/layer, the roofline of the dominant
hand-written kernel (block-sparse attention, MFMA bound) measured live with HIP events
inside the timed steps, HBM rooflines of the LayerNorm / GELU / split kernels, and the
CPU baseline (the oracle layer timed on the host cores on a bounded sample).
"""
import argparse
import importlib
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
import __graft_entry__ as graft  # noqa: E402

MFMA_PEAK = {"f16": 2.5e15, "bf16": 2.5e15, "f32": 157.3e12}       # MI355X dense matrix peak, FLOP/s
HBM_PEAK = 8.0e12                                   # B/s
PAIR_FLOP = 4 * 64 * 64 * 64                        # QK^T + PV of one (from-block, to-block) pair, d = 64
METRIC = "seqs/sec + ms/layer, BigBird-base fp16 var-len<=4096; attn MFMA %, LN HBM GB/s"


def block_pairs(seq_blocks, heads):
    tot = 0
    for s in range(len(seq_blocks) - 1):
        n = seq_blocks[s + 1] - seq_blocks[s]
        tot += n * n if n < 12 else 10 * n - 18
    return tot * heads


TRAFFIC_PROFILE = os.path.join("profiles", "memory_kernels_c3_traffic.txt")


def measured_traffic_c3():
    """HBM-side bytes per launch of the hand-written kernels at the default workload, read from the `total MB` column
    of the table in profiles/memory_kernels_c3_traffic.txt (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs, scaled by
    what the same counters read for the K/V split kernel, a copy of known size; the commands are in that file).
    Only valid for that workload and the kernels the profile was taken with; {} if the file is not there."""
    keys = {"qkv_bias_split_kernel<__half,false>": "qkv_bias_split_kernel", "qkv_bias_split_kernel<__half,true>": "qkv_bias_split_kernel_q",
            "bias_gelu_kernel<__half>": "bias_gelu_kernel", "bias_residual_layernorm_kernel<...>": "bias_residual_layernorm_kernel",
            "bs_attention_kernel<_Float16,": "bs_attention_kernel"}
    out = {}
    try:
        with open(os.path.join(ROOT, TRAFFIC_PROFILE)) as f:
            for line in f:
                tok = line.split()
                for name, key in keys.items():
                    if tok and tok[0] == name:
                        nums = [t for t in tok[1:] if t.replace(".", "", 1).isdigit()]
                        if len(nums) >= 7:                      # FETCH raw, WRITE raw, read, written, total, algorithmic, ratio
                            out[key] = float(nums[4]) * 1e6
    except OSError:
        pass
    return out


def hbm_roofline(name, bytes_per_launch, us_per_launch, traffic=None):
    ach = bytes_per_launch / (us_per_launch * 1e-6)
    return {"kernel": name, "bound": "hbm", "achieved": ach / 1e9, "peak": HBM_PEAK / 1e9, "unit": "GB/s",
            "frac": ach / HBM_PEAK, "traffic": traffic, "bytes_per_launch": bytes_per_launch,
            "us_per_launch": us_per_launch}


def host_cores():
    """Threads the CPU baselines run on: every core this job may use.  That is the scheduler affinity of the
    process, further limited by OMP_NUM_THREADS when the host sets it (a GPU box shares its cores between the
    jobs of its GPUs and exports its share there); os.cpu_count() is printed beside it."""
    n = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    env = os.environ.get("OMP_NUM_THREADS", "")
    if env.isdigit() and int(env) >= 1:
        n = min(n, int(env))
    return max(n, 1)


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def timed_median(fn, warmup, reps, budget_s):
    """Median seconds of fn(); stops early, after at least three timed runs, once `budget_s` is used up."""
    for _ in range(warmup):
        fn()
    times, t_start = [], time.perf_counter()
    for _ in range(reps):
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
        if len(times) >= 3 and time.perf_counter() - t_start > budget_s:
            break
    return float(np.median(times)), len(times)


def cpu_baseline_config1():
    """Benchmark config 1 itself on the host cores: ONE BigBird-base encoder layer, batch 1, 1024 tokens, hidden
    768, 12 x 64 heads, FFN 3072, block 64, 2 global + 3 window + 3 random blocks, fp32, N(0, 0.02) weights,
    N(0, 1) input, seed 0; the oracle's layer (PyTorch CPU), on every core of the job and on one thread."""
    from oracle import layer as ol
    from oracle import metadata as md
    hidden, heads, ffn, lens = 768, 12, 3072, [1024]
    g = torch.Generator().manual_seed(0)
    w = ol.random_layer_weights(hidden, ffn, g)
    x = torch.randn(sum(lens), hidden, generator=g)
    sb = md.seq_prefix_blocks(lens)
    idx, pos = md.hf_to_index(lens, 0, heads)
    fn = lambda: ol.encoder_layer(x, w, heads, sb, idx, pos, heads)
    cores = host_cores()
    before = torch.get_num_threads()
    torch.set_num_threads(cores)
    t_all, n_all = timed_median(fn, 3, 20, 8.0)
    torch.set_num_threads(1)
    t_one, n_one = timed_median(fn, 1, 20, 8.0)
    torch.set_num_threads(before)
    return {"value": sum(lens) / t_all, "unit": "tokens/s", "cores": cores, "kind": "port",
            "ms_per_layer": t_all * 1e3,
            "sample": "benchmark config 1 itself: one BigBird-base layer, batch 1 x 1024 tokens, fp32, the oracle's layer "
                      "(torch CPU); median of %d runs on %d threads" % (n_all, cores),
            "one_thread": {"value": sum(lens) / t_one, "unit": "tokens/s", "cores": 1, "ms_per_layer": t_one * 1e3,
                           "runs": n_one},
            "host_cpu_count": os.cpu_count(), "cpu_model": cpu_model()}


def cpu_baseline_layer(seq_lens, hidden, heads, ffn, layers, sample_seqs, reps=3):
    """Oracle encoder layer (PyTorch-CPU fp32, the reference oracle's algorithm) on the first
    `sample_seqs` sequences of the batch, scaled by tokens to the whole batch and by the layer
    count to the whole encoder: the GPU line's own workload and unit, on every core of the job."""
    from oracle import layer as ol
    from oracle import metadata as md
    cores = host_cores()
    torch.set_num_threads(cores)
    lens = list(seq_lens[:sample_seqs])
    g = torch.Generator().manual_seed(0)
    w = ol.random_layer_weights(hidden, ffn, g)
    x = torch.randn(sum(lens), hidden, generator=g)
    sb = md.seq_prefix_blocks(lens)
    idx, pos = md.hf_to_index(lens, 0, heads, max_pos=max(4096, max(lens)))
    t_layer, n = timed_median(lambda: ol.encoder_layer(x, w, heads, sb, idx, pos, heads), 0, reps, 12.0)
    t_batch = t_layer * (sum(seq_lens) / sum(lens)) * layers
    return {"value": len(seq_lens) / t_batch, "unit": "seqs/s", "cores": cores, "kind": "port",
            "sample": "oracle encoder layer (torch CPU fp32) on the first %d sequences (%d tokens), median of %d, "
                      "scaled by tokens to the batch and x%d layers; %.2f s per sampled layer"
                      % (len(lens), sum(lens), n, layers, t_layer)}


def cpu_baseline(seq_lens, hidden, heads, ffn, layers, sample_seqs):
    """The CPU figures of one encoder line: config 1 as it stands (all cores and one thread), and under
    `this_workload` the line's own workload from a bounded sample, in the line's unit."""
    out = cpu_baseline_config1()
    out["this_workload"] = cpu_baseline_layer(seq_lens, hidden, heads, ffn, layers, sample_seqs)
    return out


def cpu_baseline_attention(steps=20):
    """CPU-side figure of the isolated-attention line: the oracle's block-sparse attention on ONE of the eight
    sequences (4096 tokens, 12 heads, fp32), in algorithmic GFLOP/s, every core of the job."""
    from oracle import attention as oa
    from oracle import metadata as md
    heads, lens = 12, [4096]
    cores = host_cores()
    torch.set_num_threads(cores)
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(lens[0], heads, 64, generator=g) for _ in range(3))
    sb = md.seq_prefix_blocks(lens)
    idx, pos = md.hf_to_index(lens, 0, heads)
    t_one, n = timed_median(lambda: oa.csr_attention(q, k, v, sb, idx, pos, heads), 1, steps, 15.0)
    flops = block_pairs(list(sb), heads) * PAIR_FLOP
    return {"value": flops / t_one / 1e9, "unit": "GFLOP/s", "cores": cores, "kind": "port", "ms": t_one * 1e3,
            "ms_scaled_to_batch_8": 8 * t_one * 1e3,
            "sample": "oracle block-sparse attention (torch CPU fp32) on one sequence of 4096 tokens, 12 heads; "
                      "median of %d" % n, "host_cpu_count": os.cpu_count(), "cpu_model": cpu_model()}


def cpu_baseline_membound(steps=20):
    """CPU-side figure of the memory-bound sweep's smallest point (8192 tokens, fp32): the oracle's
    bias + residual + LayerNorm over [8192, 768] and bias + GELU over [8192, 3072], in algorithmic GB/s."""
    from oracle import layer as ol
    cores = host_cores()
    torch.set_num_threads(cores)
    g = torch.Generator().manual_seed(0)
    t = 8192
    x, r = torch.randn(t, 768, generator=g), torch.randn(t, 768, generator=g)
    b, ga, be = (torch.randn(768, generator=g) for _ in range(3))
    t_ln, _ = timed_median(lambda: ol.bias_residual_layernorm(x, r, b, ga, be, 1e-5), 3, steps, 5.0)
    y, b2 = torch.randn(t, 3072, generator=g), torch.randn(3072, generator=g)
    t_gelu, _ = timed_median(lambda: ol.bias_gelu(y, b2), 3, steps, 5.0)
    return {"value": 3 * t * 768 * 4 / t_ln / 1e9, "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": "oracle bias + residual + LayerNorm (torch CPU fp32) over [8192, 768], 3 tensor passes of 4 bytes",
            "gelu": {"value": 2 * t * 3072 * 4 / t_gelu / 1e9, "unit": "GB/s",
                     "sample": "oracle bias + GELU over [8192, 3072], 2 tensor passes of 4 bytes"},
            "host_cpu_count": os.cpu_count(), "cpu_model": cpu_model()}


DTYPES = {"f16": torch.float16, "bf16": torch.bfloat16, "f32": torch.float32}

# The encoder workloads by name: (hidden, heads, ffn, layers, dtype, lengths(util), positions the plans are drawn for)
ENCODER_WORKLOADS = {
    "c3": (768, 12, 3072, 12, "f16", lambda ut: ut.uniform_lengths(16, 512, 4096, seed=0), 4096),
    "c5": (1024, 16, 4096, 24, "bf16", lambda ut: ut.uniform_lengths(4, 2048, 16384, seed=0), 16384),
}


def encoder_inputs(mb, hidden, ffn, layers, dt, seq_lens):
    """The synthetic inputs of an encoder workload: per layer N(0, 0.02) weights in `dt` on the GPU, then the packed
    N(0, 1) hidden states, all from one generator seeded with 0 (the parity tests of the headline workloads build
    their inputs through this function, so what they check is what is timed)."""
    g = torch.Generator().manual_seed(0)
    layers_w = [mb.random_layer_weights(hidden, ffn, g, dtype=dt) for _ in range(layers)]
    x0 = torch.randn(sum(seq_lens), hidden, generator=g).to(dt).cuda()
    return layers_w, x0


def run_encoder(args, name, hidden, heads, ffn, layers, dtype, seq_lens, max_pos=4096):
    pkg = graft.load_package()
    mb = importlib.import_module("raptor_t_amd.modeling_bert")
    ut = importlib.import_module("raptor_t_amd.util")
    dt = DTYPES[dtype]
    layers_w, x0 = encoder_inputs(mb, hidden, ffn, layers, dt, seq_lens)
    mb.cxx.MetaData.set_plan(pkg.capi.RT_PLAN_HF, pkg.capi.RT_POLICY_REFERENCE_PATCHED, max_pos)
    enc = mb.BertEncoder.from_weights(layers_w, heads, async_=not args.sync_index, eps=1e-5)
    meta = mb.cxx.MetaData()
    t = sum(seq_lens)
    block_limit = args.block_limit
    spi, spi_t, total_comp, ppi_t, pp_t = ut.generate_data_metainfo(seq_lens, 64, block_limit, heads)
    hidden_states = torch.empty_like(x0)
    new = lambda w: torch.empty(t, w, dtype=dt, device="cuda")
    inter, tmp, attn = new(ffn), new(hidden), new(hidden)

    def step():
        hidden_states.copy_(x0)
        meta.update_meta_data(t, spi[-1] + 1, total_comp, spi)
        enc(hidden_states, t, block_limit, spi, spi_t, ppi_t, pp_t, tmp, inter, attn, test_info={},
            balanced=args.lpt_plan)

    mb.cxx.set_gemm_epilogue_fusion(not args.no_epilogue_fusion)
    mb.cxx.set_attention_q_from_rows(not args.materialize_q)
    mb.cxx.set_attention_host_plan(args.lpt_plan)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    # Timed region: of the attention launches (the kernel the roofline object is about) one in five carries a pair
    # of events that take the dispatch's own start and end, rotating through the layers; a timed launch costs the
    # stream about 5 us (0.6 % of the step if every attention launch carried one).
    mb.cxx.timing_begin(["attention"], 5)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    timing = mb.cxx.timing_collect()
    # Second pass over the same steps with every launcher bracketed: the other kernels' durations.
    mb.cxx.timing_begin()
    for _ in range(args.steps):
        step()
    timing_all = mb.cxx.timing_collect()
    # The same steps with the batch cut in two micro-batches on two streams (BertEncoder.call_two_streams), against
    # the one-stream steps, in interleaved rounds: the gain depends on the box's clocks under load (1 to 7 %), so it
    # is reported beside the headline, not as the headline.
    two_streams = None
    if len(seq_lens) > 1 and not args.lpt_plan and not args.no_two_streams:
        def step2():
            hidden_states.copy_(x0)
            enc.call_two_streams(hidden_states, seq_lens, block_limit, heads, tmp, inter, attn, test_info={}, balanced=False)

        def timed(fn):
            fn()
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            for _ in range(args.steps):
                fn()
            torch.cuda.synchronize()
            return (time.perf_counter() - t1) / args.steps * 1e3
        timed(step2)                                          # the GEMM plans of the two halves' row counts
        one, two = [], []
        for _ in range(3):
            one.append(timed(step))
            two.append(timed(step2))
        assert bool(torch.isfinite(hidden_states).all()), "the two-stream output is not finite"
        one, two = float(np.median(one)), float(np.median(two))
        two_streams = {"ms_per_step": two, "value": len(seq_lens) / (two * 1e-3), "unit": "seqs/s",
                       "one_stream_ms_per_step_same_rounds": one, "gain": 1.0 - two / one,
                       "how": "BertEncoder.call_two_streams: two micro-batches, two HIP streams of equal priority"}
    meta.terminate_thread()
    # outside the timed region: a step that produced a NaN or an Inf anywhere is not a measurement
    assert bool(torch.isfinite(hidden_states).all()), "the encoder's output is not finite"

    ms_step = elapsed / args.steps * 1e3
    per = {k: v[0] / v[1] for k, v in timing_all.items() if v[1]}
    per["attention"] = timing["attention"][0] / timing["attention"][1]
    gelu_note = "launches inside the timed steps"
    if "add_bias_act_kernel" not in per:
        # bias + GELU ran in the GEMM's epilogue: the stand-alone kernel is timed on the same [T, ffn] buffer
        bias = torch.zeros(ffn, dtype=dt, device="cuda")
        per["add_bias_act_kernel"] = time_kernel(lambda: pkg.capi.bias_gelu(inter, bias), 20, 3)
        gelu_note = "stand-alone launches on the step's [tokens, ffn] buffer (the steps fuse it into the GEMM)"
    pairs = block_pairs(spi, heads)
    att_us = per["attention"]
    att_flops = pairs * PAIR_FLOP
    ach = att_flops / (att_us * 1e-6)
    sz = 4 if dtype == "f32" else 2
    traffic = measured_traffic_c3() if name.startswith("c3") else {}
    out = {
        "metric": METRIC, "value": len(seq_lens) / (elapsed / args.steps), "unit": "seqs/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_step, "ms_per_layer": ms_step / layers,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": dtype, "data": "synthetic",
        "config": {"workload": name, "layers": layers, "hidden": hidden, "heads": heads, "ffn": ffn,
                   "batch": len(seq_lens), "tokens": t, "seq_lens": seq_lens, "block_limit": block_limit,
                   "balanced": args.lpt_plan, "async_index": not args.sync_index,
                   "gemm_epilogue_fusion": not args.no_epilogue_fusion,
                   "attention_q_from_rows": not args.materialize_q,
                   "weights": "random N(0,0.02)", "plan": "per-head HF plan, seed = layer index"},
        "roofline": {"kernel": "bs_attention_kernel", "bound": "mfma", "achieved": ach / 1e12,
                     "peak": MFMA_PEAK[dtype] / 1e12, "unit": "TFLOP/s", "frac": ach / MFMA_PEAK[dtype],
                     "traffic": traffic.get("bs_attention_kernel"),
                     "traffic_source": TRAFFIC_PROFILE if traffic.get("bs_attention_kernel") else None, "flop_per_launch": att_flops,
                     "block_pairs": pairs, "us_per_launch": att_us, "algorithmic_hbm_bytes": 4 * t * hidden * sz},
        "roofline_layernorm": hbm_roofline("bias_residual_layernorm_kernel", 3 * t * hidden * sz,
                                           per["add_bias_and_layernorm_kernel"],
                                           traffic.get("bias_residual_layernorm_kernel")),
        "roofline_gelu": dict(hbm_roofline("bias_gelu_kernel", 2 * t * ffn * sz, per["add_bias_act_kernel"],
                                           traffic.get("bias_gelu_kernel")), measured=gelu_note),
        # K and V only (read + write) unless Q is materialised too
        "roofline_qkv_split": hbm_roofline("qkv_bias_split_kernel", 2 * t * (3 if args.materialize_q else 2) * hidden * sz,
                                           per["add_bias_and_transpose_kernel"],
                                           traffic.get("qkv_bias_split_kernel_q" if args.materialize_q
                                                       else "qkv_bias_split_kernel")),
        "two_streams": two_streams,
        "kernel_us_per_launch": per,
        "kernel_us_per_step": {k: v[0] / args.steps for k, v in timing_all.items()},
        "kernel_timing": "HIP events holding each dispatch's own start and end (hipExtLaunchKernelGGL; the vendor GEMMs: "
                         "events recorded around the call).  attention: one launch in five inside the timed steps; "
                         "the others: a second pass over the same steps with every launcher timed",
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(seq_lens, hidden, heads, ffn, layers, args.cpu_sample_seqs)
    return out


def time_kernel(fn, steps, warmup, settle_ms=25.0):
    """Median GPU duration of one launch in microseconds; `fn` launches exactly one kernel of the library.  The
    duration is the dispatch's own (capi.time_next_launch: the start and end the GPU stamps on the kernel, what
    rocprofv3 reports), on the stream `fn` launches on; a pair of recorded events around a launch would add the
    gaps to its neighbours, 2-5 us here.  After the warm-up launches the kernel keeps running for `settle_ms`:
    from idle the GPU takes some tens of launches to reach its sustained clocks (the first launches of a 100 us
    kernel measure 10-15 % slow), and a kernel inside a running job never sees that ramp.  The timed launches are
    queued behind a spin kernel that keeps the GPU busy while the host enqueues all of them, so that they run back
    to back as in a job (a launch through Python costs the host about 10 us, more than a small kernel runs)."""
    pkg = graft.load_package()
    cxx = importlib.import_module("raptor_t_amd.modeling_bert").cxx
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < settle_ms:
        for _ in range(10):
            fn()
        torch.cuda.synchronize()
    t0 = time.perf_counter()
    fn()
    host_us = (time.perf_counter() - t0) * 1e6                 # what one enqueue costs the host
    torch.cuda.synchronize()
    evs = [cxx.event_pair_create() for _ in range(steps)]
    torch.cuda._sleep(int(2.4e3 * (3.0 * host_us + 20.0) * steps))   # cycles: three times the host's enqueue time
    for a, b in evs:
        pkg.capi.time_next_launch(a, b)
        fn()
    torch.cuda.synchronize()
    return float(np.median([cxx.event_pair_elapsed_us(a, b) for a, b in evs]))


def run_attention_only(args):
    """Benchmark config 2: isolated block-sparse attention, batch 8 x 4096 tokens, 12 heads, fp16."""
    capi = graft.load_package().capi
    heads, lens = 12, [4096] * 8
    t = sum(lens)
    sb = capi.seq_prefix_blocks(lens)
    idx, pos = capi.build_to_index(sb, heads, seed=0)
    dev = lambda a: torch.from_numpy(a).cuda()
    sb_d, idx_d, pos_d = dev(sb), dev(idx), dev(pos)
    g = torch.Generator(device="cuda").manual_seed(0)
    qkv = torch.randn(t, 3 * heads * 64, generator=g, device="cuda", dtype=torch.float16)
    bias = torch.zeros(3 * heads * 64, device="cuda", dtype=torch.float16)
    q, k, vt = (torch.empty(t * heads * 64, device="cuda", dtype=torch.float16) for _ in range(3))
    capi.qkv_bias_split(qkv, bias, q, k, vt, sb_d, heads, capi.Q_SCALE)
    out = torch.empty(t, heads * 64, device="cuda", dtype=torch.float16)
    fp, fi = capi.partition_lpt(sb, heads, args.block_limit)
    fp_d, fi_d = dev(fp), dev(fi)
    if args.lpt_plan:
        fn = lambda: capi.bs_attention_fwd(q, k, vt, out, sb_d, heads, idx_d, pos_d, heads, fi_d, fp_d)
    else:
        fn = lambda: capi.bs_attention_fwd(q, k, vt, out, sb_d, heads, idx_d, pos_d, heads)
    us = time_kernel(fn, args.steps, args.warmup)
    assert bool(torch.isfinite(out).all()), "the attention output is not finite"
    # the same batch with every sequence 17 tokens short of its last block (a padded serving batch): the kernel's second
    # instantiation, whose pipelined loop takes each row's padded tile last and masks its padded keys there
    tok_d = torch.tensor([n - 17 for n in lens], dtype=torch.int32).cuda()
    masked_us = time_kernel(lambda: capi.bs_attention_fwd(q, k, vt, out, sb_d, heads, idx_d, pos_d, heads, None, None, tok_d),
                            args.steps, args.warmup)
    pairs = block_pairs(sb.tolist(), heads)
    ach = pairs * PAIR_FLOP / (us * 1e-6)
    res = {"metric": "isolated block-sparse attention, batch 8 x 4096, 12 heads x 64, fp16", "value": ach / 1e12,
            "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": us / 1e3,
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
            "config": {"workload": "c2 isolated attention", "block_pairs": pairs, "block_limit": args.block_limit,
                       "balanced": args.lpt_plan},
            "roofline": {"kernel": "bs_attention_kernel", "bound": "mfma", "achieved": ach / 1e12, "peak": 2500.0,
                         "unit": "TFLOP/s", "frac": ach / 2.5e15, "traffic": None},
            "padded_batch": {"us_per_launch": masked_us, "frac": pairs * PAIR_FLOP / (masked_us * 1e-6) / 2.5e15,
                             "how": "every sequence 17 tokens short of its last block (rt_bs_attention_fwd_masked): "
                                    "the pipelined loop runs each row's padded tile last and masks its padded keys there"}}
    if not args.no_cpu_baseline:
        res["cpu_baseline"] = cpu_baseline_attention()
    return res


def run_membound_sweep(args):
    """Benchmark config 4: LayerNorm and GELU epilogues over tokens {8K, 32K, 64K}, fp16 and bf16.
    Every kernel is timed twice: `frac` with its launches rotating over enough separate buffers that no launch finds
    its operands where an earlier one left them (the rotation covers more than 600 MB; the memory-side cache holds
    256 MB), and `frac_resident` with every launch on the same buffers, as a loop over one tensor runs it."""
    capi = graft.load_package().capi
    rows = []

    def rotating(make, call, set_bytes):
        sets = [make() for _ in range(max(2, -(-600_000_000 // set_bytes) + 1))]
        state = [0]

        def fn():
            state[0] = (state[0] + 1) % len(sets)
            call(*sets[state[0]])
        # --sweep-mode restricts the run to one timing mode (for counter runs, where the two must not mix)
        cold = time_kernel(fn, args.steps, args.warmup) if args.sweep_mode in ("both", "rotating") else float("nan")
        warm = time_kernel(lambda: call(*sets[0]), args.steps, args.warmup) if args.sweep_mode in ("both", "resident") else float("nan")
        for st in sets:
            assert bool(torch.isfinite(st[0]).all()), "output is not finite"
        return cold, warm

    kernels = set(args.sweep_kernels.split(","))
    for dt, name in ((torch.float16, "f16"), (torch.bfloat16, "bf16")):
        if name not in args.sweep_dtypes.split(","):
            continue
        for t in [int(x) for x in args.sweep_rows.split(",")]:
            g = torch.Generator(device="cuda").manual_seed(0)
            rn = lambda *s: torch.randn(*s, generator=g, device="cuda").to(dt)
            b, ga, be, b2 = rn(768), rn(768), rn(768), rn(3072)
            if "ln" in kernels:
                us, warm = rotating(lambda: (rn(t, 768), rn(t, 768)),
                                    lambda x, r: capi.bias_residual_layernorm(x, r, b, ga, be, 1e-5), 2 * t * 768 * 2)
                rows.append(dict(hbm_roofline("bias_residual_layernorm_kernel", 3 * t * 768 * 2, us), tokens=t, dtype=name, us=us,
                                 us_resident=warm, frac_resident=3 * t * 768 * 2 / (warm * 1e-6) / HBM_PEAK))
            if "gelu" in kernels:
                us, warm = rotating(lambda: (rn(t, 3072),), lambda y: capi.bias_gelu(y, b2), t * 3072 * 2)
                rows.append(dict(hbm_roofline("bias_gelu_kernel", 2 * t * 3072 * 2, us), tokens=t, dtype=name, us=us,
                                 us_resident=warm, frac_resident=2 * t * 3072 * 2 / (warm * 1e-6) / HBM_PEAK))
            if "embed" not in kernels:
                continue
            # packed-input front end: fp32 tables (BigBird vocabulary 50358, 4096 positions), output in dt; per
            # token one fp32 word row read and one output row written (position / type rows recur and stay cached)
            gi = torch.Generator().manual_seed(0)
            word, pos, typ = (torch.randn(n, 768, generator=gi).cuda() for n in (50358, 4096, 2))
            ga32, be32 = torch.ones(768, device="cuda"), torch.zeros(768, device="cuda")
            pids = (torch.arange(t, dtype=torch.int32) % 4096).cuda()
            tids = torch.zeros(t, dtype=torch.int32, device="cuda")
            us, warm = rotating(lambda: (torch.empty(t, 768, dtype=dt, device="cuda"),
                                         torch.randint(0, 50358, (t,), generator=gi, dtype=torch.int32).cuda()),
                                lambda e, ids: capi.embed_layernorm(ids, pids, tids, word, pos, typ, ga32, be32, e),
                                t * 768 * (4 + 2))
            rows.append(dict(hbm_roofline("embed_layernorm_kernel", t * 768 * (4 + 2), us), tokens=t, dtype=name, us=us,
                             us_resident=warm, frac_resident=t * 768 * (4 + 2) / (warm * 1e-6) / HBM_PEAK))
    ln_rows = [r for r in rows if r["kernel"].startswith("bias_residual")]
    ln_fracs = [r["frac"] for r in ln_rows if r["frac"] == r["frac"]] or [r["frac_resident"] for r in ln_rows]
    best_ln = max(ln_fracs) if ln_fracs else float("nan")
    res = {"metric": "fused add-bias+LayerNorm / bias+GELU achieved HBM GB/s", "value": best_ln * 8000.0, "unit": "GB/s",
            "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": None, "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "f16/bf16", "data": "synthetic",
            "config": {"workload": "c4 memory-bound op sweep"}, "sweep": rows}
    if not args.no_cpu_baseline:
        res["cpu_baseline"] = cpu_baseline_membound()
    return res


def run_streaming(args):
    """Config 3's encoder fed a NEW batch every step (16 sequences, lengths uniform in [512, 4096], another draw
    each step), as a server sees it: the batch metadata, the LPT plan, the per-layer block indices and a GEMM plan
    for the new token count are all made inside the step, overlapped with the previous batch's layers."""
    pkg = graft.load_package()
    mb = importlib.import_module("raptor_t_amd.modeling_bert")
    ut = importlib.import_module("raptor_t_amd.util")
    hidden, heads, ffn, layers, dt = 768, 12, 3072, 12, torch.float16
    g = torch.Generator().manual_seed(0)
    layers_w = [mb.random_layer_weights(hidden, ffn, g, dtype=dt) for _ in range(layers)]
    mb.cxx.MetaData.set_plan(pkg.capi.RT_PLAN_HF, pkg.capi.RT_POLICY_REFERENCE_PATCHED, 4096)
    enc = mb.BertEncoder.from_weights(layers_w, heads, async_=not args.sync_index, eps=1e-5)
    meta = mb.cxx.MetaData()
    batches = [ut.uniform_lengths(16, 512, 4096, seed=100 + i) for i in range(args.warmup + args.steps)]
    max_t = max(sum(b) for b in batches)
    x0 = torch.randn(max_t, hidden, generator=g).to(dt).cuda()
    hs, tmp, attn, inter = (torch.empty(max_t, w, dtype=dt, device="cuda") for w in (hidden, hidden, hidden, ffn))
    host_prep = [0.0]

    def step(lens):
        t = sum(lens)
        h0 = time.perf_counter()
        spi, spi_t, total_comp, ppi_t, pp_t = ut.generate_data_metainfo(lens, 64, args.block_limit, heads)
        host_prep[0] += time.perf_counter() - h0
        h = hs[:t]
        h.copy_(x0[:t])
        meta.update_meta_data(t, spi[-1] + 1, total_comp, spi)
        enc(h, t, args.block_limit, spi, spi_t, ppi_t, pp_t, tmp[:t], inter[:t], attn[:t], test_info={},
            balanced=args.lpt_plan)

    mb.cxx.set_attention_host_plan(args.lpt_plan)
    # Start-up tuning, as a server does once: the GEMMs of every token count the batches can have (16 sequences of
    # 512..4096 tokens in steps of 64).  Without it the first batch of each token count stalls ~17 ms on timing
    # six candidate kernels per GEMM; --no-pretune shows that.
    tune_s = 0.0
    if not args.no_pretune:
        tune_s = mb.cxx.tune_layer_gemms(list(range(16 * 512, 16 * 4096 + 1, 64)), hidden, ffn, dt)
    for b in batches[:args.warmup]:
        step(b)
    torch.cuda.synchronize()
    host_prep[0] = 0.0
    t0 = time.perf_counter()
    for b in batches[args.warmup:]:
        step(b)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    meta.terminate_thread()
    assert bool(torch.isfinite(hs[:sum(batches[-1])]).all()), "the encoder's output is not finite"
    tokens = sum(sum(b) for b in batches[args.warmup:])
    return {"metric": METRIC, "value": 16 * args.steps / elapsed, "unit": "seqs/s", "n_gpus": 1, "steps": args.steps,
            "warmup": args.warmup, "ms_per_step": elapsed / args.steps * 1e3, "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
            "config": {"workload": "stream: config 3's encoder, a new batch of 16 lengths U[512,4096] every step",
                       "balanced": args.lpt_plan, "block_limit": args.block_limit},
            "tokens_per_s": tokens / elapsed, "host_batch_metadata_ms_per_step": host_prep[0] / args.steps * 1e3,
            "gemm_startup_tuning_s": tune_s}


def run_overlap(args):
    """Experiment behind the encoder's two-stream mode: config 3's batch as two micro-batches on two HIP streams of
    equal priority, one micro-batch's attention free to run beside the other's GEMMs, against the same kernels
    on one stream.  Every arrangement is timed in interleaved rounds inside this one process (clocks differ from
    box to box and drift over seconds):
      c_abi_one_stream / c_abi_two_micro_batches_one_stream / c_abi_two_streams   the library's entry points
                                                                                   called directly, no pipeline
      c_abi_split_beside_projection                                                whole batch on one stream, but the
                                                                                   K / V^T split of the first half of the
                                                                                   tokens on a second stream beside the
                                                                                   second half's projection GEMM
      layers_one_stream / layers_two_streams                                       BertEncoder.__call__ and
                                                                                   BertEncoder.call_two_streams"""
    pkg = graft.load_package()
    capi = pkg.capi
    mb = importlib.import_module("raptor_t_amd.modeling_bert")
    ut = importlib.import_module("raptor_t_amd.util")
    hidden, heads, ffn, layers, dt = 768, 12, 3072, 12, torch.float16
    seq_lens = ut.uniform_lengths(16, 512, 4096, seed=0)
    g = torch.Generator().manual_seed(0)
    weights = [mb.random_layer_weights(hidden, ffn, g, dtype=dt) for _ in range(layers)]
    wt = [{k: w[k].t().contiguous() for k in ("qkv_weight", "attn_out_weight", "inter_weight", "out_weight")}
          for w in weights]                                   # [out, in]: the layout the layer objects keep

    class Part:
        def __init__(self, lens):
            self.lens, self.t = lens, sum(lens)
            self.sb = capi.seq_prefix_blocks(lens)
            dev = lambda a: torch.from_numpy(a).cuda()
            self.sb_d = dev(self.sb)
            self.plans = [tuple(dev(a) for a in capi.build_to_index(self.sb, heads, seed=li)) for li in range(layers)]
            new = lambda *shape: torch.empty(*shape, dtype=dt, device="cuda")
            t = self.t
            self.x0 = torch.randn(t, hidden, generator=g).to(dt).cuda()
            self.x, self.qkv, self.k, self.vt = new(t, hidden), new(t, 3 * hidden), new(t * hidden), new(t * hidden)
            self.ctx, self.attn, self.inter, self.out = new(t, hidden), new(t, hidden), new(t, ffn), new(t, hidden)
            self.gemm = capi.Gemm()                           # one context (workspace) per stream

        def reset(self):
            self.x.copy_(self.x0)

        def layer(self, li):
            w, v, (idx_d, pos_d) = weights[li], wt[li], self.plans[li]
            self.gemm.bt(self.x, v["qkv_weight"], self.qkv)
            capi.qkv_bias_split(self.qkv, w["qkv_bias"], None, self.k, self.vt, self.sb_d, heads, capi.Q_SCALE)
            capi.bs_attention_fwd_qrows(self.qkv, w["qkv_bias"], capi.Q_SCALE, self.k, self.vt, self.ctx, self.sb_d, heads,
                                        idx_d, pos_d, heads)
            self.gemm.bt(self.ctx, v["attn_out_weight"], self.attn)
            capi.bias_residual_layernorm(self.attn, self.x, w["attn_out_bias"], w["attn_ln_weight"], w["attn_ln_bias"], 1e-5)
            self.gemm.bt(self.attn, v["inter_weight"], self.inter, bias=w["inter_bias"], epilogue=capi.RT_EPILOGUE_BIAS_GELU)
            self.gemm.bt(self.inter, v["out_weight"], self.out)
            capi.bias_residual_layernorm(self.out, self.attn, w["out_bias"], w["out_ln_weight"], w["out_ln_bias"], 1e-5)
            self.x, self.out = self.out, self.x

    whole = Part(seq_lens)
    run, cut = 0, 1
    for i, n in enumerate(seq_lens[:-1]):                      # the cut call_two_streams makes
        run += n
        if abs(2 * run - whole.t) < abs(2 * sum(seq_lens[:cut]) - whole.t) or i == 0:
            cut = i + 1
    halves = [Part(seq_lens[:cut]), Part(seq_lens[cut:])]
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]     # default priority, both

    def c_abi_one_stream():
        whole.reset()
        for li in range(layers):
            whole.layer(li)

    def c_abi_halves_one_stream():
        for p in halves:
            p.reset()
        for li in range(layers):
            for p in halves:
                p.layer(li)

    def c_abi_two_streams():
        cur = torch.cuda.current_stream()
        for p, st in zip(halves, streams):
            st.wait_stream(cur)
            with torch.cuda.stream(st):
                p.reset()
        for li in range(layers):                              # issue order: the two streams' layers alternate
            for p, st in zip(halves, streams):
                with torch.cuda.stream(st):
                    p.layer(li)
        for st in streams:
            cur.wait_stream(st)

    # The K / V^T split of the first half of the tokens on a second stream, beside the projection GEMM of the
    # second half (the projection cut at the same sequence boundary as the micro-batches); everything else
    # of the layer on the whole batch, one stream.
    t_a = halves[0].t
    side = torch.cuda.Stream()
    ev_a, ev_s = torch.cuda.Event(), torch.cuda.Event()

    def c_abi_split_beside_projection():
        whole.reset()
        cur = torch.cuda.current_stream()
        for li in range(layers):
            w, v, (idx_d, pos_d) = weights[li], wt[li], whole.plans[li]
            whole.gemm.bt(whole.x[:t_a], v["qkv_weight"], whole.qkv[:t_a])
            ev_a.record(cur)
            whole.gemm.bt(whole.x[t_a:], v["qkv_weight"], whole.qkv[t_a:])
            with torch.cuda.stream(side):
                side.wait_event(ev_a)
                capi.qkv_bias_split(whole.qkv[:t_a], w["qkv_bias"], None, whole.k[:t_a * hidden], whole.vt[:t_a * hidden],
                                    halves[0].sb_d, heads, capi.Q_SCALE)
                ev_s.record(side)
            capi.qkv_bias_split(whole.qkv[t_a:], w["qkv_bias"], None, whole.k[t_a * hidden:], whole.vt[t_a * hidden:],
                                halves[1].sb_d, heads, capi.Q_SCALE)
            cur.wait_event(ev_s)
            capi.bs_attention_fwd_qrows(whole.qkv, w["qkv_bias"], capi.Q_SCALE, whole.k, whole.vt, whole.ctx, whole.sb_d, heads,
                                        idx_d, pos_d, heads)
            whole.gemm.bt(whole.ctx, v["attn_out_weight"], whole.attn)
            capi.bias_residual_layernorm(whole.attn, whole.x, w["attn_out_bias"], w["attn_ln_weight"], w["attn_ln_bias"], 1e-5)
            whole.gemm.bt(whole.attn, v["inter_weight"], whole.inter, bias=w["inter_bias"], epilogue=capi.RT_EPILOGUE_BIAS_GELU)
            whole.gemm.bt(whole.inter, v["out_weight"], whole.out)
            capi.bias_residual_layernorm(whole.out, whole.attn, w["out_bias"], w["out_ln_weight"], w["out_ln_bias"], 1e-5)
            whole.x, whole.out = whole.out, whole.x

    enc = mb.BertEncoder.from_weights(weights, heads, async_=not args.sync_index, eps=1e-5)
    meta = mb.cxx.MetaData()
    t = whole.t
    spi, spi_t, total_comp, ppi_t, pp_t = ut.generate_data_metainfo(seq_lens, 64, args.block_limit, heads)
    hs = torch.empty(t, hidden, dtype=dt, device="cuda")
    tmp, attn, inter = (torch.empty(t, w_, dtype=dt, device="cuda") for w_ in (hidden, hidden, ffn))

    def layers_one_stream():
        hs.copy_(whole.x0)
        meta.update_meta_data(t, spi[-1] + 1, total_comp, spi)
        enc(hs, t, args.block_limit, spi, spi_t, ppi_t, pp_t, tmp, inter, attn, test_info={}, balanced=False)

    def layers_two_streams():
        hs.copy_(whole.x0)
        enc.call_two_streams(hs, seq_lens, args.block_limit, heads, tmp, inter, attn, test_info={}, balanced=False)

    def timed(fn):
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / args.steps * 1e3

    arrangements = (("c_abi_one_stream", c_abi_one_stream), ("c_abi_two_micro_batches_one_stream", c_abi_halves_one_stream),
                    ("c_abi_two_streams", c_abi_two_streams), ("c_abi_split_beside_projection", c_abi_split_beside_projection),
                    ("layers_one_stream", layers_one_stream),
                    ("layers_two_streams", layers_two_streams))
    for _, fn in arrangements:                                # GEMM plans of every size are tuned here
        timed(fn)
    rounds = {name: [] for name, _ in arrangements}
    for _ in range(5):
        for name, fn in arrangements:
            rounds[name].append(timed(fn))
    res = {name: float(np.median(v)) for name, v in rounds.items()}
    c_abi_one_stream()
    torch.cuda.synchronize()
    ref_c = whole.x.float().clone()
    c_abi_split_beside_projection()
    torch.cuda.synchronize()
    diff_split = (whole.x.float() - ref_c).abs().max().item()
    layers_one_stream()
    torch.cuda.synchronize()
    ref = hs.float().clone()
    layers_two_streams()
    torch.cuda.synchronize()
    meta.terminate_thread()
    assert bool(torch.isfinite(hs).all()) and bool(torch.isfinite(whole.x).all())
    diff = (hs.float() - ref).abs().max().item()
    best = res["layers_two_streams"]
    return {"metric": METRIC, "value": len(seq_lens) / (best * 1e-3), "unit": "seqs/s", "n_gpus": 1, "steps": args.steps,
            "warmup": args.warmup, "ms_per_step": best, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "f16", "data": "synthetic",
            "config": {"workload": "overlap experiment: config 3 as two micro-batches on two streams",
                       "micro_batches": [p.lens for p in halves], "tokens": [p.t for p in halves]},
            "ms_per_step_by_arrangement": res, "ms_per_step_rounds": rounds,
            "gain_c_abi": 1.0 - res["c_abi_two_streams"] / res["c_abi_one_stream"],
            "gain_layers": 1.0 - res["layers_two_streams"] / res["layers_one_stream"],
            "gain_split_beside_projection": 1.0 - res["c_abi_split_beside_projection"] / res["c_abi_one_stream"],
            "max_abs_diff_two_streams_vs_one": diff, "max_abs_diff_split_beside_projection": diff_split}


def run_issue_floor(args):
    """The figures behind the attention kernel's ceiling, from librt_probe.so (raptor-t_amd/csrc/probe_issue_floor.hip):
    the time one SIMD needs per block pair for the pair's 32 matrix instructions alone, with the 64 exponentials,
    with the 32 conversions, and with the packed row sums (the tile loop's whole instruction mix), every operand in
    registers, on one and on two waves per SIMD, together with the clock the CUs held meanwhile.  Prints, asserts
    nothing."""
    import ctypes
    path = os.path.join(ROOT, "raptor-t_amd", "lib", "librt_probe.so")
    if not os.path.exists(path):
        raise ImportError("%s is missing: run `make -C raptor-t_amd/csrc`" % path)
    lib = ctypes.CDLL(path)
    vp, I = ctypes.c_void_p, ctypes.c_int
    lib.rt_probe_issue_floor.argtypes = [I, I, I, I, vp, vp, vp]
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    out = torch.empty(cus * 512, dtype=torch.float32, device="cuda")
    clocks = torch.zeros(2 * cus, dtype=torch.int64, device="cuda")
    iters = 4000
    st = torch.cuda.current_stream().cuda_stream
    tick_hz = 100e6                                              # the constant-rate clock of wall_clock64()
    names = ["32 mfma", "+ 64 v_exp_f32", "+ 32 v_cvt_pk_f16_f32", "+ 32 v_pk_add_f16 (the loop's mix)"]
    rows = []
    for wps in (1, 2):
        for variant in range(4):
            def launch(n=iters):
                rc = lib.rt_probe_issue_floor(variant, wps, n, cus, out.data_ptr(), clocks.data_ptr(), st)
                assert rc == 0, rc
            for _ in range(3):
                launch()
            torch.cuda.synchronize()
            evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(5)]
            for a, b in evs:
                a.record()
                launch()
                b.record()
            torch.cuda.synchronize()
            us = float(np.median([a.elapsed_time(b) for a, b in evs])) * 1e3
            c = clocks.view(cus, 2).double().cpu()
            ghz = float((c[:, 0] / (c[:, 1] / tick_hz)).median()) / 1e9
            per_pair_us = us / (iters * wps)
            rows.append({"variant": names[variant], "waves_per_simd": wps, "kernel_us": us,
                         "us_per_pair_and_simd": per_pair_us, "cycles_per_pair_and_simd": per_pair_us * ghz * 1e3,
                         "clock_ghz": ghz,
                         "frac_of_2.5_pflops_if_nothing_else": PAIR_FLOP / (per_pair_us * 1e-6) * cus * 4 / 2.5e15})
    best = min(r["us_per_pair_and_simd"] for r in rows if r["variant"] == names[3])
    return {"metric": "issue floor of the attention tile loop: microseconds per block pair and SIMD", "value": best,
            "unit": "us", "n_gpus": 1, "steps": 5, "warmup": 3, "ms_per_step": None, "higher_is_better": False,
            "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
            "config": {"workload": "mfma_mix: instruction-issue probes, operands in registers", "iters": iters, "cus": cus},
            "rows": rows}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="c3", choices=["c3", "c1", "c2", "c4", "c5", "ref_e2e", "stream", "overlap", "mfma_mix"])
    ap.add_argument("--block-limit", type=int, default=1024, help="persistent workgroups of the balanced attention launch")
    ap.add_argument("--lpt-plan", action="store_true",
                    help="drive attention with the caller's LPT plan (the reference's balanced mode) instead of the kernel's own schedule")
    ap.add_argument("--sync-index", action="store_true", help="build the block index inline instead of on the workers")
    ap.add_argument("--no-epilogue-fusion", action="store_true",
                    help="keep bias + GELU as its own kernel instead of the intermediate GEMM's epilogue")
    ap.add_argument("--materialize-q", action="store_true",
                    help="the split kernel writes Q too and the attention kernel reads it from there (the reference's "
                         "arrangement) instead of taking its queries from the projection's output rows")
    ap.add_argument("--no-pretune", action="store_true",
                    help="stream workload: skip the start-up GEMM tuning over the range of token counts")
    ap.add_argument("--no-two-streams", action="store_true", help="skip the two-stream comparison after the timed steps")
    ap.add_argument("--sweep-rows", default="8192,32768,65536", help="c4: token counts of the sweep")
    ap.add_argument("--sweep-kernels", default="ln,gelu,embed", help="c4: which of ln, gelu, embed to run")
    ap.add_argument("--sweep-dtypes", default="f16,bf16", help="c4: which of f16, bf16 to run")
    ap.add_argument("--sweep-mode", default="both", choices=["both", "rotating", "resident"],
                    help="c4: time launches on buffers in rotation, on one buffer, or both")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-sample-seqs", type=int, default=2)
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (every sequence is independent: a batch would shard over GPUs by "
              "sequence, with no exchange); --gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)
    ut = importlib.import_module("raptor_t_amd.util") if graft.load_package() else None
    if args.workload == "c3":
        hidden, heads, ffn, layers, dtype, lens, max_pos = ENCODER_WORKLOADS["c3"]
        res = run_encoder(args, "c3: 12-layer BigBird-base, batch 16, len U[512,4096]", hidden, heads, ffn, layers, dtype,
                          lens(ut), max_pos=max_pos)
    elif args.workload == "c1":
        res = run_encoder(args, "c1: one BigBird-base layer, batch 1 x 1024 tokens, fp32 (the accuracy mode)", 768, 12,
                          3072, 1, "f32", [1024])
    elif args.workload == "c5":
        hidden, heads, ffn, layers, dtype, lens, max_pos = ENCODER_WORKLOADS["c5"]
        res = run_encoder(args, "c5: 24-layer BigBird-large shape, batch 4, len U[2048,16384], bf16", hidden, heads, ffn,
                          layers, dtype, lens(ut), max_pos=max_pos)
    elif args.workload == "ref_e2e":
        import random
        lens = ut.generate_array_with_avg(3584, 16, 4096, random.Random(0))
        res = run_encoder(args, "reference end2end row: batch 16, max 4096, avg 3584 (python/benchmark/metrics/end2end:31)",
                          768, 12, 3072, 12, "f16", lens)
        res["vs_baseline"] = res["value"] / (16 / 0.09359)
        res["baseline_note"] = "A100 fp16, 93.59 ms per 12-layer forward (other hardware)"
    elif args.workload == "c2":
        res = run_attention_only(args)
    elif args.workload == "stream":
        res = run_streaming(args)
    elif args.workload == "overlap":
        res = run_overlap(args)
    elif args.workload == "mfma_mix":
        res = run_issue_floor(args)
    else:
        res = run_membound_sweep(args)
    print(json.dumps(res))


if __name__ == "__main__":
    main()
