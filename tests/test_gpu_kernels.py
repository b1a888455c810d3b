"""GPU parity tests: every kernel is called through the C-ABI and compared with the CPU
oracle on the same seeded inputs.  Tolerances: 2e-2 abs error per element for fp16/bf16 outputs
(k ulp of the output type where one ulp of the expected value exceeds that: layer_harness.excess),
1e-4 for fp32 (values of order one); integer/layout work is bit exact."""
import math
import sys

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import __graft_entry__ as graft
from oracle import attention as oa
from oracle import layer as ol
from oracle import metadata as md
from tests import layer_harness as lh

pytestmark = pytest.mark.gpu

TOL = {torch.float16: 2e-2, torch.bfloat16: 2e-2, torch.float32: 1e-4}


@pytest.fixture(scope="module")
def capi():
    pkg = graft.load_package()
    pkg.capi.lib()
    assert torch.cuda.is_available()
    return pkg.capi


def say(*a):
    print(*a, flush=True)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("rows,hidden", [(1000, 768), (517, 1024), (64, 3072), (33, 4096), (9, 520), (8192, 768)])
def test_bias_residual_layernorm(capi, dtype, rows, hidden):
    say("LN", dtype, rows, hidden)
    g = torch.Generator().manual_seed(rows + hidden)
    x, r = torch.randn(rows, hidden, generator=g), torch.randn(rows, hidden, generator=g)
    b, ga, be = (torch.randn(hidden, generator=g) for _ in range(3))
    xd, rd, bd, gd, bed = (t.to(dtype).cuda() for t in (x, r, b, ga, be))
    want = ol.bias_residual_layernorm(xd.cpu(), rd.cpu(), bd.cpu(), gd.cpu(), bed.cpu(), 1e-5)
    capi.bias_residual_layernorm(xd, rd, bd, gd, bed, 1e-5)
    torch.cuda.synchronize()
    # outputs reach |y| ~ 10 here (gamma, beta ~ N(0,1)): one rounding to the output type, so one ulp
    assert lh.excess(xd, want, dtype, k=1.0) <= 0


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("rows,width", [(777, 3072), (130, 4096), (5, 40), (8192, 3072)])
def test_bias_gelu(capi, dtype, rows, width):
    say("GELU", dtype, rows, width)
    g = torch.Generator().manual_seed(rows)
    x, b = torch.randn(rows, width, generator=g) * 2, torch.randn(width, generator=g)
    xd, bd = x.to(dtype).cuda(), b.to(dtype).cuda()
    want = ol.bias_gelu(xd.cpu(), bd.cpu())
    capi.bias_gelu(xd, bd)
    torch.cuda.synchronize()
    assert lh.excess(xd, want, dtype, k=1.0) <= 0


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("rows", [32768, 65536])
def test_memory_bound_kernels_at_benchmark_row_counts(capi, dtype, rows):
    """The row counts of the memory-bound benchmark (32 K and 64 K tokens; the reference sweeps them in
    python/benchmark/mem_bound_op.py:93-108): bias + GELU over [rows, 3072], whose launch is capped so that every
    workgroup walks its grid-stride loop several times, and bias + residual + LayerNorm over [rows, 768]."""
    say("membound at benchmark size", dtype, rows)
    g = torch.Generator().manual_seed(rows)
    x = (torch.randn(rows, 3072, generator=g) * 2).to(dtype)
    b = torch.randn(3072, generator=g).to(dtype)
    xd, bd = x.cuda(), b.cuda()
    capi.bias_gelu(xd, bd)
    torch.cuda.synchronize()
    got = xd.cpu()
    for r0 in range(0, rows, 8192):
        want = ol.bias_gelu(x[r0:r0 + 8192], b)
        assert lh.excess(got[r0:r0 + 8192], want, dtype, k=1.0) <= 0, r0
    del xd, got
    x = torch.randn(rows, 768, generator=g).to(dtype)
    r = torch.randn(rows, 768, generator=g).to(dtype)
    b, ga, be = (torch.randn(768, generator=g).to(dtype) for _ in range(3))
    xd = x.cuda()
    capi.bias_residual_layernorm(xd, r.cuda(), b.cuda(), ga.cuda(), be.cuda(), 1e-5)
    torch.cuda.synchronize()
    got = xd.cpu()
    for r0 in range(0, rows, 8192):
        want = ol.bias_residual_layernorm(x[r0:r0 + 8192], r[r0:r0 + 8192], b, ga, be, 1e-5)
        assert lh.excess(got[r0:r0 + 8192], want, dtype, k=1.0) <= 0, r0


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_qkv_bias_split_layout_bit_exact(capi, dtype):
    say("split", dtype)
    heads, lens = 3, [256, 64, 832]
    sb = capi.seq_prefix_blocks(lens)
    t, dm = int(sb[-1]) * 64, heads * 64
    g = torch.Generator().manual_seed(4)
    qkv = torch.randn(t, 3 * dm, generator=g).to(dtype).cuda()
    bias = torch.randn(3 * dm, generator=g).to(dtype).cuda()
    q, k, vt = (torch.empty(t * dm, dtype=dtype, device="cuda") for _ in range(3))
    capi.qkv_bias_split(qkv, bias, q, k, vt, torch.from_numpy(sb).cuda(), heads, 0.125)
    oq, ok, ov = ol.qkv_bias_split(qkv.cpu(), bias.cpu(), heads, 0.125)
    rnd = lambda a: a.to(dtype)
    assert torch.equal(q.cpu(), lh.pack_heads(rnd(oq), sb))
    assert torch.equal(k.cpu(), lh.pack_heads(rnd(ok), sb))
    assert torch.equal(vt.cpu(), lh.pack_heads(rnd(ov), sb, transpose_v=True))
    for packed, want, tr in ((q, oq, False), (k, ok, False), (vt, ov, True)):
        flat = torch.empty(t, dm, dtype=dtype, device="cuda")
        capi.unpack_head_tiles(packed, flat, torch.from_numpy(sb).cuda(), heads, tr)
        assert torch.equal(flat.cpu().view(t, heads, 64), rnd(want))
    # without a Q output (the attention kernel then reads its queries from `qkv`): K and V^T unchanged
    k2, vt2 = (torch.full((t * dm,), float("nan"), dtype=dtype, device="cuda") for _ in range(2))
    capi.qkv_bias_split(qkv, bias, None, k2, vt2, torch.from_numpy(sb).cuda(), heads, 0.125)
    torch.cuda.synchronize()
    assert torch.equal(k2, k) and torch.equal(vt2, vt)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("lens,heads,n_wg", [
    ([768], 2, 0), ([1024, 64, 832, 512], 3, 0), ([1024, 64, 832, 512], 3, 7), ([2048, 768], 12, 160),
    ([64], 1, 0), ([128, 192], 2, 3),
])
def test_attention_matches_oracle(capi, dtype, lens, heads, n_wg):
    say("attention", dtype, lens, heads, n_wg)
    t = sum(lens)
    g = torch.Generator().manual_seed(len(lens) * 100 + heads)
    q, k, v = (torch.randn(t, heads, 64, generator=g).to(dtype).cuda() for _ in range(3))
    out, ref = lh.run_attention(capi, q, k, v, lens, heads, seed=1, n_wg=n_wg)
    assert not torch.isnan(out).any()
    assert (out.float().cpu() - ref).abs().max().item() <= TOL[dtype]


@pytest.mark.parametrize("n_wg", [0, 37])
def test_attention_rows_longer_than_64_blocks(capi, n_wg):
    """Sequences beyond 4096 tokens (the BigBird-large configuration goes to 16384): the two global rows
    list more than 64 key blocks, which the kernel walks in chunks of 64 ids, also when four waves share
    the row; 65 blocks puts a single entry into the second chunk."""
    say("attention long rows", n_wg)
    lens, heads = [8192, 4160, 768], 2
    t = sum(lens)
    g = torch.Generator().manual_seed(21)
    q, k, v = (torch.randn(t, heads, 64, generator=g).half().cuda() for _ in range(3))
    out, ref = lh.run_attention(capi, q, k, v, lens, heads, seed=4, n_wg=n_wg, max_pos=16384)
    assert not torch.isnan(out).any()
    assert (out.float().cpu() - ref).abs().max().item() <= 2e-2


@pytest.mark.parametrize("n_wg,padded,from_rows", [(0, False, False), (5, True, False), (0, True, True), (9, False, True)])
def test_attention_fp32_mode(capi, n_wg, padded, from_rows):
    """The fp32 instantiation (the layer's accuracy mode; config 1 of the benchmark runs in it) to 1e-4: a sparse
    sequence, a short one, a global row of more than 64 key blocks, padded tails, queries taken from the projection's
    rows, with and without a work plan."""
    say("attention fp32", n_wg, padded, from_rows)
    heads, seq_lens = 3, [64 * 13, 64 * 3, 64 * 66, 64]
    t, dm = sum(seq_lens), heads * 64
    g = torch.Generator().manual_seed(15)
    qkv = torch.randn(t, 3 * dm, generator=g).cuda()
    bias = (torch.randn(3 * dm, generator=g) * 0.5).cuda()
    sb, idx, pos, ph, sb_d, idx_d, pos_d = lh.device_plan(capi, seq_lens, heads, 2, None, max_pos=16384)
    seq_tokens = [n - 23 for n in seq_lens] if padded else None
    tok_d = None if seq_tokens is None else torch.tensor(seq_tokens, dtype=torch.int32).cuda()
    from_idx = from_pos = None
    if n_wg:
        fp, fi = capi.partition_lpt(sb, heads, n_wg)
        from_pos, from_idx = torch.from_numpy(fp).cuda(), torch.from_numpy(fi).cuda()
    new = lambda: torch.full((t * dm,), float("nan"), device="cuda")
    q, k, vt, out = new(), new(), new(), new().view(t, dm)
    if from_rows:
        capi.qkv_bias_split(qkv, bias, None, k, vt, sb_d, heads, capi.Q_SCALE)
        capi.bs_attention_fwd_qrows(qkv, bias, capi.Q_SCALE, k, vt, out, sb_d, heads, idx_d, pos_d, ph, from_idx, from_pos,
                                    tok_d)
    else:
        capi.qkv_bias_split(qkv, bias, q, k, vt, sb_d, heads, capi.Q_SCALE)
        capi.bs_attention_fwd(q, k, vt, out, sb_d, heads, idx_d, pos_d, ph, from_idx, from_pos, tok_d)
    torch.cuda.synchronize()
    x = qkv.cpu() + bias.cpu()
    qs = (x[:, :dm] * capi.Q_SCALE).view(t, heads, 64)
    kk, vv = (x[:, i * dm:(i + 1) * dm].view(t, heads, 64) for i in (1, 2))
    ref = oa.csr_attention(qs, kk, vv, sb.tolist(), idx, pos, ph, scale=1.0 / lh.LOG2E, seq_tokens=seq_tokens)
    rows = torch.ones(t, dtype=torch.bool)
    if padded:                                             # padded query rows are computed but not specified
        start = 0
        for n, real in zip(seq_lens, seq_tokens):
            rows[start + real:start + n] = False
            start += n
    assert torch.isfinite(out).all()
    assert (out.cpu()[rows] - ref[rows]).abs().max().item() <= 1e-4


def test_encoder_layer_config1_fp32(capi):
    """Benchmark config 1 on the GPU path: one BigBird-base layer, batch 1, 1024 tokens, hidden 768, 12 heads, FFN 3072,
    every tensor fp32, against the oracle to 1e-4."""
    say("layer config 1 fp32")
    pkg = graft.load_package()
    out, want = lh.run_layer_case_tensors(pkg, [1024], 768, 12, 3072, torch.float32, seed=0)
    err = (out - want).abs().max().item()
    say("  err", err)
    assert err <= 1e-4


@pytest.mark.parametrize("n_wg", [0, 128])
def test_attention_long_rows_bf16_sixteen_heads(capi, n_wg):
    """The large configuration's shape (16 heads, bf16, sequences beyond 4096 tokens, plans drawn for 16384
    positions): global rows of 130 and 65 key blocks in the bf16 instantiation, against the oracle."""
    say("attention long rows bf16", n_wg)
    lens, heads = [8320, 4160], 16
    t = sum(lens)
    g = torch.Generator().manual_seed(22)
    q, k, v = (torch.randn(t, heads, 64, generator=g).bfloat16().cuda() for _ in range(3))
    out, ref = lh.run_attention(capi, q, k, v, lens, heads, seed=6, n_wg=n_wg, max_pos=16384)
    assert torch.isfinite(out.float()).all()
    assert lh.excess(out, ref, torch.bfloat16, k=1.0) <= 0


def test_attention_config3_full_size_properties(capi):
    """Benchmark config 3 (16 sequences of 512 to 4096 tokens, 12 heads, fp16) at full size: finite everywhere,
    the global rows of a sparse and of a short sequence equal dense attention over the sequence, one sampled
    (sequence, head) equals the oracle, and the host's LPT partition gives the same result."""
    say("attention config 3")
    heads = 12
    lens = (64 * np.random.default_rng(0).integers(8, 65, size=16)).tolist()
    t = sum(lens)
    g = torch.Generator(device="cuda").manual_seed(1)
    q, k, v = (torch.randn(t, heads, 64, generator=g, device="cuda", dtype=torch.float16) for _ in range(3))
    sb, idx, pos, ph, sb_d, idx_d, pos_d = lh.device_plan(capi, lens, heads, seed=3)
    qs = (q.float() * (lh.LOG2E / 8)).half()
    qp, kp, vp = lh.pack_heads(qs, sb), lh.pack_heads(k, sb), lh.pack_heads(v, sb, transpose_v=True)
    out = torch.full((t, heads * 64), float("nan"), dtype=torch.float16, device="cuda")
    capi.bs_attention_fwd(qp, kp, vp, out, sb_d, heads, idx_d, pos_d, ph)
    fp, fi = capi.partition_lpt(sb, heads, 512)
    out_b = torch.full_like(out, float("nan"))
    capi.bs_attention_fwd(qp, kp, vp, out_b, sb_d, heads, idx_d, pos_d, ph, torch.from_numpy(fi).cuda(), torch.from_numpy(fp).cuda())
    torch.cuda.synchronize()
    assert torch.isfinite(out).all() and torch.isfinite(out_b).all()
    assert (out.float() - out_b.float()).abs().max().item() <= 5e-4
    longest, shortest = int(np.argmax(lens)), int(np.argmin(lens))
    assert lens[longest] >= 12 * 64
    for s in (longest, shortest):
        sel = slice(int(sb[s]) * 64, int(sb[s + 1]) * 64)
        qq, kk, vv = (x[sel].transpose(0, 1).float() for x in (q, k, v))
        rows = (slice(0, 64), slice(lens[s] - 64, lens[s])) if lens[s] >= 12 * 64 else (slice(0, lens[s]),)
        for r in rows:                                       # below 12 blocks every row attends to the whole sequence
            dense = F.scaled_dot_product_attention(qq[:, r], kk, vv).transpose(0, 1)
            assert (out[sel][r].view(-1, heads, 64).float() - dense).abs().max().item() <= 2e-2
    s, h = longest, 5
    n = lens[s] // 64
    sel = slice(int(sb[s]) * 64, int(sb[s + 1]) * 64)
    one_idx, one_pos = [], [0]
    for i in range(n):
        r = h * int(sb[-1]) + int(sb[s]) + i
        one_idx.extend(idx[pos[r]:pos[r + 1]].tolist())
        one_pos.append(len(one_idx))
    ref = oa.csr_attention(qs[sel, h:h + 1].cpu(), k[sel, h:h + 1].cpu(), v[sel, h:h + 1].cpu(), [0, n],
                           np.array(one_idx), np.array(one_pos), 1, scale=1.0 / lh.LOG2E)
    assert (out[sel, h * 64:(h + 1) * 64].float().cpu() - ref).abs().max().item() <= 2e-2


@pytest.mark.parametrize("dtype,n_wg,padded", [(torch.float16, 0, False), (torch.bfloat16, 0, False),
                                               (torch.float16, 96, False), (torch.float16, 0, True)])
def test_attention_queries_from_projection_rows(capi, dtype, n_wg, padded):
    """rt_bs_attention_fwd_qrows (queries read from the [T, 3*H*64] projection output, bias and scale applied on
    load; the split kernel called without a Q output) gives the same bits as the route through a materialised Q,
    and both match the oracle; likewise with the bias already in the rows and none handed to either kernel."""
    say("attention qrows", dtype, n_wg, padded)
    heads, seq_lens = 4, [64 * 13, 64 * 3, 64 * 20, 64]
    t, dm = sum(seq_lens), heads * 64
    g = torch.Generator().manual_seed(5)
    qkv = torch.randn(t, 3 * dm, generator=g).to(dtype).cuda()
    bias = (torch.randn(3 * dm, generator=g) * 0.5).to(dtype).cuda()
    sb, idx, pos, ph, sb_d, idx_d, pos_d = lh.device_plan(capi, seq_lens, heads, 0, None)
    seq_tokens = [n - 17 for n in seq_lens] if padded else None
    tok_d = None if seq_tokens is None else torch.tensor(seq_tokens, dtype=torch.int32).cuda()
    from_idx = from_pos = None
    if n_wg:
        fp, fi = capi.partition_lpt(sb, heads, n_wg)
        from_pos, from_idx = torch.from_numpy(fp).cuda(), torch.from_numpy(fi).cuda()
    new = lambda: torch.full((t * dm,), float("nan"), dtype=dtype, device="cuda")
    q, k, vt, k2, vt2 = new(), new(), new(), new(), new()
    out_a, out_b = new().view(t, dm), new().view(t, dm)
    capi.qkv_bias_split(qkv, bias, q, k, vt, sb_d, heads, capi.Q_SCALE)
    capi.bs_attention_fwd(q, k, vt, out_a, sb_d, heads, idx_d, pos_d, ph, from_idx, from_pos, tok_d)
    capi.qkv_bias_split(qkv, bias, None, k2, vt2, sb_d, heads, capi.Q_SCALE)
    capi.bs_attention_fwd_qrows(qkv, bias, capi.Q_SCALE, k2, vt2, out_b, sb_d, heads, idx_d, pos_d, ph, from_idx,
                                from_pos, tok_d)
    torch.cuda.synchronize()
    assert torch.equal(k, k2) and torch.equal(vt, vt2)
    assert torch.equal(out_a, out_b)
    x = qkv.float().cpu() + bias.float().cpu()
    qs = (x[:, :dm] * capi.Q_SCALE).to(dtype).view(t, heads, 64)
    kk, vv = (x[:, i * dm:(i + 1) * dm].to(dtype).view(t, heads, 64) for i in (1, 2))
    ref = oa.csr_attention(qs, kk, vv, sb.tolist(), idx, pos, ph, scale=1.0 / lh.LOG2E, seq_tokens=seq_tokens)
    assert (out_b.float().cpu() - ref).abs().max().item() <= 2e-2
    # rows that carry the bias already (what the projection's bias epilogue leaves), no bias handed over: the split
    # kernel only changes the layout, the attention kernel only applies the scale; same bits as with the bias
    # added by the kernels whenever row + bias is exact in the tensor type (here: the rows hold x + b rounded once)
    rows = (qkv.float() + bias.float()).to(dtype)
    zero = torch.zeros_like(bias)
    q3, k3, vt3, k4, vt4 = new(), new(), new(), new(), new()
    out_c, out_d = new().view(t, dm), new().view(t, dm)
    capi.qkv_bias_split(rows, zero, q3, k3, vt3, sb_d, heads, capi.Q_SCALE)
    capi.bs_attention_fwd(q3, k3, vt3, out_c, sb_d, heads, idx_d, pos_d, ph, from_idx, from_pos, tok_d)
    capi.qkv_bias_split(rows, None, None, k4, vt4, sb_d, heads, capi.Q_SCALE)
    capi.bs_attention_fwd_qrows(rows, None, capi.Q_SCALE, k4, vt4, out_d, sb_d, heads, idx_d, pos_d, ph, from_idx,
                                from_pos, tok_d)
    torch.cuda.synchronize()
    assert torch.equal(k3, k4) and torch.equal(vt3, vt4) and torch.equal(out_c, out_d)
    assert (out_d.float().cpu() - ref).abs().max().item() <= 2e-2


def test_attention_maximum_batch(capi):
    """1024 sequences in one launch is the limit of the kernel's LDS geometry tables; one more is refused."""
    say("attention max batch")
    heads = 1
    lens = [64] * 1000 + [128] * 24
    t = sum(lens)
    g = torch.Generator().manual_seed(5)
    q, k, v = (torch.randn(t, heads, 64, generator=g).half().cuda() for _ in range(3))
    out, ref = lh.run_attention(capi, q, k, v, lens, heads, seed=0)
    assert (out.float().cpu() - ref).abs().max().item() <= 2e-2
    lens = [64] * 1025
    t = sum(lens)
    q, k, v = (torch.zeros(t, heads, 64).half().cuda() for _ in range(3))
    with pytest.raises(capi.RaptorError):
        lh.run_attention(capi, q, k, v, lens, heads, seed=0)


def test_attention_reference_plan_shared_heads(capi):
    say("attention reference plan")
    lens, heads = [1024, 1536], 4
    t = sum(lens)
    g = torch.Generator().manual_seed(7)
    q, k, v = (torch.randn(t, heads, 64, generator=g).half().cuda() for _ in range(3))
    out, ref = lh.run_attention(capi, q, k, v, lens, heads, seed=5, mode=capi.RT_PLAN_REFERENCE, n_wg=11)
    assert (out.float().cpu() - ref).abs().max().item() <= 2e-2


def test_attention_on_the_reference_test_case(capi):
    """The one attention test the reference itself runs (layers/test.cpp:78-242): a single 4096-token sequence,
    12 heads, Q = K = V = the ramp 6/4095 * (i % 4096) - 2 over the head-major [12][64][64][64] buffer (:11-16,
    :182-196), its hard-coded block index shared by all heads (:89-91) and its 160-CTA partition (:95-164), which
    the kernel walks here.  The reference compares its fp16 kernel with its fp32 one at 0.1 (:35-48); the oracle
    is held to this build's 2e-2.  Scores reach 1000, so every row takes the moving-maximum route."""
    import json, os
    say("attention, reference test case")
    gold = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "layers_test_n64_h12_cta160.json")))
    heads, n = 12, 64
    i = torch.arange(heads * n * 64 * 64, dtype=torch.float64)
    ramp = (6.0 / 4095.0 * (i % 4096) - 2.0).view(heads, n * 64, 64).permute(1, 0, 2)      # token-major [T, H, d]
    k = v = ramp.to(torch.float16)
    qs = (ramp * lh.LOG2E).to(torch.float16)                    # the kernel's softmax is base 2
    sb = capi.seq_prefix_blocks([4096])
    idx = np.asarray(gold["to_select_index"], dtype=np.int32)
    pos = np.asarray(gold["to_select_index_position"], dtype=np.int32)
    fi = np.asarray(gold["from_select_index"], dtype=np.int32)
    fp = np.asarray(gold["from_select_index_position"], dtype=np.int32)
    dev = lambda a: torch.from_numpy(a).cuda()
    qp, kp = lh.pack_heads(qs.cuda(), sb), lh.pack_heads(k.cuda(), sb)
    vp = lh.pack_heads(v.cuda(), sb, transpose_v=True)
    ref = oa.csr_attention(qs, k, v, sb.tolist(), idx, pos, 1, scale=1.0 / lh.LOG2E)
    outs = []
    for plan in ((dev(fi), dev(fp)), (None, None)):             # the reference's partition / the kernel's own schedule
        out = torch.full((4096, heads * 64), float("nan"), dtype=torch.float16, device="cuda")
        capi.bs_attention_fwd(qp, kp, vp, out, dev(sb), heads, dev(idx), dev(pos), 1, plan[0], plan[1], None)
        torch.cuda.synchronize()
        outs.append(out.float().cpu())
        assert (outs[-1] - ref).abs().max().item() <= 2e-2
    assert torch.equal(outs[0], outs[1])


def test_attention_large_logits_and_constant_v(capi):
    """Online softmax must survive scores of several hundred; constant V must come back exactly."""
    say("attention extremes")
    lens, heads = [896], 2
    g = torch.Generator().manual_seed(3)
    q, k = (torch.randn(896, heads, 64, generator=g) * 6 for _ in range(2))
    v = torch.full((896, heads, 64), 0.75)
    out, ref = lh.run_attention(capi, q.half().cuda(), k.half().cuda(), v.half().cuda(), lens, heads)
    assert torch.isfinite(out).all()
    assert (out.float().cpu() - 0.75).abs().max().item() <= 1e-3
    v2 = torch.randn(896, heads, 64, generator=g)
    out, ref = lh.run_attention(capi, q.half().cuda(), k.half().cuda(), v2.half().cuda(), lens, heads)
    assert (out.float().cpu() - ref).abs().max().item() <= 2e-2


def test_attention_config2_full_size_properties(capi):
    """Benchmark config 2 (batch 8 x 4096 tokens, 12 heads, fp16): too big for the CPU oracle, so
    check what the mathematics fixes: global rows equal dense SDPA over the sequence, a
    sample of sparse rows equals the oracle on that one (sequence, head), balanced == unbalanced."""
    say("attention config 2")
    lens, heads = [4096] * 8, 12
    t = sum(lens)
    g = torch.Generator(device="cuda").manual_seed(0)
    q, k, v = (torch.randn(t, heads, 64, generator=g, device="cuda", dtype=torch.float16) for _ in range(3))
    sb, idx, pos, ph, sb_d, idx_d, pos_d = lh.device_plan(capi, lens, heads, seed=0)
    assert len(idx) == 12 * 8 * 622
    qs = (q.float() * (lh.LOG2E / 8)).half()
    qp, kp, vp = lh.pack_heads(qs, sb), lh.pack_heads(k, sb), lh.pack_heads(v, sb, transpose_v=True)
    out = torch.empty(t, heads * 64, dtype=torch.float16, device="cuda")
    capi.bs_attention_fwd(qp, kp, vp, out, sb_d, heads, idx_d, pos_d, ph)
    fp, fi = capi.partition_lpt(sb, heads, 512)
    out_b = torch.empty_like(out)
    capi.bs_attention_fwd(qp, kp, vp, out_b, sb_d, heads, idx_d, pos_d, ph, torch.from_numpy(fi).cuda(), torch.from_numpy(fp).cuda())
    torch.cuda.synchronize()
    # same algorithm, two inlined copies of the wave loop: results may differ in the last fp16 bit
    assert (out.float() - out_b.float()).abs().max().item() <= 5e-4
    o4 = out.view(8, 4096, heads, 64)
    for s in (0, 5):
        qq, kk, vv = (x.view(8, 4096, heads, 64)[s].transpose(0, 1).float() for x in (q, k, v))
        for rows in (slice(0, 64), slice(4032, 4096)):
            dense = F.scaled_dot_product_attention(qq[:, rows], kk, vv).transpose(0, 1)
            assert (o4[s, rows].float() - dense).abs().max().item() <= 2e-2
    s, h = 3, 7
    sel = slice(s * 4096, (s + 1) * 4096)
    one_idx, one_pos = [], [0]
    for i in range(64):
        r = h * int(sb[-1]) + s * 64 + i
        one_idx.extend(idx[pos[r]:pos[r + 1]].tolist())
        one_pos.append(len(one_idx))
    ref = oa.csr_attention(qs[sel, h:h + 1].cpu(), k[sel, h:h + 1].cpu(), v[sel, h:h + 1].cpu(), [0, 64],
                           np.array(one_idx), np.array(one_pos), 1, scale=1.0 / lh.LOG2E)
    assert (out[sel, h * 64:(h + 1) * 64].float().cpu() - ref).abs().max().item() <= 2e-2

@pytest.mark.parametrize("dtype,n_wg,reference_plan", [(torch.float16, 0, False), (torch.bfloat16, 0, False),
                                                       (torch.float16, 96, False), (torch.float16, 0, True),
                                                       (torch.bfloat16, 96, True)])
def test_attention_padded_tail_matches_oracle(capi, dtype, n_wg, reference_plan):
    """Sequences whose last block ends in padding: the keys past the true length get no weight.  Covers a
    sparse sequence, a full-attention one (below 12 blocks), a tail of a single token, no padding at all, a
    sequence of one block (its only tile is the padded one: the pipelined loop's reference has to leave the
    padded keys out too) and one of two; 768 tokens are 12 blocks, where rows list the last block twice (those
    take the moving-maximum loop), and the reference's head-shared plan keeps more duplicates still.  The padded
    rows hold large values so that a missed mask shows."""
    say("attention padded", dtype, n_wg, reference_plan)
    heads = 4
    seq_lens = [1024, 320, 832, 768, 64, 128]
    seq_tokens = [1000, 257, 832, 705, 40, 100]
    _check_padded_attention(capi, dtype, n_wg, reference_plan, heads, seq_lens, seq_tokens)


@pytest.mark.parametrize("dtype,n_wg,reference_plan", [(torch.float16, 0, False), (torch.bfloat16, 0, False),
                                                       (torch.float32, 0, False), (torch.float16, 96, False),
                                                       (torch.bfloat16, 0, True)])
def test_attention_padded_blocks_match_oracle(capi, dtype, n_wg, reference_plan):
    """Sequences kept at a padded batch's width: whole blocks of padding behind the real tokens.  Their keys get no
    weight (the tiles are taken off the pipelined loop's list), the block the real tokens end in is masked from
    the tail on.  Covers real tokens ending inside a block and exactly at a block's end, a single real block, a
    single real token, and a sequence without padding beside them."""
    say("attention padded blocks", dtype, n_wg, reference_plan)
    heads = 4
    seq_lens = [1024, 1024, 1024, 768, 320, 1024, 832]
    seq_tokens = [700, 128, 50, 100, 64, 1, 832]
    _check_padded_attention(capi, dtype, n_wg, reference_plan, heads, seq_lens, seq_tokens)


def _check_padded_attention(capi, dtype, n_wg, reference_plan, heads, seq_lens, seq_tokens):
    t = sum(seq_lens)
    g = torch.Generator().manual_seed(11)
    q, k, v = (torch.randn(t, heads, 64, generator=g) for _ in range(3))
    start = 0
    for n, real in zip(seq_lens, seq_tokens):              # loud padding: a key that would dominate if it counted
        k[start + real:start + n] = 6.0 * torch.sign(q[start:start + 1])
        v[start + real:start + n] = 50.0
        start += n
    q, k, v = (x.to(dtype).cuda() for x in (q, k, v))
    out, ref = lh.run_attention(capi, q, k, v, seq_lens, heads, seed=2, n_wg=n_wg, seq_tokens=seq_tokens,
                                mode=capi.RT_PLAN_REFERENCE if reference_plan else None)
    start = 0
    for n, real in zip(seq_lens, seq_tokens):              # real query rows only
        over = lh.excess(out[start:start + real], ref[start:start + real], dtype, k=1.0)
        assert over <= 0, (n, real, over)
        start += n
    assert torch.isfinite(out.float()).all()



@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_gemm_matches_torch(capi, dtype):
    say("gemm", dtype)
    g = torch.Generator().manual_seed(0)
    gemm = capi.Gemm()
    for m, n, k in [(832, 2304, 768), (832, 768, 3072), (64, 768, 768)]:
        a = torch.randn(m, k, generator=g).to(dtype).cuda()
        b = (torch.randn(k, n, generator=g) * 0.05).to(dtype).cuda()
        c = torch.empty(m, n, dtype=dtype, device="cuda")
        gemm(a, b, c)
        torch.cuda.synchronize()
        want = a.float().cpu() @ b.float().cpu()
        tol = 2e-2 if dtype != torch.float32 else 2e-3
        assert (c.float().cpu() - want).abs().max().item() <= tol * max(1.0, want.abs().max().item() / 4)
    gemm.close()


def test_gemm_exhaustive_tuning_keeps_results(capi):
    """RT_GEMM_TUNE_ALL times every library solution once per (N, K, dtype); later calls with another M reuse
    the winner by index.  Results must not depend on the tuning mode."""
    say("gemm tune all")
    g = torch.Generator().manual_seed(2)
    a = torch.randn(320, 256, generator=g).half().cuda()
    b = (torch.randn(256, 512, generator=g) * 0.05).half().cuda()
    want = a.float().cpu() @ b.float().cpu()
    for mode in (1, capi.RT_GEMM_TUNE_ALL):
        gemm = capi.Gemm()
        gemm.set_tuning(mode)
        for rows in (320, 192):                       # the second M takes the cached winner
            c = torch.empty(rows, 512, dtype=torch.float16, device="cuda")
            gemm(a[:rows].contiguous(), b, c)
            torch.cuda.synchronize()
            assert (c.float().cpu() - want[:rows]).abs().max().item() <= 2e-2
        gemm.close()
    gemm = capi.Gemm()
    with pytest.raises(capi.RaptorError):
        gemm.set_tuning(0)
    with pytest.raises(capi.RaptorError):
        gemm.set_retuning(9)
    gemm.close()


@pytest.mark.parametrize("dtype,width", [(torch.float16, 768), (torch.bfloat16, 1024), (torch.float32, 200)])
def test_sequence_pool_matches_oracle(capi, dtype, width):
    say("sequence pool", dtype, width)
    g = torch.Generator().manual_seed(9)
    seq_lens = [64 * 5, 64, 64 * 33, 64 * 2]
    sb = capi.seq_prefix_blocks(seq_lens)
    sb_d = torch.from_numpy(sb).cuda()
    hidden = torch.randn(sum(seq_lens), width, generator=g).to(dtype).cuda()
    tokens = [300, 1, 64 * 33 - 63, 128]
    tok_d = torch.tensor(tokens, dtype=torch.int32).cuda()
    tol = 1e-5 if dtype == torch.float32 else (2e-3 if dtype == torch.float16 else 1.6e-2)
    for name, code in (("First", capi.RT_POOL_FIRST), ("Last", capi.RT_POOL_LAST), ("Mean", capi.RT_POOL_MEAN),
                       ("Max", capi.RT_POOL_MAX)):
        for toks, toks_d in ((None, None), (tokens, tok_d)):
            out = torch.full((4, width), float("nan"), dtype=dtype, device="cuda")
            capi.sequence_pool(hidden, sb_d, code, out, toks_d)
            torch.cuda.synchronize()
            want = ol.sequence_pool(hidden.float().cpu(), sb.tolist(), name, seq_tokens=toks)
            err = (out.float().cpu() - want).abs().max().item()
            assert err <= tol, (name, toks is not None, err)
            if name in ("First", "Last", "Max"):               # selections: the stored values themselves
                assert torch.equal(out.float().cpu(), want)
    with pytest.raises(capi.RaptorError):
        capi.sequence_pool(hidden, sb_d, 7, out)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_pooler_dense_tanh_matches_oracle(capi, dtype):
    say("pooler", dtype)
    g = torch.Generator().manual_seed(10)
    for batch, d_in, d_out in ((16, 768, 768), (3, 200, 50), (1, 8, 1)):
        x = torch.randn(batch, d_in, generator=g).to(dtype).cuda()
        w = (torch.randn(d_in, d_out, generator=g) * 0.05).to(dtype).cuda()
        b = torch.randn(d_out, generator=g).to(dtype).cuda()
        out = torch.full((batch, d_out), float("nan"), dtype=dtype, device="cuda")
        capi.pooler_dense_tanh(x, w.t().contiguous(), b, out)
        torch.cuda.synchronize()
        want = ol.pooler(x.float().cpu(), w.float().cpu(), b.float().cpu())
        tol = 1e-5 if dtype == torch.float32 else (1e-3 if dtype == torch.float16 else 8e-3)
        assert (out.float().cpu() - want).abs().max().item() <= tol


@pytest.mark.parametrize("retune", [0, 3, 8])
def test_gemm_retuning_for_new_token_counts_keeps_results(capi, retune):
    """A new M of a kind already tuned times `retune` of the kind's best solutions (or none): same results."""
    say("gemm retune", retune)
    g = torch.Generator().manual_seed(6)
    a = torch.randn(1000, 256, generator=g).half().cuda()
    bt = (torch.randn(384, 256, generator=g) * 0.05).half().cuda()
    bias = torch.randn(384, generator=g).half().cuda()
    want = ol.bias_gelu(a.double().cpu() @ bt.double().cpu().t(), bias.cpu())
    gemm = capi.Gemm()
    gemm.set_retuning(retune)
    for rows in (1000, 640, 64, 1):
        c = torch.empty(rows, 384, dtype=torch.float16, device="cuda")
        for _ in range(2):                                  # the second call takes the cached plan
            gemm.bt(a[:rows].contiguous(), bt, c, bias=bias, epilogue=capi.RT_EPILOGUE_BIAS_GELU)
            torch.cuda.synchronize()
            assert (c.double().cpu() - want[:rows]).abs().max().item() <= 2e-2
    gemm.close()


@pytest.mark.parametrize("table_dtype,out_dtype,hidden", [
    (torch.float32, torch.float16, 768), (torch.float32, torch.bfloat16, 1024), (torch.float16, torch.float16, 768),
    (torch.float32, torch.float32, 1536), (torch.float32, torch.float16, 200)])
def test_embed_layernorm_matches_oracle(capi, table_dtype, out_dtype, hidden):
    say("embed", table_dtype, out_dtype, hidden)
    g = torch.Generator().manual_seed(3)
    vocab, max_pos, types, t = 1000, 4096, 2, 1000 + 37
    mk = lambda *shape: torch.randn(*shape, generator=g).to(table_dtype)
    word, pos, typ, gamma, beta = mk(vocab, hidden), mk(max_pos, hidden), mk(types, hidden), mk(hidden), mk(hidden)
    ids = torch.randint(0, vocab, (t,), generator=g, dtype=torch.int32)
    pids = torch.randint(0, max_pos, (t,), generator=g, dtype=torch.int32)
    tids = torch.randint(0, types, (t,), generator=g, dtype=torch.int32)
    ids[0], ids[1], pids[2] = -5, vocab + 9, max_pos          # outside their tables: clamped to the nearest row
    out = torch.empty(t, hidden, dtype=out_dtype, device="cuda")
    capi.embed_layernorm(ids.cuda(), pids.cuda(), tids.cuda(), word.cuda(), pos.cuda(), typ.cuda(), gamma.cuda(),
                         beta.cuda(), out)
    torch.cuda.synchronize()
    want = ol.embeddings_layernorm(ids.clamp(0, vocab - 1), pids.clamp(0, max_pos - 1), tids, word, pos, typ, gamma, beta)
    assert lh.excess(out, want, out_dtype, k=1.0) <= 0
    empty = torch.empty(0, hidden, dtype=out_dtype, device="cuda")
    z = torch.empty(0, dtype=torch.int32, device="cuda")
    capi.embed_layernorm(z, z, z, word.cuda(), pos.cuda(), typ.cuda(), gamma.cuda(), beta.cuda(), empty)
    with pytest.raises(capi.RaptorError):
        capi.embed_layernorm(ids.cuda(), pids.cuda(), tids.cuda(), word.cuda()[:, :-4].contiguous(), pos.cuda(), typ.cuda(),
                             gamma.cuda(), beta.cuda(), torch.empty(t, hidden - 4, dtype=out_dtype, device="cuda"))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_gemm_bias_gelu_epilogue_matches_oracle(capi, dtype):
    """The fused epilogue against the oracle's bias + tanh GELU applied to an fp32 product, and against
    the library's own two-kernel path (GEMM, then bias_gelu)."""
    say("gemm epilogue", dtype)
    g = torch.Generator().manual_seed(1)
    gemm = capi.Gemm()
    for m, n, k in [(832, 3072, 768), (64, 1024, 256), (1, 768, 768)]:
        a = torch.randn(m, k, generator=g).to(dtype).cuda()
        b = (torch.randn(k, n, generator=g) * 0.05).to(dtype).cuda()
        bias = torch.randn(n, generator=g).to(dtype).cuda()
        fused = torch.empty(m, n, dtype=dtype, device="cuda")
        gemm.bias_act(a, b, bias, fused)
        plain = torch.empty(m, n, dtype=dtype, device="cuda")
        gemm.bias_act(a, b, bias, plain, capi.RT_EPILOGUE_BIAS)
        two = torch.empty(m, n, dtype=dtype, device="cuda")
        gemm(a, b, two)
        capi.bias_gelu(two, bias)
        torch.cuda.synchronize()
        prod = a.double().cpu() @ b.double().cpu()
        want = ol.bias_gelu(prod, bias.cpu())
        assert lh.excess(fused, want, dtype, k=1.0) <= 0
        assert lh.excess(two, want, dtype, k=2.0) <= 0          # the two-kernel path rounds the product to T first
        assert lh.excess(plain, prod + bias.double().cpu(), dtype, k=1.0) <= 0
    with pytest.raises(capi.RaptorError):
        gemm.bias_act(a, b, bias, fused, epilogue=7)
    gemm.close()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_gemm_transposed_weights_match_plain(capi, dtype):
    """rt_gemm_bt (weights kept as [N, K]) against an fp64 product and against rt_gemm / rt_gemm_bias_act on the
    [K, N] copy of the same weights, for each epilogue."""
    say("gemm bt", dtype)
    g = torch.Generator().manual_seed(4)
    gemm = capi.Gemm()
    for m, n, k in [(832, 2304, 768), (200, 768, 3072), (1, 512, 256)]:
        a = torch.randn(m, k, generator=g).to(dtype).cuda()
        bt = (torch.randn(n, k, generator=g) * 0.05).to(dtype).cuda()
        b = bt.t().contiguous()
        bias = torch.randn(n, generator=g).to(dtype).cuda()
        prod = a.double().cpu() @ bt.double().cpu().t()
        # fp32: products of 768 to 3072 terms, summed in another order than the fp64 reference
        within = (lambda x, y: (x.double().cpu() - y.double().cpu()).abs().max().item() <= 2e-3) if dtype == torch.float32 \
            else (lambda x, y: lh.excess(x, y, dtype, k=1.0) <= 0)
        got, ref = (torch.empty(m, n, dtype=dtype, device="cuda") for _ in range(2))
        gemm.bt(a, bt, got)
        gemm(a, b, ref)
        torch.cuda.synchronize()
        assert within(got, prod)
        assert within(got, ref)
        if dtype == torch.float32:
            continue                                        # the library has no fp32 bias epilogue for every shape
        for ep, want in ((capi.RT_EPILOGUE_BIAS, prod + bias.double().cpu()),
                         (capi.RT_EPILOGUE_BIAS_GELU, ol.bias_gelu(prod, bias.cpu()))):
            gemm.bt(a, bt, got, bias=bias, epilogue=ep)
            gemm.bias_act(a, b, bias, ref, ep)
            torch.cuda.synchronize()
            assert within(got, want)
            assert within(got, ref)
    with pytest.raises(capi.RaptorError):
        gemm.bt(a, bt, got, bias=None, epilogue=capi.RT_EPILOGUE_BIAS)
    gemm.close()


@pytest.mark.parametrize("dtype,hidden,heads,ffn,n_wg", [
    (torch.float16, 768, 12, 3072, 0), (torch.bfloat16, 1024, 16, 4096, 64), (torch.float16, 768, 12, 3072, 160)])
def test_encoder_layer_matches_oracle(capi, dtype, hidden, heads, ffn, n_wg):
    say("layer", dtype, hidden, n_wg)
    pkg = graft.load_package()
    out, want = lh.run_layer_case_tensors(pkg, [1024, 320, 832], hidden, heads, ffn, dtype, seed=0, n_wg=n_wg)
    say("  layer err", (out - want).abs().max().item())
    # a whole layer: the rounding of its intermediate tensors adds to the output's own, hence two ulp
    assert lh.excess(out, want, dtype, k=2.0) <= 0


def test_pipeline_on_device(capi):
    say("pipeline device")
    heads, layers = 4, 3
    pipe = capi.Pipeline(layers, heads, device=0)
    for lens in ([768, 1024], [2048], [832, 64, 1280]):
        sb = capi.seq_prefix_blocks(lens)
        pipe.publish(sb)
        for layer in range(layers):
            idx_p, pos_p, ph, wait = pipe.acquire(layer)
            n_idx, n_pos = capi.to_index_size(sb, ph)
            torch.cuda.current_stream().synchronize()
            got_idx = torch.empty(n_idx, dtype=torch.int32, device="cuda")
            got_pos = torch.empty(n_pos, dtype=torch.int32, device="cuda")
            import ctypes
            from ctypes import c_void_p
            hip = ctypes.CDLL("libamdhip64.so")
            assert hip.hipMemcpy(c_void_p(got_idx.data_ptr()), c_void_p(idx_p), n_idx * 4, 3) == 0
            assert hip.hipMemcpy(c_void_p(got_pos.data_ptr()), c_void_p(pos_p), n_pos * 4, 3) == 0
            want_idx, want_pos = capi.build_to_index(sb, ph, seed=layer)
            assert np.array_equal(got_idx.cpu().numpy(), want_idx) and np.array_equal(got_pos.cpu().numpy(), want_pos)
            pipe.release(layer)
    pipe.close()


def test_pipeline_keeps_a_slot_until_late_readers_finish(capi):
    """A layer launched AGAIN after the batch's last layer was released (a second, partial pass without a new
    publish) is a reader no closing record covered when the per-batch event was tied to the last layer alone: two
    publishes later the worker would overwrite the slot while that reader still waits on the GPU.  The reader here
    is a device copy of the slot queued behind a sleeping kernel; it must see the batch it acquired."""
    say("pipeline late reader")
    import ctypes
    from ctypes import c_void_p
    hip = ctypes.CDLL("libamdhip64.so")
    heads, layers = 2, 3
    pipe = capi.Pipeline(layers, heads, device=0)
    sb_a, sb_b, sb_c = (capi.seq_prefix_blocks(l) for l in ([832, 1024], [1280], [1024, 768]))
    pipe.publish(sb_a)
    for layer in range(layers):
        pipe.acquire(layer)
        pipe.release(layer)                                  # the last layer closes the batch
    idx_p, pos_p, ph, _ = pipe.acquire(0)                    # second, partial pass: layer 0 only
    n_idx, n_pos = capi.to_index_size(sb_a, ph)
    seen = torch.zeros(n_idx, dtype=torch.int32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    torch.cuda._sleep(int(2.0e8))                            # about 0.1 s: the reader is queued, not running
    assert hip.hipMemcpyAsync(c_void_p(seen.data_ptr()), c_void_p(idx_p), n_idx * 4, 3, c_void_p(stream)) == 0
    pipe.release(0)
    pipe.publish(sb_b)
    pipe.acquire(0)
    pipe.release(0)
    pipe.publish(sb_c)                                       # the workers now rebuild the slots batch A used
    idx_c, _, _, _ = pipe.acquire(0)
    assert idx_c == idx_p                                    # batch C sits in the buffer batch A used
    torch.cuda.synchronize()
    want_idx, _ = capi.build_to_index(sb_a, ph, seed=0)
    assert np.array_equal(seen.cpu().numpy(), want_idx)
    pipe.close()


def test_attention_random_geometries(capi):
    """Twenty seeded draws of batch geometry (1 to 7 sequences of 1 to 40 blocks, so sparse and full-attention
    sequences mix), head count, dtype, plan mode, schedule (the kernel's own / a work plan of random size) and
    padding, each against the oracle."""
    say("attention random geometries")
    rng = np.random.default_rng(2024)
    for case in range(20):
        batch = int(rng.integers(1, 8))
        lens = [64 * int(rng.integers(1, 41)) for _ in range(batch)]
        heads = int(rng.choice([1, 2, 3, 5]))
        dtype = [torch.float16, torch.bfloat16, torch.float32][int(rng.integers(0, 3))]
        mode = capi.RT_PLAN_REFERENCE if rng.integers(0, 4) == 0 else None
        n_wg = int(rng.integers(1, 60)) if rng.integers(0, 2) else 0
        padded = bool(rng.integers(0, 2))
        wide = bool(rng.integers(0, 2))                    # padding of whole blocks, not only of a block's tail
        seq_tokens = None
        if padded:
            seq_tokens = [int(rng.integers(1, n + 1)) if wide else n - int(rng.integers(0, 64)) for n in lens]
        say("  case", case, lens, heads, dtype, mode, n_wg, seq_tokens)
        t = sum(lens)
        g = torch.Generator().manual_seed(1000 + case)
        q, k, v = (torch.randn(t, heads, 64, generator=g).to(dtype).cuda() for _ in range(3))
        out, ref = lh.run_attention(capi, q, k, v, lens, heads, seed=case, mode=mode, n_wg=n_wg, seq_tokens=seq_tokens)
        rows = torch.ones(t, dtype=torch.bool)
        if padded:                                         # padded query rows are computed but not specified
            start = 0
            for n, real in zip(lens, seq_tokens):
                rows[start + real:start + n] = False
                start += n
        assert torch.isfinite(out.float()).all(), case
        assert lh.excess(out[rows.cuda()], ref[rows], dtype, k=1.0) <= 0, case
