"""Shared helpers of the GPU parity tests and of `__graft_entry__.smoke()`: drive the
C-ABI through `raptor_t_amd.capi` and compare with the CPU oracle.  Not collected by
pytest (no test_ prefix)."""
import math

import numpy as np
import torch

from oracle import attention as oa
from oracle import layer as ol
from oracle import metadata as md

LOG2E = 1.4426950408889634
SLOT_PERM = [0, 1, 2, 3, 8, 9, 10, 11, 4, 5, 6, 7, 12, 13, 14, 15]


MANTISSA_BITS = {torch.float16: 10, torch.bfloat16: 7}


def ulp(y, dtype):
    """Spacing of `dtype`'s numbers at |y|, per element (y: fp32/fp64 tensor)."""
    e = torch.floor(torch.log2(y.abs().double().clamp_min(2.0 ** -14)))
    return torch.exp2(e - MANTISSA_BITS[dtype])


def excess(got, want, dtype, k=1.0):
    """Largest amount by which |got - want| goes over the per-element bound; <= 0 means inside it everywhere.
    The bound is 2e-2 for fp16 and bf16, widened to k ulp of the output type where the expected value is so
    large that one ulp is more than that (bf16: |y| >= 4), and 1e-4 for fp32."""
    got, want = got.detach().double().cpu(), want.detach().double().cpu()
    if dtype == torch.float32:
        bound = torch.full_like(want, 1e-4)
    else:
        bound = torch.maximum(torch.full_like(want, 2e-2), k * ulp(want, dtype))
    return ((got - want).abs() - bound).max().item()


def outliers(got, want, dtype, k=1.0):
    """(share of elements outside excess()'s per-element bound, largest error in ulp of its row's largest expected
    value, rms error).  For outputs that went through several tensors stored in `dtype`: a rounding of a LayerNorm
    input of magnitude 4 to 8 that falls the other way moves an output of any size by one ulp of THAT magnitude, so
    isolated elements leave the per-element bound; what a test can still demand is that they stay isolated, that
    none is further off than the ulp of the row's largest values, and that the rms error stays at rounding level."""
    got, want = got.detach().double().cpu(), want.detach().double().cpu()
    err = (got - want).abs()
    bound = torch.maximum(torch.full_like(want, 2e-2), k * ulp(want, dtype))
    row_ulp = ulp(want.abs().amax(dim=-1, keepdim=True), dtype)
    return (err > bound).double().mean().item(), (err / row_ulp).max().item(), err.pow(2).mean().sqrt().item()


def check_stack_output(got, want, dtype):
    """Bound for the output of a few layers.  fp16 and fp32: excess() with one ulp.  bf16, against an oracle that
    stores its tensors in bf16 too: at most 1 element in 10 000 outside max(2e-2, 2 ulp(|y|)), none further off than
    three ulp of its row's largest value, rms error at most 4e-3.  Measured on two layers: 3e-5, 2.0, 2.8e-3; the
    largest error is a whole number of ulp, and which GEMM kernel the library picks on a box moves single roundings,
    so the bound leaves one ulp above what was seen."""
    if dtype != torch.bfloat16:
        over = excess(got, want, dtype, k=1.0)
        assert over <= 0, over
        return
    share, worst, rms = outliers(got, want, dtype, k=2.0)
    assert share <= 1e-4 and worst <= 3.0 and rms <= 4e-3, (share, worst, rms)


def slot_tokens():
    return torch.tensor([(p & ~15) | SLOT_PERM[p & 15] for p in range(64)], dtype=torch.long)


def pack_heads(x, seq_blocks, transpose_v=False):
    """Token-major [T, H, d] -> the head-major packed layout as a flat tensor (torch statement
    of the layout documented in include/raptor_t_hip.h): per (sequence, head, block) a 64x64
    tile [row][col] (row = token, col = d; for V row = d, col = slot) stored as fragments
    [row>>5][col>>4][(col>>3)&1][row&31][col&7]."""
    t, heads, d = x.shape
    parts = []
    st = slot_tokens().to(x.device)
    for s in range(len(seq_blocks) - 1):
        n = int(seq_blocks[s + 1] - seq_blocks[s])
        blk = x[int(seq_blocks[s]) * 64: int(seq_blocks[s + 1]) * 64].view(n, 64, heads, d).permute(2, 0, 1, 3)
        if transpose_v:
            blk = blk[:, :, st, :].transpose(2, 3)          # [H, n, d, slot]
        blk = blk.reshape(heads, n, 2, 32, 4, 2, 8).permute(0, 1, 2, 4, 5, 3, 6)
        parts.append(blk.contiguous().view(-1))
    return torch.cat(parts)


def device_plan(capi, seq_lens, heads, seed=0, mode=None, plan_heads=None, device="cuda", max_pos=4096):
    sb = capi.seq_prefix_blocks(seq_lens)
    mode = capi.RT_PLAN_HF if mode is None else mode
    ph = (1 if mode == capi.RT_PLAN_REFERENCE else heads) if plan_heads is None else plan_heads
    idx, pos = capi.build_to_index(sb, ph, mode=mode, seed=seed, max_pos=max_pos)
    dev = lambda a: torch.from_numpy(a).to(device)
    return sb, idx, pos, ph, dev(sb), dev(idx), dev(pos)


def run_attention(capi, q, k, v, seq_lens, heads, seed=0, mode=None, n_wg=0, seq_tokens=None, max_pos=4096):
    """q, k, v: [T, H, 64] CUDA tensors (q unscaled).  Returns (gpu_out [T, H*64], oracle fp32).
    seq_tokens: true token count per sequence when its last block ends in padding."""
    sb, idx, pos, ph, sb_d, idx_d, pos_d = device_plan(capi, seq_lens, heads, seed, mode, max_pos=max_pos)
    qs = (q.float() * (LOG2E / 8.0)).to(q.dtype)          # the kernel's softmax is base 2
    qp, kp = pack_heads(qs, sb), pack_heads(k, sb)
    vp = pack_heads(v, sb, transpose_v=True)
    out = torch.full((q.shape[0], heads * 64), float("nan"), dtype=q.dtype, device=q.device)
    from_idx = from_pos = None
    if n_wg:
        fp, fi = capi.partition_lpt(sb, heads, n_wg)
        from_pos, from_idx = torch.from_numpy(fp).cuda(), torch.from_numpy(fi).cuda()
    tok_d = None if seq_tokens is None else torch.tensor(seq_tokens, dtype=torch.int32).cuda()
    capi.bs_attention_fwd(qp, kp, vp, out, sb_d, heads, idx_d, pos_d, ph, from_idx, from_pos, tok_d)
    torch.cuda.synchronize()
    ref = oa.csr_attention(qs.cpu(), k.cpu(), v.cpu(), sb.tolist(), idx, pos, ph, scale=1.0 / LOG2E,
                           seq_tokens=seq_tokens)
    return out, ref


def run_layer_case(pkg, seq_lens, hidden, heads, ffn, dtype, seed=0, eps=1e-5, n_wg=0):
    """One encoder layer through the C-ABI on cuda:0 against the oracle; returns max abs error."""
    out, want = run_layer_case_tensors(pkg, seq_lens, hidden, heads, ffn, dtype, seed, eps, n_wg)
    return (out - want).abs().max().item()


def run_layer_case_tensors(pkg, seq_lens, hidden, heads, ffn, dtype, seed=0, eps=1e-5, n_wg=0):
    """The same case; returns (layer output as fp32 on the host, the oracle's output)."""
    capi = pkg.capi
    g = torch.Generator().manual_seed(seed)
    w32 = ol.random_layer_weights(hidden, ffn, g)
    t = sum(seq_lens)
    x32 = torch.randn(t, hidden, generator=g)
    w = {k_: v_.to(dtype).cuda() for k_, v_ in w32.items()}
    x = x32.to(dtype).cuda()
    sb, idx, pos, ph, sb_d, idx_d, pos_d = device_plan(capi, seq_lens, heads, seed)
    gemm = capi.Gemm()
    new = lambda *shape: torch.empty(*shape, dtype=dtype, device="cuda")
    qkv, q, k, vt = new(t, 3 * hidden), new(t * hidden), new(t * hidden), new(t * hidden)
    ctx, attn, inter, out = new(t, hidden), new(t, hidden), new(t, ffn), new(t, hidden)
    from_idx = from_pos = None
    if n_wg:
        fp, fi = capi.partition_lpt(sb, heads, n_wg)
        from_pos, from_idx = torch.from_numpy(fp).cuda(), torch.from_numpy(fi).cuda()
    gemm(x, w["qkv_weight"], qkv)
    capi.qkv_bias_split(qkv, w["qkv_bias"], q, k, vt, sb_d, heads, LOG2E / math.sqrt(hidden // heads))
    capi.bs_attention_fwd(q, k, vt, ctx, sb_d, heads, idx_d, pos_d, ph, from_idx, from_pos)
    gemm(ctx, w["attn_out_weight"], attn)
    capi.bias_residual_layernorm(attn, x, w["attn_out_bias"], w["attn_ln_weight"], w["attn_ln_bias"], eps)
    gemm(attn, w["inter_weight"], inter)
    capi.bias_gelu(inter, w["inter_bias"])
    gemm(inter, w["out_weight"], out)
    capi.bias_residual_layernorm(out, attn, w["out_bias"], w["out_ln_weight"], w["out_ln_bias"], eps)
    torch.cuda.synchronize()
    gemm.close()
    wr = {k_: v_.to(dtype).float() for k_, v_ in w32.items()}          # the oracle sees the rounded weights
    want = ol.encoder_layer(x32.to(dtype).float(), wr, heads, sb.tolist(), idx, pos, ph, eps)
    return out.float().cpu(), want
