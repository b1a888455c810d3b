"""rt_bs_attention_fwd_no_alloc (queue counters in a static device array, no device allocation) against
rt_bs_attention_fwd_masked on the same inputs: the two run the same kernel over the same plan, so the outputs
must be the same bits.  Two calls in a row share the static counters, the second on a smaller batch; a third
goes back to the larger one; both also match the CPU oracle.  Sizes beyond the stated limits are refused."""
import pytest
import torch

import __graft_entry__ as graft
from oracle import attention as oa
from tests import layer_harness as lh

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def capi():
    pkg = graft.load_package()
    pkg.capi.lib()
    assert torch.cuda.is_available()
    return pkg.capi


def _case(capi, dtype, seq_lens, heads, seed, padded):
    t, dm = sum(seq_lens), heads * 64
    g = torch.Generator().manual_seed(seed)
    qkv = torch.randn(t, 3 * dm, generator=g).to(dtype).cuda()
    bias = (torch.randn(3 * dm, generator=g) * 0.5).to(dtype).cuda()
    sb, idx, pos, ph, sb_d, idx_d, pos_d = lh.device_plan(capi, seq_lens, heads, seed, None)
    seq_tokens = [n - 9 for n in seq_lens] if padded else None
    tok_d = None if seq_tokens is None else torch.tensor(seq_tokens, dtype=torch.int32).cuda()
    q, k, vt = (torch.full((t * dm,), float("nan"), dtype=dtype, device="cuda") for _ in range(3))
    capi.qkv_bias_split(qkv, bias, q, k, vt, sb_d, heads, capi.Q_SCALE)
    x = qkv.float().cpu() + bias.float().cpu()
    qs = (x[:, :dm] * capi.Q_SCALE).to(dtype).view(t, heads, 64)
    kk, vv = (x[:, i * dm:(i + 1) * dm].to(dtype).view(t, heads, 64) for i in (1, 2))
    ref = oa.csr_attention(qs, kk, vv, sb.tolist(), idx, pos, ph, scale=1.0 / lh.LOG2E, seq_tokens=seq_tokens)
    return dict(t=t, dm=dm, q=q, k=k, vt=vt, sb_d=sb_d, idx_d=idx_d, pos_d=pos_d, ph=ph, tok_d=tok_d, heads=heads,
                ref=ref, dtype=dtype)


def _run(capi, c, no_alloc):
    out = torch.full((c["t"], c["dm"]), float("nan"), dtype=c["dtype"], device="cuda")
    if no_alloc:
        capi.bs_attention_fwd_no_alloc(c["q"], c["k"], c["vt"], out, c["sb_d"], c["heads"], c["idx_d"], c["pos_d"],
                                       c["ph"], c["tok_d"])
    else:
        capi.bs_attention_fwd(c["q"], c["k"], c["vt"], out, c["sb_d"], c["heads"], c["idx_d"], c["pos_d"], c["ph"],
                              None, None, c["tok_d"])
    return out


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_no_alloc_entry_point_matches_allocating_one(capi, dtype):
    print("no_alloc", dtype, flush=True)
    large = _case(capi, dtype, [64 * 21, 64 * 3, 64 * 40, 64, 64 * 12], 6, 11, padded=False)
    small = _case(capi, dtype, [64 * 14, 64 * 2], 3, 12, padded=True)
    want = {id(c): _run(capi, c, no_alloc=False) for c in (large, small)}
    torch.cuda.synchronize()
    # back to back on one stream, nothing in between: the second call finds the first call's counters
    got = [(c, _run(capi, c, no_alloc=True)) for c in (large, small, large)]
    torch.cuda.synchronize()
    for c, out in got:
        assert torch.isfinite(out).all()
        assert torch.equal(out, want[id(c)])
        assert (out.float().cpu() - c["ref"]).abs().max().item() <= 2e-2


def test_no_alloc_entry_point_refuses_sizes_beyond_its_limits(capi):
    print("no_alloc limits", flush=True)
    z = torch.zeros(64, 64, dtype=torch.float16, device="cuda")
    i32 = torch.zeros(8, dtype=torch.int32, device="cuda")
    L, vp = capi.lib(), capi._dp
    args = lambda batch, blocks: (vp(z), vp(z), vp(z), vp(z), vp(i32), None, batch, blocks, 1, vp(i32), vp(i32), 1,
                                  capi.RT_F16, None)
    assert L.rt_bs_attention_fwd_no_alloc(*args(1025, 1025)) == capi.RT_EINVAL
    assert b"at most" in L.rt_last_error_string()
    assert L.rt_bs_attention_fwd_no_alloc(*args(1, 4097)) == capi.RT_EINVAL
    assert L.rt_bs_attention_fwd_no_alloc(*args(0, 1)) == capi.RT_EINVAL
