"""Bad tensors are refused on the host, before any launch: a host tensor, a strided view, a wrong dtype or too few
elements would make a kernel read memory it must not.  No GPU is needed: nothing here reaches a kernel."""
import importlib

import numpy as np
import pytest
import torch

import __graft_entry__ as graft


@pytest.fixture(scope="module")
def capi():
    pkg = graft.load_package()
    pkg.capi.lib()
    return pkg.capi


@pytest.fixture(scope="module")
def kernels():
    graft.load_package()
    return importlib.import_module("raptor_t_amd.modeling_bert").cxx.kernels


def test_capi_refuses_host_tensors_and_wrong_dtypes(capi):
    heads, t = 2, 128
    h = lambda *shape: torch.zeros(*shape, dtype=torch.float16)
    i32 = lambda n: torch.zeros(n, dtype=torch.int32)
    with pytest.raises(ValueError, match="GPU tensor"):
        capi.bias_gelu(h(4, 8), h(8))
    with pytest.raises(ValueError, match="GPU tensor"):
        capi.bias_residual_layernorm(h(4, 8), h(4, 8), h(8), h(8), h(8), 1e-5)
    with pytest.raises(ValueError, match="GPU tensor"):
        capi.qkv_bias_split(h(t, 3 * heads * 64), h(3 * heads * 64), h(t * heads * 64), h(t * heads * 64), h(t * heads * 64),
                            i32(2), heads, 1.0)
    with pytest.raises(ValueError):
        capi.qkv_bias_split(h(t, 3 * heads * 64 - 8), h(3 * heads * 64), None, h(1), h(1), i32(2), heads, 1.0)
    with pytest.raises(ValueError, match="GPU tensor"):
        capi.bs_attention_fwd(h(t * heads * 64), h(t * heads * 64), h(t * heads * 64), h(t, heads * 64), i32(2), heads,
                              i32(4), i32(2 * heads + 1), heads)
    with pytest.raises(ValueError, match="GPU tensor"):
        capi.bs_attention_fwd_no_alloc(h(t * heads * 64), h(t * heads * 64), h(t * heads * 64), h(t, heads * 64), i32(2),
                                       heads, i32(4), i32(2 * heads + 1), heads)
    with pytest.raises(ValueError):
        capi.bs_attention_fwd(h(1), h(1), h(1), h(t, heads * 64 + 8), i32(2), heads, i32(4), i32(5), heads)
    with pytest.raises(ValueError):
        capi.bs_attention_fwd(h(1), h(1), h(1), h(t, heads * 64), i32(2), heads, i32(4), i32(5), 3)


def test_capi_pointer_helper_checks_each_property(capi):
    class Fake:                                             # a GPU tensor as far as the helper can tell
        def __init__(self, dtype=torch.float16, n=16, contiguous=True):
            self.is_cuda, self.dtype, self._n, self._c, self.device = True, dtype, n, contiguous, "cuda:0"

        def is_contiguous(self):
            return self._c

        def numel(self):
            return self._n

        def data_ptr(self):
            return 4096

    assert capi._dp(None).value in (0, None)
    assert capi._dp(Fake()).value == 4096
    with pytest.raises(ValueError, match="contiguous"):
        capi._dp(Fake(contiguous=False))
    with pytest.raises(ValueError, match="dtype"):
        capi._dp(Fake(dtype=torch.float32), torch.float16)
    with pytest.raises(ValueError, match="dtype"):
        capi._ip(Fake(dtype=torch.int64))
    with pytest.raises(ValueError, match="holds 16 elements"):
        capi._dp(Fake(), torch.float16, 17)
    assert capi._ip(Fake(dtype=torch.int32), 16).value == 4096


def test_partition_check_accepts_lpt_plans_and_names_what_is_wrong(capi):
    sb = capi.seq_prefix_blocks([832, 64, 1024])
    heads, n_wg = 3, 7
    pos, ids = capi.partition_lpt(sb, heads, n_wg)
    nb = int(sb[-1])
    capi.check_partition(pos, ids, nb, heads)
    bad = ids.copy()
    bad[5] = nb * heads                                     # one past the last unit
    with pytest.raises(capi.RaptorError, match="outside"):
        capi.check_partition(pos, bad, nb, heads)
    bad = ids.copy()
    bad[5] = -1
    with pytest.raises(capi.RaptorError, match="outside"):
        capi.check_partition(pos, bad, nb, heads)
    bad = ids.copy()
    bad[3] = bad[4]
    with pytest.raises(capi.RaptorError, match="twice"):
        capi.check_partition(pos, bad, nb, heads)
    p2 = pos.copy()
    p2[-1] -= 1
    with pytest.raises(capi.RaptorError, match="from_pos"):
        capi.check_partition(p2, ids, nb, heads)
    p2 = pos.copy()
    p2[2], p2[3] = pos[3] + 1, pos[2]
    with pytest.raises(capi.RaptorError, match="decreases"):
        capi.check_partition(p2, ids, nb, heads)
    with pytest.raises(ValueError):
        capi.check_partition(pos, ids[:-1], nb, heads)


def test_to_index_check_accepts_built_indices_and_names_what_is_wrong(capi):
    sb = capi.seq_prefix_blocks([832, 64, 1024, 320])
    for plan_heads, mode in ((3, capi.RT_PLAN_HF), (1, capi.RT_PLAN_REFERENCE)):
        idx, pos = capi.build_to_index(sb, plan_heads, mode=mode, seed=4)
        capi.check_to_index(idx, pos, sb, plan_heads)
        row = 2                                                 # block 2 of the 13-block sequence: a sparse row
        bad = idx.copy()
        bad[pos[row] + 1] = 13                                  # one past the sequence's last block
        with pytest.raises(capi.RaptorError, match="names block 13"):
            capi.check_to_index(bad, pos, sb, plan_heads)
        bad = idx.copy()
        bad[pos[13]] = 1                                        # the one-block sequence has only block 0
        with pytest.raises(capi.RaptorError, match="names block 1"):
            capi.check_to_index(bad, pos, sb, plan_heads)
        bad = idx.copy()
        bad[pos[row]] = -1
        with pytest.raises(capi.RaptorError, match="names block -1"):
            capi.check_to_index(bad, pos, sb, plan_heads)
        p2 = pos.copy()
        p2[row + 1] = p2[row]
        with pytest.raises(capi.RaptorError, match="empty"):
            capi.check_to_index(idx, p2, sb, plan_heads)
        p2 = pos.copy()
        p2[-1] += 5
        with pytest.raises(capi.RaptorError, match="to_idx holds"):
            capi.check_to_index(idx, p2, sb, plan_heads)
        p2 = pos.copy()
        p2[0] = 1
        with pytest.raises(capi.RaptorError, match="start at 0"):
            capi.check_to_index(idx, p2, sb, plan_heads)
        with pytest.raises(ValueError):
            capi.check_to_index(idx, pos[:-1], sb, plan_heads)


def test_layer_launchers_refuse_bad_tensors(kernels):
    """The shims under the reference's kernel names (layers/kernels/kernel.h) check device, layout, dtype and sizes
    before they time or launch anything; on this machine every tensor is a host tensor, so each call must raise."""
    h = lambda *shape: torch.zeros(*shape, dtype=torch.float16)
    i32 = lambda n: torch.zeros(n, dtype=torch.int32)
    heads, nb = 2, 2
    t = nb * 64
    with pytest.raises(ValueError, match="GPU tensor"):
        kernels.add_bias_act_kernel(h(8), h(4, 8), 4, 8)
    with pytest.raises(ValueError, match="GPU tensor"):
        kernels.add_bias_and_layernorm_kernel(h(4, 8), h(4, 8), h(8), 4, 8, 1e-5, h(8), h(8))
    with pytest.raises(ValueError, match="GPU tensor"):
        kernels.add_bias_and_transpose_kernel(h(3 * heads * 64), h(t, 3 * heads * 64), h(t * heads * 64), h(t * heads * 64),
                                              h(t * heads * 64), i32(2), 1, heads, nb)
    with pytest.raises(ValueError, match="head size"):
        kernels.add_bias_and_transpose_kernel(h(3 * heads * 32), h(t, 3 * heads * 32), h(1), h(1), h(1), i32(2), 1, heads, nb, 32)
    with pytest.raises(ValueError, match="GPU"):
        kernels.sparse_attention(h(t * heads * 64), h(t * heads * 64), h(t * heads * 64), h(t, heads * 64), 1, i32(2),
                                 i32(nb * heads), i32(3), i32(4), i32(heads * nb + 1), heads, 2, nb, heads)
    with pytest.raises(ValueError, match="bad"):
        kernels.add_bias_act_kernel(h(8), h(4, 8), -1, 8)
