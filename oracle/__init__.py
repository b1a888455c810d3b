"""CPU oracle for the block-sparse (BigBird-pattern) encoder layer.

TEST INFRASTRUCTURE ONLY.  Nothing under this directory is part of the shipped
path: it may be imported by `tests/`, by `__graft_entry__.smoke()` and by the
`cpu_baseline` leg of `bench.py`, always as the checker and never as the thing
that is measured or shipped.  The product (the HIP library and the layer API on
top of it) never imports it and has no CPU fallback.

Every function restates, in numpy / PyTorch-CPU fp32 (fp64 for the brute force
checks), the algorithm of the reference path and cites the reference file:line
it follows.  What pins each function:

  plans.rand_attn_max_plan, plans.rand_attn_with_head,
  plans.single_block_row_attention, plans.rand_attn_plan
        golden vectors written by the installed HuggingFace `transformers`
        BigBird code (tests/golden/hf_plans.json) plus structural invariants.
  metadata.to_index_from_rand_attn, metadata.reference_to_index
        layers/test.cpp golden CSR (n=64), closed form sum(10n-18), legality.
  metadata.lpt_partition, metadata.data_metainfo
        layers/test.cpp golden plan (160 CTAs, 12 heads) -- bit exact.
  attention.bigbird_5part
        golden output of the installed HuggingFace BigBird block-sparse
        attention (tests/golden/hf_attention.npz) and the brute force below.
  attention.multiset_attention
        textbook softmax in fp64 with a log(count) multiplicity mask; special
        cases that reduce to torch SDPA.
  layer.*  torch.nn.functional.layer_norm / gelu(approximate="tanh") / matmul.

No function here is "parity unpinned".
"""
