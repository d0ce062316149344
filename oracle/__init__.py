"""CPU oracle for the chunk-scheduled compute path.  TEST INFRASTRUCTURE ONLY.

A plain numpy / torch-CPU restatement of what the reference's device code
computes, used as the checker by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py.  Nothing under syncopate_amd/ imports it, and it
is never the thing that is shipped or measured as the product.

Pinning of each function (what fixes it besides its own formula):

* visit_order.gemm_tile_visits / get_pid_mn — the literal tile orders the
  reference's tests hold (tests/computation/transform/test_transform_pass.py:253-291),
  plus brute-force properties (every tile exactly once, waves contiguous).
* visit_order.attn_tile_work — the per-tile tuples the reference's own GENERATED
  dispatch text gives when it is evaluated tile by tile (its AnnotationTransformer
  applied to its annotated attention example; tests/golden/attn_dispatch_cases.json,
  written by tests/golden/make_attn_dispatch_fixtures.py), a hand-evaluated literal
  of get_pid_range (attn/template.py:39-44) that a swap of z, h or q fails, and
  brute-force coverage: every (z, h, q block, kv block) exactly once.
* numerics.ring_reduce — closed form on exactly representable inputs, and
  torch's own bf16/fp16 addition (a library routine) for the per-add rounding.
* numerics.gemm_fp32 — torch.matmul in fp32 (library routine).
* numerics.chunked_attention — reduces to
  torch.nn.functional.scaled_dot_product_attention over the gathered K/V
  (library routine) for every chunking and arrival order; lse against
  torch.logsumexp.
"""
