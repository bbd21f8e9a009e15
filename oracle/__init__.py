"""CPU restatement of the reference's batch-invariant token-logprob path.

TEST INFRASTRUCTURE ONLY. Nothing under ``oracle/`` is part of the product: only ``tests/``,
``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline`` leg may import it, and only as
the checker. The product path (``skyrl-isoexec_amd/``) never imports it and has no CPU fallback.

What it restates, and from where (paths relative to the reference's
``skyrl/backends/skyrl_train/isoexec/``):

  logprobs.py  ops/logprobs/rowinv.py:136-245,547-570 (leaf exp-sum tree, Kahan, combine_order)
  norms.py     ops/norms/fused_outnorm.py:113-232, ops/norms/zero_centered_norm.py:36-37,
               runtimes/megatron/gdn_fla_shim.py:390-425
  mm.py        ops/moe/moe_batch_invariant.py:422-473 (what the aten mm override computes)
  gdn.py       ops/gdn/gdn_ops.py:74-170 (conv), :173-213 (l2norm), :261-315 (chunked fp32
               reference), :400-441 (recurrent scan semantics), :1197-1210 (gating)
  moe.py       ops/moe/moe_router_o2_kernel.py:369-397, ops/moe/moe_batched_experts.py:496-503,
               ops/moe/moe_batch_invariant.py:276-320

The arithmetic the reference runs on GPUs lives in third-party kernels that are not in its tree
(vLLM's FLA/batch-invariant/fused-MoE Triton kernels, torch's quack RMSNorm), pinned as binaries
for sm90; none can run here. Each function therefore follows the reference's in-tree eager
expression for the op, with the reduction orders this build's kernels declare written out
explicitly. How each function is pinned independently of this restatement is listed in its own
module docstring; a function with no independent check says "parity unpinned".

Transcendentals are pluggable (``prims.Prims``): with the default numpy functions the oracle is a
tolerance reference; with the device's own exp/log plugged in (tests do this through the C ABI's
``ix_prim_unary``) the oracle reproduces the kernels' rounding schedule bit for bit, which is
what pins the ORDER of operations separately from libm differences.
"""
