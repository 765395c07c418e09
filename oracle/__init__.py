"""CPU restatement of the reference's attention-op hot path.  TEST INFRASTRUCTURE ONLY.

Nothing in ``paraattention_amd`` imports this package; only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` do, and
only as the checker.  Each function cites the reference lines it restates.

Where the arithmetic lives (the reference is pure Python over torch, pinned
torch==2.6.0 in its README.md:153 and torch==2.5.0 in quick_install.sh:3):
  attention.py  softmax(QK^T)V + log-sum-exp: the aten SDPA kernels called at
                src/para_attn/ops/__init__.py:58-109; restated in fp64 numpy and,
                as the library routine, torch's CPU flash kernel
  merge.py      torch _SDPAMerger (torch/distributed/tensor/experimental/
                _context_parallel/_attention.py:138-223)
  sparse.py     src/para_attn/sparse_attn.py:74-278 (ranges, run scan, merges)
  fbcache.py    src/para_attn/first_block_cache/utils.py:220-234, 269-286
  taylorseer.py src/para_attn/first_block_cache/taylorseer.py:4-64 (finite differences, extrapolation)
  inputs.py     seeded generators of the benchmark configurations

Pinning status (what fixes each function besides its own formula):
  attention.sdpa_lse_f64       closed forms (K=0, constant V, one dominant key,
                               Skv=1), key-permutation invariance, and torch's
                               CPU SDPA library routine
  merge.merge_step             torch's own _SDPAMerger on CPU; logaddexp closed
                               form; identity on an empty partial; split-KV
                               attention + merge == full attention
  sparse.mask_row_runs /       brute force over all masks of <= 8 blocks against
  sparse.struct_sparse_f64     the -inf-masked dense closed form
  fbcache.residual_diff_ratio  torch's bf16/fp16 CPU op chain on fixtures incl.
                               near-threshold cases; decision-table known answers
  taylorseer.finite_differences torch's bf16/fp16/fp32 CPU op chain evaluating the
  / extrapolate / TaylorSeer   reference's expressions, bit for bit; closed forms (a linear
                               sequence is extrapolated exactly, t^2 with unit window gives
                               (t+e)^2 - e); the compute/skip schedule by enumeration
The reference's own tests hold no golden vectors for this path
(tests/ops/test_ops.py:62 compares the output with itself), so none are used.
"""
