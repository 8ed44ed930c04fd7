"""CPU oracle for the ReDrafter per-step hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this directory; it is used by
`tests/`, by `__graft_entry__.smoke()` and by the `cpu_baseline` leg of `bench.py` as the checker
(and as the timed CPU baseline), never as the thing being shipped.

Modules
  tree_oracle     integer work: prefix dedup, unpacker, pack, tree mask, padding/causal masks
  accept_oracle   greedy / speculative-sampling acceptance, residual distribution, KV + ids update
  fp_oracle       floating point: masked attention (fp64), beam-search post-GEMM chain, argmax
  torch_path      torch restatement of the whole decode step (models + loop); the CPU baseline
"""
