"""CPU restatement of the reference's per-rank hot path (BlackSamorez/tensor_parallel v2.0.0).

TEST INFRASTRUCTURE ONLY. Nothing under `tensor_parallel_amd/` imports this package; only `tests/`, the smoke
check and the benchmark's CPU-baseline leg do, and only as the checker or the baseline being timed.

Modules and the reference code each one follows:
  slicing.py        Split / SplitInChunks / SplitInGroupedChunks / Scale and their undo
                    (src/tensor_parallel/state_actions.py:39-119), split_heads and the integer attribute
                    rules (src/tensor_parallel/aux_actions.py:18-40), numpy on raw element arrays
  naming.py         get_parameter_name_mapping (src/tensor_parallel/config.py:157-191) and
                    convert_state_dict (src/tensor_parallel/dispatch.py:75-131) over the oracle's actions
  reduce.py         the "sum" rule's arithmetic (src/tensor_parallel/cross_device_ops.py:49), bit-level
  shard_forward.py  rank-shard Linears, the SiLU-gated MLP shard and the W-thread forward
                    (src/tensor_parallel/wrapper.py:69-72, tensor_parallel.py:237-287), torch on CPU
  attention.py      the attention core the wrapped module runs on a rank's heads (softmax(q k^T) v, grouped-query,
                    causal aligned to the end of the keys), float64; the reference has no attention code of its own
  rope.py           rotary embedding of the new query / key rows and their hand-over to the rank-local cache, in the
                    arithmetic of the wrapped transformers module (the reference only routes the cache tensors:
                    src/tensor_parallel/aux_actions.py:7-15)
  sharding.py       flat per-rank shards of the replicated parameters and their recombination
                    (src/tensor_parallel/sharding.py:96-180)
  quant.py          int8 weight-only quantisation with outlier columns - NOT in the reference: parity
                    unpinned against it; defined in closed form and checked against fp64 matmul

How each function is pinned (tests/test_oracle_*.py):
  slicing      the reference's three docstring vectors (state_actions.py:40,67,94); torch.tensor_split on
               every (n, W) with n < 40, W <= 9; brute-force index enumeration on small tensors;
               undo(split) == identity; the shard shapes of Llama-2-7B and of Falcon-40B at W = 2, 4, 8
  naming       hand-derived Llama names; golden vectors written by tests/golden/make_golden.py
  reduce       torch CPU bf16/fp16 addition (a third-party routine), W = 2 and chained W = 3..8
  forward      sum of row-parallel partials == unsplit Linear, concat of column-parallel == unsplit Linear,
               both in fp64
  attention    torch's CPU scaled_dot_product_attention where it covers the case, explicit loops on tiny inputs for
               grouped heads and Sq < Skv causal, rows of probabilities sum to one, a single visible key returns its value
  rope         transformers' apply_rotary_pos_emb bit for bit (bf16, fp16, fp32), the complex-rotation closed form in
               fp64, norm preservation, identity at position 0
  sharding     combine(make(x)) == x on ragged sizes, equal flat lengths, the parameter counts asserted by the
               reference's own test (tests/test_basic.py:110-135)
  quant        dequantised weights within scale/2 of the originals; fp64 matmul of the definition
"""
