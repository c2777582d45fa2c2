"""CPU oracle for the attention path (forward results and gradients).  TEST INFRASTRUCTURE ONLY.

Nothing in the product (the ``attentionengine_amd`` package) imports this package; only
``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` do, and only
as the checker.

Modules
  attention_ref.py  closed-form restatements of the reference's eager-PyTorch references
  online_interp.py  interpreter that runs traced score_mod / mask_mod / OnlineFunc graphs
                    tile by tile (the online algorithm of attn_script/Readme.md:45-65)
  masks.py          brute-force mask / block-mask evaluation

How each function is pinned (see the tests named below, all in tests/test_oracle.py):
  softmax_attention      vs torch.nn.functional.scaled_dot_product_attention (library routine),
                         vs a pure-python triple loop on tiny inputs, rows of P sum to one,
                         lse == logsumexp of the masked scaled scores, GQA == repeat_interleave MHA
  sigmoid_attention      PARITY UNPINNED by the reference (its only sigmoid reference is the external
                         flash_sigmoid package, bench_utils.py:736-744); pinned here by the closed
                         form vs a python loop and by sigmoid(x) == (tanh(x/2)+1)/2
  relu_attention         vs python loop (restates bench_utils.py:979-984)
  mla_decode             equals softmax_attention on the concatenated operands (restates
                         mla_decode_tl.py:266-306 / mla_decode_cute.py:88-105), vs python loop
  merge_partials         merging partial (o, lse) over any KV partition == unsplit result
  block masks            known answers hand-derived from core/transform/core.py:410-488 for the three
                         masks of attention_engine/tests/test_blockmask.py:3-10, vs python loops
  online interpreter     equals the closed forms for every block size (block-size invariance)
"""
