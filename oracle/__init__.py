"""CPU oracle for the paged-attention path.  TEST INFRASTRUCTURE ONLY.

Nothing under this package is part of the shipped product: only the test
suite, the smoke check and the CPU-baseline leg of the benchmark may import
it, and only as the checker.  The product package never imports it.

Contents
--------
dense_attention   torch restatement of the reference's dense attention
                  arithmetic (ironcore/layers/attention.py:68-142), same ops,
                  same order, same dtype at every step.
paged             block-table gather + KV-append closed form that drive the
                  dense restatement through a block KV cache (the cache
                  interface is defined by this build; the reference has none).
brute_force       independent float64 loops used to pin dense_attention.
rope              rotary position embedding (ironcore/layers/
                  positional_embedding/rotary.py:31-83) with the table row of a
                  token as an explicit argument.
gpt2              CPU restatement of the reference's GPT-2-shaped forward
                  (ironcore/language_model.py:67-100, ironcore/models/
                  transformer.py:77-132) with a full-recompute generate loop
                  and a block-KV-cache generate loop.

Pinning status (what checks each function; see tests/test_oracle_*.py)
-----------------------------------------------------------------------
dense_attention.dense_attention   pinned: float64 brute force on tiny shapes,
                                  torch scaled_dot_product_attention in fp32,
                                  closed forms (ctx=1, equal keys, shift
                                  invariance), GQA == MHA on repeated K/V.
                                  The reference's tests hold no golden vectors
                                  for it (shape/finiteness checks only).
paged.gather_kv / paged_decode /
  paged_prefill                   pinned: block-permutation invariance, equals
                                  dense over contiguous rows, chunked prefill
                                  equals rows [P, P+C) of one causal pass.
paged.kv_append                   pinned: closed form vs torch index_copy_,
                                  sentinel preservation, idempotence.
rope.rope_tables / rope_rotate    pinned: float64 complex multiplication,
                                  position 0 == identity, norm preservation,
                                  relative-position property, closed-form
                                  tables.
gpt2.*                            pinned: cached generate == full recompute
                                  (causal-model identity); layer arithmetic vs
                                  torch.nn.functional primitives; logits and
                                  greedy tokens vs transformers' GPT-2 and Llama
                                  on the same random weights
                                  (tests/test_weights_hf.py, test_weights_llama.py).
Committed vectors                 tests/golden/*.npz (float64-loop attention
                                  outputs; transformers' logits and greedy
                                  continuations for seeded GPT-2 and Llama
                                  weights), checked by tests/test_golden.py.
_flash_attention numerics         parity unpinned (third-party flash_attn wheel,
                                  absent here; ironcore/layers/attention.py:
                                  144-206).  Not restated: the layer's flash
                                  branch is checked against dense_attention
                                  under the causal mask, the comparison the
                                  reference's own tests make
                                  (tests/test_attention.py:618-789).
"""
