"""CPU oracle for the dlBLAS inference operators -- TEST INFRASTRUCTURE, not product code.

Each function restates, in plain PyTorch-CPU / numpy, the ground-truth formula the reference
(DLCompiler's dlBLAS) uses in its own tests for one operator, citing the reference file:line
it follows.  Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this package, and only as the checker; nothing in ``dlcompiler_amd``
imports it.

Pinning status (what, other than the formula itself, each function is checked against in
``tests/test_oracle_*.py``):

* ``activation.silu_and_mul``       pinned: torch.nn.functional.silu, closed-form special cases
* ``moe_gating.topk_softmax``       pinned: torch.softmax/torch.topk on tie-free rows, brute force
* ``moe_gating.start_end``          pinned: one-hot/cumsum identity of the reference docstring
* ``moe_gating.align_block_size``   parity unpinned w.r.t. the reference (the pad-to-block
                                    layout does not exist there); pinned to a brute-force
                                    Python loop and to its invariants
* ``attention.prefill_attention``   pinned: torch scaled_dot_product_attention, closed forms
* ``attention.paged_decode``        pinned: same dense routine after an independent gather,
                                    page-permutation invariance; window = shorter context,
                                    soft-cap limits (identity / mean of V)
* ``attention.paged_prefill``       pinned: no history = prefill_attention, every row = a
                                    paged_decode over the context ending there, the reference
                                    test's additive-bias formulation
* ``decoder_ops.fill_kv_cache``     pinned: page-by-page copy loop of the reference test
* ``decoder_ops.rms_norm``          pinned: torch.nn.functional.rms_norm, fp64 evaluation
* ``decoder_ops.apply_rotary_pos_emb``  pinned: complex rotation identity, norm preservation
* ``fp8.per_token_group_quant`` / ``fp8.fused_moe_fp8``  parity unpinned w.r.t. the reference
                                    (no fp8 MoE exists there); pinned to torch's own e4m3fn
                                    cast, round-trip bounds and an fp64 dense evaluation
* ``fused_moe.fused_moe``           pinned: fp64 evaluation of the per-expert MLP loop
"""
