"""CPU oracle for the packed-SFT document-masked attention path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package (``maester_amd``) may import
this module; only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` use it, and only as the checker -- never as the thing measured or shipped.

Every function is a restatement (our own code, CPU, numpy/torch/C) of the reference
algorithm for this path and cites the reference ``file:line`` it follows.  The arithmetic
of the attention itself lives in a third-party dependency of the reference --
``torch.nn.attention.flex_attention`` (reference pins ``torch>=2.7`` in
``pyproject.toml:13``) -- which is importable here, so the oracle also exposes thin
wrappers that drive torch's own ``create_block_mask`` / ``flex_attention`` with the
restated mask predicates.  No file of the reference is imported or executed.

Pinning status (what each function is checked against, in ``tests/test_oracle_*.py``):

===========================  ====================================================================
function                     pinned by
===========================  ====================================================================
masks.allowed / dense_mask   truth tables of reference tests/test_packed_sft.py:72-102,410-430 and
                             tests/test_packed_attention.py:279-336 (window inclusive)
tile_map.tile_lists (numpy)  torch ``create_block_mask`` (live) on tiny and ragged S, the known
tile_map_ref.c (C)           layouts of tests/test_packed_sft.py:112-115,170-176, invariants
                             (disjoint, diagonal partial, q lists = transpose), each other
prologue.rope_tables/apply   HF ``rotate_half`` form (tests/test_rope.py:85-138), norm preservation,
                             position 0 = identity, closed form on 2-d rotation
prologue.rms_norm            transformers ``Gemma3RMSNorm`` (local instantiation), unit mean-square
                             invariant, scale invariance
attention.dense_attention    torch eager ``flex_attention`` on CPU, the v=-1/+1 known answer of
                             tests/test_packed_sft.py:164-212, fp64 brute-force loops on tiny
                             inputs, ``torch.autograd.gradcheck`` (backward)
packed_ids.*                 exact expectations of tests/test_packed_sft.py:22-66
linear_ce.linear_cross_...   ``torch.nn.functional.cross_entropy`` + autograd in fp64 (train.py:258-259),
                             scipy ``logsumexp``, closed forms, zero row sums, central differences
===========================  ====================================================================

No function of the attention path is "parity unpinned".  The gradient filter of cut-cross-entropy
(the dependency behind model.py:762-769, absent here) is not restated: "parity unpinned".
"""
