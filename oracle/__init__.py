"""CPU restatement of the MALTOS hot path -- TEST INFRASTRUCTURE ONLY.

Nothing under oracle/ is part of the product: only tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py may import it, and only as the checker.  The product (maltos_amd)
never imports this package and has no CPU fallback.

The reference (xing7code/maltos) is pure Python over stock PyTorch ops, so the restatement is
plain PyTorch as well (device-agnostic: it runs on whatever device its inputs live on).  Every
function cites the reference lines it follows.  How each function is pinned (reference-held known
answers in tests/golden/reference_known_answers.json, library routines, closed forms, invariants)
is listed beside its test in tests/test_oracle_*.py.

Parity unpinned: the numerical output of the third-party `flash_attn` CUDA kernels that the
reference calls at runtime/layers/flash_utils.py:189-202,239-258,504-514 (package absent from the
reference tree and from this image, no pinned version).  The restatement follows the published
FlashAttention-2 formulas, which the reference's own dense stand-in
(tests/sequence_ids_attention_mask.py:196-206) also implements, and those ARE pinned.

There is no C restatement to compile: the reference has no compiled code on this path.
"""
