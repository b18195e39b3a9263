"""CPU oracle for the MoEspresso attention hot path.

TEST INFRASTRUCTURE ONLY. Nothing in the product package imports this. Only
the test suite, the smoke check and the CPU-baseline leg of the benchmark may
call it, and there only as the checker.

Every function restates, in NumPy, an algorithm of the reference and cites the
reference file:line it follows. The reference cannot run outside Apple Metal
(MLX), so the restatement is pinned by the reference's own known-answer tests,
by closed forms and by brute force on tiny inputs (see tests/test_oracle_*.py).

Parity status per function group ("pinned" = a check that a plausible mistake
would fail; "unpinned" = only self-consistency is available):

  hadamard128 / indexer_qat          pinned  (H.H=128 I vs scipy, ones KAT, lattice invariants)
  pow2 group scale bit patterns      parity unpinned at stress exponents: the
                                     reference keeps Metal's precise::log/exp
                                     bits; this oracle uses correctly rounded
                                     float32 log/exp (exactly 2^k for |k| <= 12,
                                     a few ulp off 2^k beyond, as in the reference)
  e4m3fn table / fp8_kv_roundtrip    pinned  (torch.float8_e4m3fn cast away from ties, table closed form)
  indexer scores                     pinned  (64*scale KAT, 144/sqrt(128) KAT, float64 closed form)
  score_tail reduction order         parity unpinned (MLX col_reduce/simd_sum tree is
                                     not observable; own fixed order, value pinned by float64)
  radix_select_topk                  pinned  (lexsort brute force, all-tie -> arange, reference KAT)
  rope / yarn                        pinned  (reference pinned inv-freq and angle values)
  sink attention / visit rules       pinned  (single-key+sink KAT, torch.softmax when sink=-inf,
                                     visibility KATs, brute-force row lists)
  prefill visit rules / last_pos     pinned  (independent per-position walk with torch.softmax float64; the
                                     composed reference form with its filter rule on sorted and unsorted ids)
  fused_decode_prep                  pinned  (all-tie -> arange KAT, integer data against a brute-force
                                     float64 sum and lexsort, prepared row against rope and FP8 parts)
  round_bf16 / round_f16             pinned  (torch.bfloat16 / float16 casts incl. ties, inf, NaN, denormals)
  q8 quantisers (affine g64)         parity unpinned (MLX mx.quantize edge rules not in the
                                     reference tree; own documented rule, round trip bounded)
  gqa decode / causal flash prefill  pinned  (float64 torch.softmax closed form)
  indexer_q_qat_live                 tie rule pinned (the seven lattice midpoints, hand values) and
                                     scale rule pinned on exact inputs; parity unpinned within an ulp
                                     of a power of two (Metal log2/exp2 bits unknown; the reference
                                     tests this kernel to 1e-5 only)
  indexer_scores_tiled_live          pinned  (term-by-term float64 sum on half-rounded operands,
                                     visibility against the closed form)
  fused_partial_rope                 pinned  (float64 rope closed form, NumPy's native float16
                                     arithmetic for the per-operation rounding, offset form ==
                                     positions form, inverse undoes forward); parity unpinned in the
                                     last bit of cos/sin: correctly rounded float32 here, Metal's
                                     precise::cos/sin bits unknown
"""
