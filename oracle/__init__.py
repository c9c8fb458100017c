"""CPU oracle for the expert-worker hot path.  TEST INFRASTRUCTURE ONLY.

This package restates, on the CPU, what the reference computes on the path
routing ids -> row mapping -> token permute -> per-expert SwiGLU FFN (grouped
GEMM) -> gate-weighted unpermute/combine.  It exists to CHECK the HIP kernels:
only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import it.  Nothing in ``disagmoe_amd`` imports it, and the
product path raises when the HIP library is missing instead of falling back to
this code.

Every function cites the reference file:line it follows (paths relative to the
reference checkout).  How each function is pinned (independently of its own
formula) is listed below; the checks live in ``tests/test_oracle_*.py``.

  routing.get_mappings_from_exp_ids   hand-derived known answers
      (tests/golden/routing_kat.json), brute-force rank counting on small
      random inputs, permutation / sortedness / count invariants.
  routing.get_mappings_stable          ``torch.sort(stable=True)`` inverse.
  routing.merge_by_exp_ids             equals the single-stream rule on the
      concatenation (the reference runs the same loop over several batches).
  routing.expert_batch_sizes           ``numpy.bincount`` + index select.
  routing.sort_by_prefill_order        the reference's own known answer
      (tests/engine/test_exp_engine.py:29-40) in tests/golden/prefill_kat.json.
  routing.fused_topk                   closed forms: logits ``ln(1..E)`` give
      probabilities ``i / sum``; renormalised weights equal the softmax over the
      kept logits alone (float64); brute-force selection on small inputs; ties.
  rows.permute_tokens / gather_rows    the reference test's row loop
      (tests/ops/test_memory.py:27-31) and ``torch.index_select``.
  ffn.gmm                               E=1 equals ``torch.matmul``; float64
      block matmul on small cases; ``trans_b``; zero-row experts.
  ffn.moe_experts_forward               composition of per-expert
      ``silu(x@w1) * (x@w3) @ w2`` in float64 on small cases.
  ffn.combine / combine_reference_chain closed form on small cases; k=2 chain
      equals the two torch statements the reference executes.
  fp8.quantize_* / dequantize           torch's ``float8_e4m3fn`` cast and the
      ``absmax/448`` rule; round trip error bound 2^-4 relative.

PARITY UNPINNED (no reference fixture or importable implementation exists):
  * the exact bf16 bit pattern of the third-party CUTLASS grouped GEMM
    (``hogura99/grouped_gemm@async``, not vendored, no commit pinned); graded
    instead at max relative error 1e-2 against the fp32-accumulated result;
  * ``gmm``'s behaviour for ragged sizes / zero-row experts / ``trans_b`` is not
    covered by any reference test (tests/ops/test_gemm.py only checks
    self-consistency) and is pinned by the textbook definition;
  * the fp8 path has no reference code at all; its oracle is the bf16 ``gmm``
    on de-quantised weights.
"""
