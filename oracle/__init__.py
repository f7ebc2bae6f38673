"""CPU restatement of the reference's quantized-weight linear path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may import this: it is the checker that
tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg compare the HIP path against.

Each function cites the reference file:line it follows (paths relative to the reference tree).

Pinning status (what independent evidence fixes each function):
  ggml.dequant_q8_0      reference KAT test/unit/test_gguf.py:36-40 + closed form d*q
  ggml.dequant_mxfp4     reference KATs test/unit/test_gguf.py:42-48, :65-87 (seed 42 closed form), :89-105 (real block)
  ggml.dequant_q4_0      no reference vector without gguf-py; pinned by the published ggml scalar loop
                         (ggml-quants.c dequantize_row_q4_0, restated in oracle/c/oracle.c) + brute force
  ggml.dequant_q6_k      same: published ggml scalar loop dequantize_row_q6_K + exactness argument (23 significant bits)
  linear.*               float64 textbook x @ W.T as the tolerance anchor; dtype rules from mixin/op.py:367-392
  mxfp8.float_to_e4m3    exhaustive round trip over all 256 codes, brute-force nearest-even on a grid, torch.float8_e4m3fn cross-check
  mxfp8.quantize_mxfp8   closed form + invariants (scaled block max in [1,2), powers of two exact); test twin test_asm_gemm.py:278-292
  moe.pairwise_topk      reference vectors test/unit/test_attention.py:249-270, argsort equivalence
  moe.route / rows_e / dispatch / combine   no reference test exists; pinned by a case worked by hand from moe_routing.py:109-122 (a tie, an
                         empty expert, literal topi / weights / off / dest_row / tile experts), minimal padding at 255 / 256 / 257 rows,
                         and invariants (bijection into 256-padded expert ranges, identity-expert round trip): tests/test_oracle_pins.py
  mxfp8.grouped_mx_gemm_ref   no reference test exists; pinned by an exact rational brute-force sum over E4M3 codes and E8M0 scales
                         decoded from their definitions, on both sides of an expert boundary with an empty expert: tests/test_oracle_pins.py
  llm.Model.forward      MoE block: closed forms from test/unit/test_llm_moe.py:15-124.  Dense wiring: closed forms that separate the
                         plausible mistakes (residual pass-through, single position returns v with the repeat_interleave head mapping,
                         uniform attention = mean of the values written at 0..pos, FFN fed from the post-attention residual, greedy =
                         first maximum): tests/test_oracle_pins.py.  The reference's own 32-token stream cannot be produced here
                         (the reference needs Python >= 3.11): PARITY UNPINNED at the token-stream level only
"""
