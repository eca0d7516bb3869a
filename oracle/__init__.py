"""CPU oracle for the int8 weight-only linear + decode-attention path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this
directory; it is used by tests/, by __graft_entry__.smoke() and by the
cpu_baseline leg of bench.py, always as the checker and never as the thing
that is measured or shipped.

Every function restates, in numpy / plain C, what the reference computes and
cites the reference file:line it follows (paths relative to the reference
checkout).  How each function is pinned:

  quantize_ref128        known answers recorded from the unmodified reference
                         quantiser (tests/golden/quant_known_answers.json),
                         closed forms, brute force on tiny matrices, and the
                         independent plain-C restatement oracle/quant_ref.c
  preprocess_ref_sm80    known byte orders of the reference's processed layout
                         (same fixture) + "is a permutation of q+128"
  dequant_matmul         textbook fp32 matmul; identity / one-hot special cases
  rmsnorm, swiglu, rope  closed forms, norm preservation, pos=0 identity,
                         equality with the rotate_half formulation
  layernorm, add_bias,   float64 textbook LayerNorm (zero mean / unit variance with
  add_bias_residual_norm gamma = 1, beta = 0; shift and scale invariance), the two fp16 adds
                         brute-forced element by element, RMSnorm form without a bias
  decode_attention       step=1 => v/(1+1e-6), uniform keys => mean(V),
                         brute-force softmax, padded prefix has zero weight
  alibi_slopes / mask    closed form for n=40 and powers of two
  quantize_sym127        scalar brute force; closed-form scale; extremes at +-127
  layer / decoder        an independently written float64 model in the Hugging
                         Face formulation without a KV cache
                         (tests/hf_formulation.py), with planted-mistake
                         controls; zero-projection identity; one-token closed
                         form; incremental call == last row of a longer prefill
                         (tests/test_oracle_composition.py)

The reference itself holds no test, fixture or golden vector for any function
on this path, so every pin above is one the mathematics or the published model
definitions fix.

The reference's own build of the quantiser needs <cuda_runtime.h> and the
cutlass headers, which this image lacks, so no oracle/_ref build exists.
"""
