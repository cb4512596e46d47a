"""CPU restatement of RISA's quantized attention path (test infrastructure only).

This package is the parity oracle for the HIP kernels.  It restates, in numpy,
the arithmetic of the reference's CUDA sources operation by operation (IEEE
binary32 with round-to-nearest-even, fused multiply-add only where the CUDA
source spells ``fmaf``, reductions in the order the CUDA thread layout fixes).
It is slow, single-purpose and deliberately free of any dependency on the
product package: only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may import it, and only as the checker.

Arithmetic conventions (they decide bits, so they are stated once here):

* ``a / b`` is the correctly rounded binary32 quotient; the reference binary is
  built with ``--use_fast_math`` (csrc/CMakeLists.txt:40) where the same source
  expression becomes an approximate quotient.  The source-level IEEE meaning is
  the definition used here and by the HIP kernels.
* separate ``*`` and ``+`` in the CUDA source stay separate (no contraction);
  ``fmaf`` is a single rounding.
* ``ex2.approx``/``lg2.approx``/``rcp.approx`` are replaced by the correctly
  rounded functions, so attention outputs are compared with a tolerance and
  everything before the softmax is compared bit for bit.

Parity pins (what each function is checked against in ``tests/``):

* ``prepare.quantize_values``: exact known answer of
  tests/cuda/test_value_quantization.py:18-52 (power-of-two scales), centre
  identity of tests/cuda/test_probability_mass.py:148-155.
* ``prepare.rotate``/``quantize_queries``/``quantize_keys``: the reference holds
  no code-level vector for these ("parity unpinned" at the level of the shipped
  binary); pinned by the closed form y = H_n diag(s) x / sqrt(n) against a dense
  Sylvester matrix, orthogonality, dot-product invariance and brute-force group
  maxima on tiny inputs.
* ``prepare.detect_key_anchor``: brute-force float64 evaluation of the same
  criterion on inputs whose decision is not near a tie.
* ``attention.attend``: tile-max known answer of
  tests/cuda/test_risa_attention.py:20-92, probability-mass preservation of
  tests/cuda/test_probability_mass.py:21-70, FP32 SDPA tolerances of
  tests/cuda/test_risa_attention.py:94-193.
* ``selection.select_retained_mass``: brute force against the pure-torch
  algorithm of src/risa_attention/reference.py:115-131.
* ``masks.key_mask_tiles``: known answer of
  tests/cuda/test_key_mask_tiles.py:78-104.
* ``prepare.lse_shift``: closed form of tests/cuda/test_lse_correction.py:9-31.
"""
