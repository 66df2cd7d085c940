"""CPU oracle for the SC-MXFP4 W4A8 linear-layer path.  TEST INFRASTRUCTURE ONLY.

This package restates, in numpy, the algorithms of the reference's numpy layer and the arithmetic its kernels are
specified to perform.  It exists to check the HIP kernels; it is never the thing that ships or is measured.  Only
the test-suite, the smoke check and the `cpu_baseline` leg of the benchmark may import it.  The product package
never does, and it raises when its HIP library is missing rather than falling back to anything here.

Module map (reference files are cited as path:line inside each function):
  bf16        bfloat16 bit helpers (round-to-nearest-even on the FP32 pattern)
  quantizer   E2M1 rounding, block exponents ("search"), spread constraint, INT8 embedding, byte-shift packing
  layout      the packed storage format (4-bit codes + block codes + row scale), standard MXFP4 (E8M0) view
  family      the integer-exact format family quantizer (float row base, integer block multipliers)
  linear      activation quantization, INT32 GEMM, scaling epilogues, SwiGLU, RMSNorm+quant, decode GEMV
  moe         token sort / expert offsets, grouped GEMM, weighted combine

Parity status
  pinned by golden vectors written from the reference's own numpy modules (tests/golden/):
      quantizer.*  layout.*  family.quantize  family.pack_parts  linear.act_quant (via reference quant_ref formula)
  pinned by closed forms / brute force (tests/test_oracle_*.py):
      bf16.*, linear.int_gemm (int64 brute force), linear.epilogue (float64 cross-check), moe.route_sort
      (permutation properties), moe.combine (sequential bf16 sum restated two ways), layout.e8m0 map (closed form)
  parity unpinned (the arithmetic lives in MLX / mlx-lm, which are not vendored in the reference and not installed):
      linear.swiglu (exp rounding), linear.rmsnorm_quant / rmsnorm reduction order, linear.headnorm, linear.fullnorm.
      These follow the prose and kernel text of e2e/sc_kernels.py:120-160,317-328 with this build's own wave-64
      reduction order; the kernels are held bit-exact to THIS restatement and within 1e-2 relative Frobenius error
      of a float64 evaluation.
"""
