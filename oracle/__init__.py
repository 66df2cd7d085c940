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
  pinned by closed forms / brute force / an independent bf16 implementation (tests/test_oracle_*.py):
      bf16.*, linear.int_gemm (int64 brute force), linear.epilogue (float64 cross-check), moe.route_sort
      (permutation properties), moe.combine (sequential bf16 sum restated two ways), layout.e8m0 map (closed form),
      linear.swiglu rounding structure (torch bf16, every gate pattern), moe.route (torch CPU ops, brute force),
      linear.rmsnorm / rmsnorm_quant / res_norm_quant / swiglu_quant / headnorm / fullnorm STRUCTURE
      (tests/test_oracle_norms.py: `w * bf16(x * inv)` against torch bf16 with wrong orders shown to differ, eps
      inside the root, mean not sum, per-head slices and their weight vectors, whole-width statistics, head-major
      outputs, untouched v, zero padding rows, fused kernels == composition of their parts), linear.row_sumsq
      (every element counted once; within (log2 K + 4) half-ulps of math.fsum)
  parity unpinned (the arithmetic lives in MLX / mlx-lm, which are not vendored in the reference and not installed):
      the ORDER of the FP32 additions inside the sum of squares (MLX: 32-lane simd_sum tree; here: 64-lane
      butterfly) and metal::precise::rsqrt against IEEE 1/sqrt -- a few FP32 ulps of `inv`, which can flip a bf16
      rounding of x * inv in rare elements; metal::precise::exp inside linear.swiglu (linear.exp_f32 rounds to the
      same bf16 as the exact exponential for every bf16 input, so only a mis-rounding MLX exp could differ);
      moe.route at exact probability ties (argpartition's choice) and MLX's softmax rounding at a bf16 tie.
      No vector can settle these without MLX; the kernels are held bit-exact to THIS restatement and within 1e-2
      relative Frobenius error of a float64 evaluation.
"""
