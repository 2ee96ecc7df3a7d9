"""CPU oracle of the INT8 quantized-linear hot path -- TEST INFRASTRUCTURE ONLY.

This package restates, on torch-CPU tensors in un-fused IEEE fp32, the arithmetic
of every function of jiaoch/Triton-INT8's quantize -> int8 GEMM -> dequant path.
It is the checker the HIP kernels are compared against and the timed CPU baseline
of the benchmark.  Nothing in the product package may import it: only ``tests/``,
``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline`` leg do.

One module per reference script, same function names and argument meaning:

=============================  ==============================================
oracle module                  reference file followed
=============================  ==============================================
``block_channel_fwd32``        triton/block_channel_fwd32.py
``block_channel_bwd33``        triton/block_channel_bwd33.py
``double_channel_fwd32``       triton/double-channle_fwd32.py
``double_channel_bwd33``       triton/double_channel_bwd33.py
``fused_fwd32``                triton/fused_triton_fwd32.py
``fused_bwd33``                triton/fused_triton_bwd33.py
``tilelang_block_channel_fwd`` tilelang/block_channel_fwd.py
``tilelang_block_channel_bwd`` tilelang/block_channel_bwd.py
``hadamard``                   external fast_hadamard_transform (closed form)
``linear``                     linear-layer wiring + modes (no reference file)
=============================  ==============================================

Pinning status (what fixes each function besides its own formula):

* quantizers -- brute-force scalar loops in plain C (``oracle/c/ti8_ref.c``,
  written independently), planted ties / zero groups / outliers, the
  invariants ``max|q| == 127``, ``|x - q*s| <= s/2`` and ``Q(x^T) == Q(x)^T``.
* integer GEMM -- exact by definition; checked against float64 matmul,
  ``torch._int_mm``, identity and +-127 saturation cases.
* promotion / epilogue -- literal fp32 loop, cross-checked against a float64
  evaluation within fp32 rounding and against the C restatement bit-for-bit.
* Hadamard -- ``scipy.linalg.hadamard`` (Sylvester order), involution
  ``H(H(x)) == n x``, one-hot rows; exact on small-integer inputs.
  The summation order INSIDE the external fast_hadamard_transform CUDA kernel
  is not available (its source is not part of the reference): the butterfly
  order used here (strides 1, 2, 4, ...) is this build's own, so values that
  depend on fp32 rounding order after the transform are **parity unpinned**
  against that library.  The reference pins that boundary only with
  ``calc_diff < 1e-3`` end to end, which the tests repeat.
* end to end -- the reference's own acceptance bar ``calc_diff(C, bf16 matmul)
  < 1e-3`` on N(0,1) operands.
"""
