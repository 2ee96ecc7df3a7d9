"""Double-channel INT8 GEMM, 3-D x 2-D: drop-in for triton/double-channle_fwd32.py
(importable spelling of the reference's file name).

Both operands are rotated by a full-length Walsh-Hadamard transform, quantised per
row, multiplied with int32 accumulation over the whole K, dequantised by
``sA[m]*sB[n]`` and scaled by 1/K.  The reference's two-pass quantiser (absmax pass,
torch glue, quantise pass) is one single-pass kernel here, and its separate
``C * inv_K`` pass is folded into the GEMM epilogue (as a second bf16 rounding, so
the result is unchanged).
"""
import torch

from . import ops
from ._common import calc_diff, need_bf16_out
from ._lib import INV_AMAX_DIV_127, SCALE_ROW

__all__ = ["hadamard_transform", "rotate_and_row_quant", "triton_per_row_quant_2d", "triton_per_row_quant_3d", "triton_gemm",
           "int8_gemm_pipeline", "fwd_32", "calc_diff"]


def hadamard_transform(x: torch.Tensor, scale: float = 1.0):
    """Replacement of ``fast_hadamard_transform.hadamard_transform`` (the reference's
    external dependency, triton/double-channle_fwd32.py:8): ``x @ H_n * scale`` along
    the last dim, Sylvester order, bf16 in -> bf16 out, n a power of two in [128, 32768].
    Other lengths (multiples of 16 up to 32768) are handled as the external library handles
    them: zero-extended to the next power of two, transformed, cut back -- which is not an
    orthogonal rotation any more, so the pipeline's result is only as good as the reference's
    own at such a K (14336 of the Llama MLP)."""
    return ops.fwht(x, None, scale)


def _row_quant(x, BLOCK_N):
    # BLOCK_N only chunks the reference's absmax pass; its loads are unmasked, so the
    # reference needs N % BLOCK_N == 0 -- kept as the same precondition
    if x.shape[-1] % int(BLOCK_N) != 0:
        raise ValueError(f"last dim {x.shape[-1]} is not a multiple of BLOCK_N={BLOCK_N}")
    return ops.quant_row(x, clamp=True, inv_mode=INV_AMAX_DIV_127)


def rotate_and_row_quant(x, BLOCK_N=2048):
    """``triton_per_row_quant_2d/3d(hadamard_transform(x))`` (triton/double-channle_fwd32.py:273-278) in one pass over
    ``x``: the rotated bf16 tensor, which the reference writes once and reads twice, stays on chip.  Same bits."""
    if x.shape[-1] % int(BLOCK_N) != 0:
        raise ValueError(f"last dim {x.shape[-1]} is not a multiple of BLOCK_N={BLOCK_N}")
    return ops.fwht_quant_row(x, clamp=True, inv_mode=INV_AMAX_DIV_127)


def triton_per_row_quant_2d(x: torch.Tensor, BLOCK_N: int = 2048):
    """[M,N] bf16 -> (int8 [M,N], fp32 [M]) (triton/double-channle_fwd32.py:140-175)."""
    if x.dim() != 2:
        raise ValueError("x must be 2-D")
    return _row_quant(x, BLOCK_N)


def triton_per_row_quant_3d(x: torch.Tensor, BLOCK_N: int = 2048):
    """[B,M,N] bf16 -> (int8 [B,M,N], fp32 [B,M]) (triton/double-channle_fwd32.py:229-266)."""
    if x.dim() != 3:
        raise ValueError("x must be 3-D")
    return _row_quant(x, BLOCK_N)


def triton_gemm(A_int8, B_int8, A_scale, B_scale, out_dtype=torch.bfloat16, post_scale=0.0):
    """int8 [B,M,K] x int8 [N,K], A_scale [B,M], B_scale [N] -> bf16 [B,M,N]
    (triton/double-channle_fwd32.py:62-90).  ``post_scale`` != 0 applies the pipeline's
    ``C * inv_K`` in the epilogue as a second rounding."""
    need_bf16_out(out_dtype)
    return ops.gemm_i8_nt(A_int8, B_int8, A_scale, SCALE_ROW, B_scale, SCALE_ROW, acc_i32_full=True,
                          post_scale=post_scale)


def int8_gemm_pipeline(A_bf, B_bf, out_dtype=torch.bfloat16, hadamard=True):
    """triton/double-channle_fwd32.py:269-285.  ``hadamard=False`` skips the rotation and
    its 1/K factor (needed when K is not a power of two)."""
    torch.cuda.set_device(A_bf.device)
    inv_K = 1.0 / A_bf.shape[-1]
    if A_bf.dim() != 3 or B_bf.dim() != 2:
        raise ValueError("A_bf must be [B, M, K] and B_bf [N, K]")
    if hadamard:   # rotation + quantiser fused: one read of each operand
        A_int8, A_scale = rotate_and_row_quant(A_bf)
        B_int8, B_scale = rotate_and_row_quant(B_bf)
    else:
        A_int8, A_scale = triton_per_row_quant_3d(A_bf, BLOCK_N=128)
        B_int8, B_scale = triton_per_row_quant_2d(B_bf, BLOCK_N=128)
    return triton_gemm(A_int8, B_int8, A_scale, B_scale, out_dtype=out_dtype,
                       post_scale=inv_K if hadamard else 0.0)


def fwd_32(a: torch.Tensor, b: torch.Tensor, hadamard=True):
    """triton/double-channle_fwd32.py:295-311."""
    return int8_gemm_pipeline(a, b, out_dtype=torch.bfloat16, hadamard=hadamard)
