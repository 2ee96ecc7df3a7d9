""""Fused" quantise + GEMM, 3-D x 2-D: drop-in for triton/fused_triton_fwd32.py.

The reference kernel quantises each bf16 tile inside the GEMM loop, so an A tile is
re-quantised for every N tile and a B tile for every M tile.  The quantised values
depend only on (tile, K step): here each operand is quantised once by an HBM-bound
kernel with the fused kernel's own formula (additive 1e-5, no clamp; A per 128x128
tile, B per (row, 128-wide K group)) and the GEMM divides by the scale product.
"""
import torch

from . import ops
from ._common import calc_diff
from ._lib import COMBINE_DIV_PROD, INV_MULTIPLIER, SCALE_BLOCK128, SCALE_ROW_K128

__all__ = ["fused_int8_gemm", "fwd_32", "calc_diff"]


def fused_int8_gemm(A_bf, B_bf, strict=False):
    """bf16 [B,M,K] x bf16 [N,K] -> bf16 [B,M,N] (triton/fused_triton_fwd32.py:71-96)."""
    if A_bf.dim() != 3 or B_bf.dim() != 2:
        raise ValueError("A_bf must be [B, M, K] and B_bf [N, K]")
    qa, sa = ops.quant_block(A_bf.contiguous(), clamp=False, eps_add=True, inv_mode=INV_MULTIPLIER)
    qb, sb = ops.quant_row(B_bf, clamp=False, group=128, eps_add=True, inv_mode=INV_MULTIPLIER)
    return ops.gemm_i8_nt(qa, qb, sa, SCALE_BLOCK128, sb, SCALE_ROW_K128, combine=COMBINE_DIV_PROD, strict=strict)


def fwd_32(a: torch.Tensor, b: torch.Tensor):
    """triton/fused_triton_fwd32.py:104-108 (the reference moves its inputs to the GPU)."""
    return fused_int8_gemm(A_bf=a.cuda(), B_bf=b.cuda())
