"""Double-channel INT8 GEMM, 3-D x 3-D: drop-in for triton/double_channel_bwd33.py."""
import torch

from . import ops
from ._common import calc_diff, need_bf16_out
from ._lib import SCALE_ROW
from .double_channel_fwd32 import _row_quant, hadamard_transform, rotate_and_row_quant

__all__ = ["hadamard_transform", "triton_per_row_quant_3d", "triton_gemm", "int8_gemm_pipeline", "bwd_33",
           "calc_diff"]


def triton_per_row_quant_3d(x: torch.Tensor, BLOCK_N: int = 2048, num_warps=4, num_stages=2):
    """[B,M,N] bf16 -> (int8, fp32 [B,M]) (triton/double_channel_bwd33.py:142-176).
    ``num_warps`` / ``num_stages`` are accepted for signature compatibility only."""
    if x.dim() != 3:
        raise ValueError("x must be 3-D")
    return _row_quant(x, BLOCK_N)


def triton_gemm(A_int8, B_int8, A_scale, B_scale, out_dtype=torch.bfloat16, post_scale=0.0):
    """int8 [B,M,K] x int8 [B,N,K], scales [B,M] and [B,N] (triton/double_channel_bwd33.py:60-87)."""
    need_bf16_out(out_dtype)
    if B_int8.dim() != 3:
        raise ValueError("B_int8 must be [B, N, K]")
    return ops.gemm_i8_nt(A_int8, B_int8, A_scale, SCALE_ROW, B_scale, SCALE_ROW, acc_i32_full=True,
                          post_scale=post_scale)


def int8_gemm_pipeline(A_bf, B_bf, out_dtype=torch.bfloat16, hadamard=True):
    """triton/double_channel_bwd33.py:186-201."""
    torch.cuda.set_device(A_bf.device)
    inv_K = 1.0 / A_bf.shape[-1]
    if A_bf.dim() != 3 or B_bf.dim() != 3:
        raise ValueError("A_bf must be [B, M, K] and B_bf [B, N, K]")
    if hadamard:   # rotation + quantiser fused: one read of each operand
        A_int8, A_scale = rotate_and_row_quant(A_bf)
        B_int8, B_scale = rotate_and_row_quant(B_bf)
    else:
        A_int8, A_scale = triton_per_row_quant_3d(A_bf, BLOCK_N=128)
        B_int8, B_scale = triton_per_row_quant_3d(B_bf, BLOCK_N=128)
    return triton_gemm(A_int8, B_int8, A_scale, B_scale, out_dtype=out_dtype,
                       post_scale=inv_K if hadamard else 0.0)


def bwd_33(a: torch.Tensor, b: torch.Tensor, hadamard=True):
    """triton/double_channel_bwd33.py:204-220."""
    return int8_gemm_pipeline(a, b, out_dtype=torch.bfloat16, hadamard=hadamard)
