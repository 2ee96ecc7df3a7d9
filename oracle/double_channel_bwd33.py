"""Oracle of triton/double_channel_bwd33.py (3-D x 3-D twin of the double-channel
forward: both operands Hadamard-rotated and per-row quantised).

TEST INFRASTRUCTURE -- torch-CPU restatement, un-fused IEEE fp32.
"""
import torch

from ._prims import calc_diff
from .double_channel_fwd32 import (dequant_epilogue, gemm_i32, row_quant, K_ok,
                                   scale_bf16)
from .hadamard import hadamard_transform

__all__ = ["triton_per_row_quant_3d", "triton_gemm", "int8_gemm_pipeline", "bwd_33",
           "calc_diff", "hadamard_transform"]


def triton_per_row_quant_3d(x: torch.Tensor, BLOCK_N: int = 2048, num_warps=4, num_stages=2):
    """triton/double_channel_bwd33.py:142-176 (launch hints have no arithmetic effect)."""
    assert x.dim() == 3
    return row_quant(x, BLOCK_N)


def triton_gemm(A_int8, B_int8, A_scale, B_scale, out_dtype=torch.bfloat16):
    """triton/double_channel_bwd33.py:60-87; A_scale [B,M], B_scale [B,N]."""
    assert B_int8.dim() == 3 and K_ok(A_int8, B_int8)
    return dequant_epilogue(gemm_i32(A_int8, B_int8), A_scale, B_scale, out_dtype)


def int8_gemm_pipeline(A_bf, B_bf, out_dtype=torch.bfloat16):
    """triton/double_channel_bwd33.py:186-201."""
    inv_K = 1.0 / A_bf.shape[-1]
    A_bf = hadamard_transform(A_bf)
    B_bf = hadamard_transform(B_bf)
    A_int8, A_scale = triton_per_row_quant_3d(A_bf)
    B_int8, B_scale = triton_per_row_quant_3d(B_bf)
    C = triton_gemm(A_int8, B_int8, A_scale, B_scale, out_dtype=out_dtype)
    return scale_bf16(C, inv_K)


def bwd_33(a: torch.Tensor, b: torch.Tensor):
    """triton/double_channel_bwd33.py:204-220."""
    return int8_gemm_pipeline(a, b, out_dtype=torch.bfloat16)
