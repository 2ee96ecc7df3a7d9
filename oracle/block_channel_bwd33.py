"""Oracle of triton/block_channel_bwd33.py (3-D x 3-D, both operands 128x128 blocks).

TEST INFRASTRUCTURE -- torch-CPU restatement, un-fused IEEE fp32.
"""
import torch

from ._prims import F32, calc_diff, int_dot_k128
from .block_channel_fwd32 import block_quant

__all__ = ["triton_per_block_quant", "triton_gemm", "int8_gemm_pipeline", "bwd_33", "calc_diff"]


def triton_per_block_quant(x: torch.Tensor):
    """triton/block_channel_bwd33.py:87-138: the unclamped block quantiser (:114).

    The reference does not make ``x`` contiguous and allocates ``q`` with
    ``empty_like`` (:126), so a transposed view in gives a transposed view out;
    values do not depend on strides, which is all the oracle models."""
    q, s = block_quant(x, clamp=False)
    if not x.is_contiguous() and x.transpose(1, 2).is_contiguous():
        q = q.transpose(1, 2).contiguous().transpose(1, 2)  # same strides as the input view
    return q, s


def triton_gemm(A_int8, B_int8, A_scale, B_scale, out_dtype=torch.bfloat16):
    """int8_gemm_kernel, triton/block_channel_bwd33.py:17-56.

    ``acc = acc + (f32(dot) * sA[b, mb, kb]) * sB[b, nb, kb]`` per K block (:53)."""
    B, M, K = A_int8.shape
    N = B_int8.shape[1]
    assert B_int8.shape[0] == B and B_int8.shape[2] == K
    assert K % 128 == 0 and M % 128 == 0 and N % 128 == 0
    C = torch.empty((B, M, N), dtype=out_dtype)
    for b in range(B):
        acc = torch.zeros((M, N), dtype=F32)
        for kb in range(K // 128):
            ks = slice(kb * 128, (kb + 1) * 128)
            d = int_dot_k128(A_int8[b, :, ks], B_int8[b, :, ks])
            sa = A_scale[b, :, kb].to(F32).repeat_interleave(128)
            sb = B_scale[b, :, kb].to(F32).repeat_interleave(128)
            t = d * sa[:, None]
            t = t * sb[None, :]
            acc = acc + t
        C[b] = acc.to(out_dtype)
    return C


def int8_gemm_pipeline(A_bf, B_bf, out_dtype=torch.bfloat16):
    """triton/block_channel_bwd33.py:148-172 without its per-call sync + print."""
    A_int8, A_scale = triton_per_block_quant(A_bf)
    B_int8, B_scale = triton_per_block_quant(B_bf)
    return triton_gemm(A_int8, B_int8, A_scale, B_scale, out_dtype=out_dtype)


def bwd_33(a: torch.Tensor, b: torch.Tensor):
    """triton/block_channel_bwd33.py:175-177: C[B,M,N] = a[B,M,K] @ b[B,N,K]^T."""
    return int8_gemm_pipeline(a, b, out_dtype=torch.bfloat16)
