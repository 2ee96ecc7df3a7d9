"""Block-channel INT8 GEMM, 3-D x 2-D: drop-in for triton/block_channel_fwd32.py.

``fwd_32(a[B,M,K], b[N,K]) -> bf16 [B,M,N] = a @ b^T`` with ``a`` quantised per
128x128 block and ``b`` per row (output channel), the per-K-block partial dots
promoted into an fp32 accumulator.  Same function names, argument meaning and
return values as the reference; the kernels are hand-written gfx950 HIP behind
``libti8.so``.
"""
import torch

from . import ops
from ._common import StageTimer, calc_diff, need_bf16_out
from ._lib import COMBINE_MUL_MUL, INV_RCP_OF_SCALE, SCALE_BLOCK128, SCALE_ROW

__all__ = ["triton_per_block_quant", "triton_per_token_quant", "triton_gemm", "int8_gemm_pipeline",
           "fwd_32", "calc_diff"]


def triton_per_block_quant(x: torch.Tensor):
    """[B,M,N] bf16 -> (int8 [B,M,N], fp32 [B,M/128,N/128]); clamped variant
    (triton/block_channel_fwd32.py:194-212).  The input is made contiguous, as there."""
    return ops.quant_block(x.contiguous(), clamp=True, inv_mode=INV_RCP_OF_SCALE)


def triton_per_token_quant(x: torch.Tensor):
    """[M,N] bf16 -> (int8 [M,N], fp32 [M,1]), one scale per row
    (triton/block_channel_fwd32.py:132-157)."""
    assert x.dim() == 2 and x.shape[1] % 128 == 0
    q, s = ops.quant_row(x, clamp=True, inv_mode=INV_RCP_OF_SCALE)
    return q, s.reshape(x.shape[0], 1)


def triton_gemm(A_int8, B_int8, A_scale, B_scale, out_dtype=torch.bfloat16, strict=False):
    """int8 [B,M,K] x int8 [N,K] with A_scale [B,M/128,K/128], B_scale [N,1] -> bf16 [B,M,N]
    (triton/block_channel_fwd32.py:68-96).  ``strict`` evaluates the promotion
    ``acc += (f32(dot)*sA)*sB`` with the reference's exact association and roundings."""
    need_bf16_out(out_dtype)
    return ops.gemm_i8_nt(A_int8, B_int8, A_scale, SCALE_BLOCK128, B_scale, SCALE_ROW,
                          combine=COMBINE_MUL_MUL, strict=strict)


def int8_gemm_pipeline(A_bf, B_bf, out_dtype=torch.bfloat16, verbose=False):
    """Quantise both operands, then the GEMM (triton/block_channel_fwd32.py:216-239).
    ``verbose=True`` restores the reference's per-call device sync + timing prints."""
    torch.cuda.set_device(A_bf.device)
    t = StageTimer(A_bf.device, verbose)
    t.start()
    A_int8, A_scale = triton_per_block_quant(A_bf)
    B_int8, B_scale = triton_per_token_quant(B_bf)
    t.stop("int8 time")
    t.start()
    C = triton_gemm(A_int8, B_int8, A_scale, B_scale, out_dtype=out_dtype)
    t.stop("kernel time")
    return C


def fwd_32(a: torch.Tensor, b: torch.Tensor):
    """triton/block_channel_fwd32.py:252-254."""
    return int8_gemm_pipeline(a, b, out_dtype=torch.bfloat16)
