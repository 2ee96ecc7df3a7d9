"""Block-channel INT8 GEMM, 3-D x 3-D: drop-in for triton/block_channel_bwd33.py.

``bwd_33(a[B,M,K], b[B,N,K]) -> bf16 [B,M,N] = a[b] @ b[b]^T`` with both operands
quantised per 128x128 block.  Operands may be transposed views (the backward of a
linear layer passes ``dY^T`` and ``X^T``): a 128x128 block quantisation commutes
with transposition, so the quantiser reads the underlying memory coalesced and
writes the int8 tensor in the K-contiguous layout the GEMM consumes.
"""
import torch

from . import ops
from ._common import StageTimer, calc_diff, need_bf16_out
from ._lib import COMBINE_MUL_MUL, INV_RCP_OF_SCALE, SCALE_BLOCK128

__all__ = ["triton_per_block_quant", "triton_gemm", "int8_gemm_pipeline", "bwd_33", "calc_diff"]


def triton_per_block_quant(x: torch.Tensor, out="like"):
    """Unclamped block quantiser (triton/block_channel_bwd33.py:122-138).  Like the
    reference it honours the strides of ``x`` and returns ``q`` with the same strides
    (``empty_like``); ``out="contiguous"`` returns it contiguous instead."""
    return ops.quant_block(x, clamp=False, inv_mode=INV_RCP_OF_SCALE, out=out)


def triton_gemm(A_int8, B_int8, A_scale, B_scale, out_dtype=torch.bfloat16, strict=False):
    """int8 [B,M,K] x int8 [B,N,K], scales [B,M/128,K/128] and [B,N/128,K/128]
    (triton/block_channel_bwd33.py:58-84)."""
    need_bf16_out(out_dtype)
    return ops.gemm_i8_nt(A_int8, B_int8, A_scale, SCALE_BLOCK128, B_scale, SCALE_BLOCK128,
                          combine=COMBINE_MUL_MUL, strict=strict)


def int8_gemm_pipeline(A_bf, B_bf, out_dtype=torch.bfloat16, verbose=False):
    """triton/block_channel_bwd33.py:148-172 (sync + prints only with ``verbose``)."""
    torch.cuda.set_device(A_bf.device)
    t = StageTimer(A_bf.device, verbose)
    t.start()
    A_int8, A_scale = triton_per_block_quant(A_bf, out="contiguous")
    B_int8, B_scale = triton_per_block_quant(B_bf, out="contiguous")
    t.stop("int8 time")
    t.start()
    C = triton_gemm(A_int8, B_int8, A_scale, B_scale, out_dtype=out_dtype)
    t.stop("kernel time")
    return C


def bwd_33(a: torch.Tensor, b: torch.Tensor):
    """triton/block_channel_bwd33.py:175-177."""
    return int8_gemm_pipeline(a, b, out_dtype=torch.bfloat16)
