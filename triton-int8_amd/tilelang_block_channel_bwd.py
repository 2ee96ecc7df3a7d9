"""Drop-in for tilelang/block_channel_bwd.py: 3-D x 3-D block-channel GEMM whose
promotion multiplies by the scale PRODUCT (``acc += f32(dot) * (sA*sB)``)."""
import torch

from . import ops
from typing import Tuple

from ._common import StageTimer, bf16_reference_nt, calc_diff, ceildiv
from ._lib import COMBINE_MUL_PROD, INV_RCP_OF_SCALE, SCALE_BLOCK128

__all__ = ["tl_gemm", "triton_per_block_quant", "bwd_33", "per_block_cast_to_int8", "assert_tl_gemm_correctness", "ceildiv",
           "calc_diff"]


def triton_per_block_quant(x: torch.Tensor, out="like"):
    """tilelang/block_channel_bwd.py:141-156 (128x128 groups, fp32 scales, no clamp)."""
    return ops.quant_block(x, clamp=False, inv_mode=INV_RCP_OF_SCALE, out=out)


def tl_gemm(B, M, N, K, block_N, in_dtype, out_dtype, accum_dtype):
    """Returns ``kernel(A_int8, B_int8, C, A_scale, B_scale)`` (tilelang/block_channel_bwd.py:16-88)."""
    assert in_dtype in ["int8"], "Currently only int8 is supported"
    assert out_dtype in ["bfloat16"], "Currently only bfloat16 is supported"

    def kernel(A_int8, B_int8, C, A_scale, B_scale):
        if tuple(A_int8.shape) != (B, M, K) or tuple(B_int8.shape) != (B, N, K) or tuple(C.shape) != (B, M, N):
            raise ValueError("operand shapes do not match the shapes the kernel was built for")
        ops.gemm_i8_nt(A_int8, B_int8, A_scale, SCALE_BLOCK128, B_scale, SCALE_BLOCK128, combine=COMBINE_MUL_PROD, out=C)
        return C

    return kernel


def bwd_33(a, b, verbose=False):
    """tilelang/block_channel_bwd.py:197-225."""
    torch.cuda.set_device(a.device)
    B, M, N, K = a.shape[0], a.shape[1], b.shape[1], a.shape[2]
    t = StageTimer(a.device, verbose)
    t.start()
    A_int8, A_scale = triton_per_block_quant(a, out="contiguous")
    B_int8, B_scale = triton_per_block_quant(b, out="contiguous")
    t.stop("to int8 time")
    C = torch.zeros(B, M, N, device=a.device, dtype=torch.bfloat16)
    t.start()
    kernel = tl_gemm(B, M, N, K, 128, "int8", "bfloat16", "int32")
    kernel(A_int8, B_int8, C, A_scale, B_scale)
    t.stop("kernel time")
    return C


def per_block_cast_to_int8(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """[B,M,N] bf16 -> (int8, fp32 [B,M/128,N/128]): the pure-torch block quantiser of
    tilelang/block_channel_bwd.py:96-104 (unused at its call sites, :201-202) as a HIP kernel.  This
    copy takes the absmax in fp32, so scale and product are fp32: reciprocal(amax) * 127, round half
    to even, clamp +-127, returned scale reciprocal(scale)."""
    assert x.dim() == 3
    return ops.quant_block(x.contiguous(), torch_arith="f32")


def assert_tl_gemm_correctness(B, M, N, K, block_N, in_dtype, out_dtype, accum_dtype):
    """The reference's self-check (tilelang/block_channel_bwd.py:165-193): N(0,1) operands, both 3-D,
    ``calc_diff`` against the bf16 product below 1e-3."""
    kernel = tl_gemm(B, M, N, K, block_N, in_dtype, out_dtype, accum_dtype)
    a = torch.randn(B, M, K).to(torch.bfloat16).cuda()
    b = torch.randn(B, N, K).to(torch.bfloat16).cuda()
    A_int8, A_scale = triton_per_block_quant(a.clone())
    B_int8, B_scale = triton_per_block_quant(b.clone())
    C = torch.zeros(B, M, N, device="cuda", dtype=torch.bfloat16)
    kernel(A_int8, B_int8, C, A_scale, B_scale)
    diff = calc_diff(C, bf16_reference_nt(a, b))
    print(f"diff: {diff}")
    assert diff < 1e-3
    return float(diff)
