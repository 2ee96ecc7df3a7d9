"""Drop-in for tilelang/block_channel_fwd.py: the TileLang variant of the block-channel
forward, which differs from the Triton one in three ways -- A groups are 128x256, the
stored scales are rounded through bf16, and the caller pre-allocates ``C``.
"""
from typing import Tuple

import torch

from . import ops
from ._common import StageTimer, bf16_reference_nt, calc_diff
from ._lib import COMBINE_MUL_PROD, INV_RCP_OF_SCALE, SCALE_BLOCK_K256, SCALE_ROW

__all__ = ["tl_gemm", "triton_per_block_quant", "triton_per_token_quant", "fwd_32", "per_token_cast_to_int8",
           "per_block_cast_to_int8", "assert_tl_gemm_correctness", "calc_diff"]


def triton_per_block_quant(x: torch.Tensor):
    """[B,M,N] -> (int8, fp32 [B,M/128,N/256]) with bf16-rounded scales, no clamp
    (tilelang/block_channel_fwd.py:185-203)."""
    return ops.quant_block(x.contiguous(), clamp=False, group_c=256, scale_bf16=True, inv_mode=INV_RCP_OF_SCALE)


def triton_per_token_quant(x: torch.Tensor):
    """[M,N] -> (int8, fp32 [M,1]) with bf16-rounded scales, no clamp
    (tilelang/block_channel_fwd.py:124-149)."""
    assert x.dim() == 2 and x.shape[1] % 128 == 0
    q, s = ops.quant_row(x, clamp=False, scale_bf16=True, inv_mode=INV_RCP_OF_SCALE)
    return q, s.reshape(x.shape[0], 1)


def tl_gemm(B, M, N, K, block_N, in_dtype, out_dtype, accum_dtype):
    """Returns ``kernel(A_int8, B_int8, C, A_scale, B_scale)`` writing into the caller's
    ``C`` like the jitted TileLang kernel (tilelang/block_channel_fwd.py:15-88,260-262)."""
    assert in_dtype in ["int8"], "Currently only int8 is supported"
    assert out_dtype in ["bfloat16"], "Currently only bfloat16 is supported"

    def kernel(A_int8, B_int8, C, A_scale, B_scale):
        if tuple(A_int8.shape) != (B, M, K) or tuple(B_int8.shape) != (N, K) or tuple(C.shape) != (B, M, N):
            raise ValueError("operand shapes do not match the shapes the kernel was built for")
        ops.gemm_i8_nt(A_int8, B_int8, A_scale, SCALE_BLOCK_K256, B_scale, SCALE_ROW, combine=COMBINE_MUL_PROD, out=C)
        return C

    return kernel


def fwd_32(a, b, verbose=False):
    """tilelang/block_channel_fwd.py:271-293 (sync + prints only with ``verbose``)."""
    torch.cuda.set_device(a.device)
    B, M, N, K = a.shape[0], a.shape[1], b.shape[0], a.shape[2]
    t = StageTimer(a.device, verbose)
    t.start()
    A_int8, A_scale = triton_per_block_quant(a)
    B_int8, B_scale = triton_per_token_quant(b)
    t.stop("int8 time")
    C = torch.zeros(B, M, N, device=a.device, dtype=torch.bfloat16)
    t.start()
    kernel = tl_gemm(B, M, N, K, 128, "int8", "bfloat16", "int32")
    kernel(A_int8, B_int8, C, A_scale, B_scale)
    t.stop("kernel time")
    return C


def per_token_cast_to_int8(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """[M,N] bf16 -> (int8 [M,N], bf16 [M,1]): the reference author's pure-torch per-row quantiser
    (tilelang/block_channel_fwd.py:215-220; commented out at its call sites, :255-256) as a HIP
    kernel.  Evaluated as torch evaluates it on a bf16 tensor: every intermediate in bf16,
    ``127.0 / amax`` as reciprocal times 127, round half to even, clamp +-127, so it is NOT equal to
    the Triton kernels (exact .5 ties, and the bf16 rounding of ``x * scale``)."""
    m, n = x.shape
    q, s = ops.quant_row(x, torch_arith="bf16")
    return q.view(m, n), s.to(x.dtype).view(m, -1)


def per_block_cast_to_int8(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """[B,M,N] bf16 -> (int8, bf16 [B,M/128,N/128]) (tilelang/block_channel_fwd.py:222-230);
    see :func:`per_token_cast_to_int8`."""
    assert x.dim() == 3
    q, s = ops.quant_block(x.contiguous(), torch_arith="bf16")
    return q, s.to(x.dtype)


def assert_tl_gemm_correctness(B, M, N, K, block_N, in_dtype, out_dtype, accum_dtype):
    """The reference's self-check (tilelang/block_channel_fwd.py:242-268): N(0,1) operands through the
    quantisers and the kernel ``tl_gemm`` returns, ``calc_diff`` against the bf16 product below 1e-3.
    There is no generated source to look at here (the reference asserts that TileLang produced some)."""
    kernel = tl_gemm(B, M, N, K, block_N, in_dtype, out_dtype, accum_dtype)
    a = torch.randn(B, M, K).to(torch.bfloat16).cuda()
    b = torch.randn(N, K).to(torch.bfloat16).cuda()
    A_int8, A_scale = triton_per_block_quant(a)
    B_int8, B_scale = triton_per_token_quant(b)
    C = torch.zeros(B, M, N, device="cuda", dtype=torch.bfloat16)
    kernel(A_int8, B_int8, C, A_scale, B_scale)
    diff = calc_diff(C, bf16_reference_nt(a, b))
    print(f"diff: {diff}")
    assert diff < 1e-3
    return float(diff)
