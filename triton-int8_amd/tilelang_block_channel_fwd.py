"""Drop-in for tilelang/block_channel_fwd.py: the TileLang variant of the block-channel
forward, which differs from the Triton one in three ways -- A groups are 128x256, the
stored scales are rounded through bf16, and the caller pre-allocates ``C``.
"""
from typing import Tuple

import torch

from . import ops
from ._common import StageTimer, calc_diff
from ._lib import COMBINE_MUL_PROD, INV_RCP_OF_SCALE, SCALE_BLOCK_K256, SCALE_ROW

__all__ = ["tl_gemm", "triton_per_block_quant", "triton_per_token_quant", "fwd_32", "per_token_cast_to_int8",
           "per_block_cast_to_int8", "calc_diff"]


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
    """The reference author's pure-torch quantiser (tilelang/block_channel_fwd.py:215-220),
    unused at its call sites (:255-256); round-half-to-even and clamp +-127, so it is NOT
    equal to the kernels on exact .5 ties.  Plain torch ops on whatever device ``x`` is on."""
    m, n = x.shape
    x_amax = x.abs().amax(dim=1, keepdim=True).clamp(min=1e-4)
    scale = 127.0 / x_amax
    x_int8 = (x * scale).round().clamp(-127, 127).to(torch.int8)
    return x_int8.view(m, n), (1.0 / scale).view(m, -1)


def per_block_cast_to_int8(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """tilelang/block_channel_fwd.py:222-230; see :func:`per_token_cast_to_int8`."""
    assert x.dim() == 3
    b, m, n = x.shape
    x_view = x.view(b, m // 128, 128, n // 128, 128)
    x_amax = x_view.abs().amax(dim=(2, 4), keepdim=True).clamp(min=1e-4)
    scale = 127.0 / x_amax
    x_int8 = (x_view * scale).round().clamp(-127, 127).to(torch.int8)
    return x_int8.view(b, m, n), (1.0 / scale).view(b, m // 128, n // 128)
