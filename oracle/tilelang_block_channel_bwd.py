"""Oracle of tilelang/block_channel_bwd.py (128x128 groups, fp32 scales,
scale product formed before the promotion).

TEST INFRASTRUCTURE -- torch-CPU restatement, un-fused IEEE fp32.
"""
import torch

from ._prims import F32, calc_diff, int_dot_k128
from .block_channel_fwd32 import block_quant

__all__ = ["triton_per_block_quant", "tl_gemm", "bwd_33", "per_block_cast_to_int8", "calc_diff"]


def triton_per_block_quant(x: torch.Tensor):
    """tilelang/block_channel_bwd.py:141-156 (unclamped, fp32 scales)."""
    return block_quant(x, clamp=False)


def tl_gemm(A_int8, B_int8, C, A_scale, B_scale):
    """tilelang/block_channel_bwd.py:47-86: ``accf += f32(acci) * (sA * sB)`` (:74-79)."""
    B, M, K = A_int8.shape
    for b in range(B):
        acc = torch.zeros((M, B_int8.shape[1]), dtype=F32)
        for kb in range(K // 128):
            ks = slice(kb * 128, (kb + 1) * 128)
            d = int_dot_k128(A_int8[b, :, ks], B_int8[b, :, ks])
            sa = A_scale[b, :, kb].to(F32).repeat_interleave(128)
            sb = B_scale[b, :, kb].to(F32).repeat_interleave(128)
            acc = acc + d * (sa[:, None] * sb[None, :])
        C[b] = acc.to(C.dtype)
    return C


def bwd_33(a, b):
    """tilelang/block_channel_bwd.py:197-225 without the sync + print."""
    A_int8, A_scale = triton_per_block_quant(a)
    B_int8, B_scale = triton_per_block_quant(b)
    C = torch.zeros(a.shape[0], a.shape[1], b.shape[1], dtype=torch.bfloat16)
    return tl_gemm(A_int8, B_int8, C, A_scale, B_scale)


def per_block_cast_to_int8(x: torch.Tensor):
    """tilelang/block_channel_bwd.py:96-104: the author's pure-torch block quantiser of this file;
    unlike the copy in block_channel_fwd.py it widens the absmax to fp32 (:100), so the scale and
    the product ``x * scale`` are fp32.  Evaluated by torch itself: ``127.0 / amax`` is
    ``amax.reciprocal() * 127.0`` there, ``round()`` is half-to-even."""
    assert x.dim() == 3
    b, m, n = x.shape
    x_view = x.view(b, m // 128, 128, n // 128, 128)
    x_amax = x_view.abs().float().amax(dim=(2, 4), keepdim=True).clamp(min=1e-4)
    scale = 127.0 / x_amax
    x_int8 = (x_view * scale).round().clamp(-127, 127).to(torch.int8)
    return x_int8.view(b, m, n), (1.0 / scale).view(b, m // 128, n // 128)
