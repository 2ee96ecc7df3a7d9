"""Oracle of tilelang/block_channel_fwd.py (128x256 A groups, bf16-rounded scales).

TEST INFRASTRUCTURE -- torch-CPU restatement, un-fused IEEE fp32.
"""
from typing import Tuple

import torch

from ._prims import F32, calc_diff, int_dot_k128
from .block_channel_fwd32 import block_quant, token_quant

__all__ = ["triton_per_block_quant", "triton_per_token_quant", "tl_gemm", "fwd_32",
           "per_token_cast_to_int8", "per_block_cast_to_int8", "calc_diff"]


def triton_per_block_quant(x: torch.Tensor):
    """tilelang/block_channel_fwd.py:185-203: 128x256 groups (:187-188), no clamp
    (:177), scale stored to a bf16 tensor and widened (:191,203)."""
    return block_quant(x.contiguous(), clamp=False, block_m=128, block_n=256,
                       scale_dtype=torch.bfloat16)


def triton_per_token_quant(x: torch.Tensor):
    """tilelang/block_channel_fwd.py:124-149: no clamp (:115), bf16-stored scale (:133,149)."""
    return token_quant(x.contiguous(), clamp=False, scale_dtype=torch.bfloat16)


def tl_gemm(A_int8, B_int8, C, A_scale, B_scale):
    """The TileLang kernel body, tilelang/block_channel_fwd.py:46-86, writing into
    the caller's ``C`` (:260-262).  Per K block the scale PRODUCT is formed first
    (:75) and then ``accf += f32(acci) * (sA[b, mb, kb//2] * sB[n])`` (:79-81)."""
    B, M, K = A_int8.shape
    N = B_int8.shape[0]
    sB = B_scale.reshape(N).to(F32)
    for b in range(B):
        acc = torch.zeros((M, N), dtype=F32)
        for kb in range(K // 128):
            ks = slice(kb * 128, (kb + 1) * 128)
            d = int_dot_k128(A_int8[b, :, ks], B_int8[:, ks])
            sa_rows = A_scale[b, :, (kb * 128) // 256].to(F32).repeat_interleave(128)
            sc = sa_rows[:, None] * sB[None, :]
            acc = acc + d * sc
        C[b] = acc.to(C.dtype)
    return C


def fwd_32(a, b):
    """tilelang/block_channel_fwd.py:271-293 without the sync + print."""
    A_int8, A_scale = triton_per_block_quant(a)
    B_int8, B_scale = triton_per_token_quant(b)
    C = torch.zeros(a.shape[0], a.shape[1], b.shape[0], dtype=torch.bfloat16)
    return tl_gemm(A_int8, B_int8, C, A_scale, B_scale)


def per_token_cast_to_int8(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """tilelang/block_channel_fwd.py:215-220: the author's pure-torch quantiser
    (bf16 arithmetic, round-half-to-even, clamp +-127); NOT equal to the Triton
    kernels on exact .5 ties.  Kept because it documents the intent."""
    m, n = x.shape
    x_amax = x.abs().amax(dim=1, keepdim=True).clamp(min=1e-4)
    scale = 127.0 / x_amax
    x_int8 = (x * scale).round().clamp(-127, 127).to(torch.int8)
    return x_int8.view(m, n), (1.0 / scale).view(m, -1)


def per_block_cast_to_int8(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """tilelang/block_channel_fwd.py:222-230."""
    assert x.dim() == 3
    b, m, n = x.shape
    x_view = x.view(b, m // 128, 128, n // 128, 128)
    x_amax = x_view.abs().amax(dim=(2, 4), keepdim=True).clamp(min=1e-4)
    scale = 127.0 / x_amax
    x_int8 = (x_view * scale).round().clamp(-127, 127).to(torch.int8)
    return x_int8.view(b, m, n), (1.0 / scale).view(b, m // 128, n // 128)
