"""Oracle of triton/double-channle_fwd32.py (3-D x 2-D, per-row scales on both,
full-K int32 accumulation, Hadamard rotation of both operands).

TEST INFRASTRUCTURE -- torch-CPU restatement, un-fused IEEE fp32.
"""
from math import ceil

import torch

from ._prims import F32, calc_diff, f32, floor_half_up, int_matmul_nt, to_int8, widen
from .hadamard import hadamard_transform

__all__ = ["triton_per_row_quant_2d", "triton_per_row_quant_3d", "triton_gemm",
           "int8_gemm_pipeline", "fwd_32", "calc_diff", "hadamard_transform"]


def row_quant(x: torch.Tensor, BLOCK_N: int = 2048, rcp_mul: bool = False):
    """Two-pass per-row quantiser, any leading dims.

    triton/double-channle_fwd32.py:140-175 (2-D) and :229-266 (3-D):
      pass 1: per (row, BLOCK_N chunk) max|x| -> fp32 partial            :106-111
      torch : amax = clamp(max(partial), min=1e-4)                        :157-158
              scale_mul = 127.0 / amax ; scale_inv = amax / 127.0         :159-160
      pass 2: q = clamp(floor(f32(x) * scale_mul + 0.5), -128, 127)       :132-135
    The returned scale is ``scale_inv`` -- a single division, unlike the block
    kernels' ``1/(127/amax)``.  ``rcp_mul`` selects ``amax * (1/127)`` instead,
    which is how torch's GPU kernels evaluate a division by a host scalar."""
    N = x.shape[-1]
    assert N % BLOCK_N == 0, "the reference's loads are unmasked: N must be a multiple of BLOCK_N"
    xf = widen(x.contiguous())
    num_n = ceil(N / BLOCK_N)
    partial = xf.abs().reshape(*x.shape[:-1], num_n, BLOCK_N).amax(dim=-1)
    amax = torch.clamp(partial.amax(dim=-1), min=1e-4)
    scale_mul = f32(127.0) / amax
    if rcp_mul:
        scale_inv = amax * (f32(1.0) / f32(127.0))
    else:
        scale_inv = amax / f32(127.0)
    q = to_int8(floor_half_up(xf * scale_mul[..., None]), clamp=True)
    return q, scale_inv


def triton_per_row_quant_2d(x: torch.Tensor, BLOCK_N: int = 2048):
    assert x.dim() == 2
    return row_quant(x, BLOCK_N)  # s: [M]


def triton_per_row_quant_3d(x: torch.Tensor, BLOCK_N: int = 2048):
    assert x.dim() == 3
    return row_quant(x, BLOCK_N)  # s: [B, M]


def gemm_i32(A_int8, B_int8):
    """Raw accumulators of the double-channel GEMM: exact int32 over the whole K
    (triton/double-channle_fwd32.py:44,51-56).  B_int8 is [N,K] or [B,N,K]."""
    B, M, K = A_int8.shape
    out = []
    for b in range(B):
        bq = B_int8 if B_int8.dim() == 2 else B_int8[b]
        out.append(int_matmul_nt(A_int8[b], bq))
    return torch.stack(out)


def dequant_epilogue(acc_i32, sA, sB, out_dtype=torch.bfloat16):
    """``acc * sA[:, None] * sB[None, :]`` (:59): int32 -> fp32 (RNE above 2^24),
    times the row scale, times the column scale, store rounds to bf16."""
    t = acc_i32.to(F32) * sA.to(F32)[..., :, None]
    sBv = sB.to(F32)
    t = t * (sBv[None, None, :] if sBv.dim() == 1 else sBv[:, None, :])
    return t.to(out_dtype)


def scale_bf16(C, inv_K: float):
    """``C * inv_K`` on a bf16 tensor (:284,310): torch widens to fp32, multiplies by
    the python scalar rounded to fp32, and rounds the product back to bf16."""
    return (C.to(F32) * f32(inv_K)).to(C.dtype)


def triton_gemm(A_int8, B_int8, A_scale, B_scale, out_dtype=torch.bfloat16):
    """triton/double-channle_fwd32.py:62-90; A_scale [B,M], B_scale [N]."""
    assert K_ok(A_int8, B_int8)
    return dequant_epilogue(gemm_i32(A_int8, B_int8), A_scale, B_scale, out_dtype)


def K_ok(A_int8, B_int8):
    K = A_int8.shape[-1]
    return B_int8.shape[-1] == K and K % 128 == 0 and A_int8.shape[1] % 128 == 0 \
        and B_int8.shape[-2] % 128 == 0


def int8_gemm_pipeline(A_bf, B_bf, out_dtype=torch.bfloat16):
    """triton/double-channle_fwd32.py:269-285.  The final ``C * inv_K`` is a torch
    multiply of a bf16 tensor by a python float: fp32 product, second rounding to
    bf16 (:284)."""
    inv_K = 1.0 / A_bf.shape[-1]
    A_bf = hadamard_transform(A_bf)
    B_bf = hadamard_transform(B_bf)
    A_int8, A_scale = triton_per_row_quant_3d(A_bf)
    B_int8, B_scale = triton_per_row_quant_2d(B_bf)
    C = triton_gemm(A_int8, B_int8, A_scale, B_scale, out_dtype=out_dtype)
    return scale_bf16(C, inv_K)


def fwd_32(a: torch.Tensor, b: torch.Tensor):
    """triton/double-channle_fwd32.py:295-311."""
    return int8_gemm_pipeline(a, b, out_dtype=torch.bfloat16)
