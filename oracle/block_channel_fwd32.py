"""Oracle of triton/block_channel_fwd32.py (3-D x 2-D, a: 128x128 blocks, b: rows).

TEST INFRASTRUCTURE -- torch-CPU restatement, un-fused IEEE fp32.
"""
import torch

from ._prims import (F32, calc_diff, eps_floor, f32, floor_half_up, int_dot_k128,
                     to_int8, widen)

__all__ = ["triton_per_block_quant", "triton_per_token_quant", "triton_gemm",
           "int8_gemm_pipeline", "fwd_32", "calc_diff"]


def block_quant(x: torch.Tensor, clamp: bool, block_m: int = 128, block_n: int = 128,
                scale_dtype=F32):
    """Per (block_m x block_n) tile absmax quantisation of a [B, M, N] tensor.

    per_block_quant_kernel, triton/block_channel_fwd32.py:160-192:
      amax = max|x| (fp32)            :181
      amax = amax > 1e-4 ? amax : 1e-4 :182
      scale = 127.0 / amax            :183
      q = clamp(floor(x*scale + 0.5)) :184-186
      stored scale = 1.0 / scale      :190
    ``scale_dtype`` bf16 reproduces the TileLang copy, which stores the scale
    into a bf16 tensor and widens it again (tilelang/block_channel_fwd.py:191,203).
    """
    assert x.dim() == 3
    B, M, N = x.shape
    assert M % block_m == 0 and N % block_n == 0
    xf = widen(x).reshape(B, M // block_m, block_m, N // block_n, block_n)
    amax = xf.abs().amax(dim=(2, 4), keepdim=True)
    amax = eps_floor(amax)
    scale = f32(127.0) / amax
    q = to_int8(floor_half_up(xf * scale), clamp).reshape(B, M, N)
    s = (f32(1.0) / scale).reshape(B, M // block_m, N // block_n)
    if scale_dtype != F32:
        s = s.to(scale_dtype).to(F32)
    return q, s


def triton_per_block_quant(x: torch.Tensor):
    """triton/block_channel_fwd32.py:194-212 (clamped; input made contiguous)."""
    return block_quant(x.contiguous(), clamp=True)


def token_quant(x: torch.Tensor, clamp: bool, scale_dtype=F32):
    """Per-row (whole row) absmax quantisation of a 2-D tensor.

    per_token_quant_kernel, triton/block_channel_fwd32.py:101-129: same formula as
    the block kernel with a row-wise amax (:118-123) and ``s = 1/scale`` (:127)."""
    assert x.dim() == 2 and x.shape[1] % 128 == 0
    xf = widen(x)
    amax = eps_floor(xf.abs().amax(dim=1, keepdim=True))
    scale = f32(127.0) / amax
    q = to_int8(floor_half_up(xf * scale), clamp)
    s = f32(1.0) / scale
    if scale_dtype != F32:
        s = s.to(scale_dtype).to(F32)
    return q, s  # s: [M, 1]


def triton_per_token_quant(x: torch.Tensor):
    """triton/block_channel_fwd32.py:132-157."""
    return token_quant(x.contiguous(), clamp=True)


def triton_gemm(A_int8, B_int8, A_scale, B_scale, out_dtype=torch.bfloat16):
    """int8_gemm_kernel, triton/block_channel_fwd32.py:23-66.

    acc (fp32) starts at 0; for each 128-deep K block IN ORDER
    ``acc = acc + (f32(dot) * sA[b, mb, kb]) * sB[n]`` (:63, left-to-right), then
    the store casts to ``out_dtype`` with round-to-nearest-even (:65-66)."""
    B, M, K = A_int8.shape
    N = B_int8.shape[0]
    assert B_int8.shape[1] == K and K % 128 == 0 and M % 128 == 0 and N % 128 == 0
    assert A_scale.shape == (B, M // 128, K // 128)
    sB = B_scale.reshape(N).to(F32)
    C = torch.empty((B, M, N), dtype=out_dtype)
    for b in range(B):
        acc = torch.zeros((M, N), dtype=F32)
        for kb in range(K // 128):
            d = int_dot_k128(A_int8[b, :, kb * 128:(kb + 1) * 128], B_int8[:, kb * 128:(kb + 1) * 128])
            sa_rows = A_scale[b, :, kb].to(F32).repeat_interleave(128)  # [M]
            t = d * sa_rows[:, None]
            t = t * sB[None, :]
            acc = acc + t
        C[b] = acc.to(out_dtype)
    return C


def int8_gemm_pipeline(A_bf, B_bf, out_dtype=torch.bfloat16):
    """triton/block_channel_fwd32.py:216-239 without its per-call sync + print."""
    A_int8, A_scale = triton_per_block_quant(A_bf)
    B_int8, B_scale = triton_per_token_quant(B_bf)
    return triton_gemm(A_int8, B_int8, A_scale, B_scale, out_dtype=out_dtype)


def fwd_32(a: torch.Tensor, b: torch.Tensor):
    """triton/block_channel_fwd32.py:252-254: C[B,M,N] = a[B,M,K] @ b[N,K]^T."""
    return int8_gemm_pipeline(a, b, out_dtype=torch.bfloat16)
