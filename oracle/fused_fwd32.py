"""Oracle of triton/fused_triton_fwd32.py (quantise-inside-the-GEMM, 3-D x 2-D).

TEST INFRASTRUCTURE -- torch-CPU restatement, un-fused IEEE fp32.  The reference
kernel re-quantises each A tile for every N tile and each B tile for every M tile;
the values depend only on (tile, K step), so each is computed once here.
"""
import torch

from ._prims import F32, calc_diff, f32, floor_half_up, int_dot_k128, to_int8, widen

__all__ = ["fused_int8_gemm", "fwd_32", "calc_diff"]


def tile_quant_additive_eps(x: torch.Tensor, block_m: int):
    """Per (block_m x 128) group: ``amax = max|x| + 1e-5`` (additive eps),
    ``scale = 127/amax``, ``q = int8(floor(x*scale + 0.5))`` with no clamp
    (triton/fused_triton_fwd32.py:49-51 with block_m = 128 for A; :57-59 with
    block_m = 1 for B, whose tile is reduced over its 128 k's only).
    Returns q [B, M, K] and the MULTIPLIER ``scale`` [B, M/block_m, K/128]."""
    B, M, K = x.shape
    assert M % block_m == 0 and K % 128 == 0
    xf = widen(x).reshape(B, M // block_m, block_m, K // 128, 128)
    amax = xf.abs().amax(dim=(2, 4), keepdim=True) + f32(1e-5)
    scale = f32(127.0) / amax
    q = to_int8(floor_half_up(xf * scale), clamp=False).reshape(B, M, K)
    return q, scale.reshape(B, M // block_m, K // 128)


def fused_gemm_from_quant(qa, sa, qb, sb, b_block: int, out_dtype=torch.bfloat16):
    """``acc += f32(dot) / (scale_a * scale_b)`` per K step (:65); qb is [Bb, N, K]
    with Bb in {1, B}; sb is [Bb, N/b_block, K/128]."""
    B, M, K = qa.shape
    N = qb.shape[1]
    C = torch.empty((B, M, N), dtype=out_dtype)
    for b in range(B):
        bb = b if qb.shape[0] > 1 else 0
        acc = torch.zeros((M, N), dtype=F32)
        for kb in range(K // 128):
            ks = slice(kb * 128, (kb + 1) * 128)
            d = int_dot_k128(qa[b, :, ks], qb[bb, :, ks])
            sa_rows = sa[b, :, kb].repeat_interleave(128)
            sb_cols = sb[bb, :, kb].repeat_interleave(b_block)
            den = sa_rows[:, None] * sb_cols[None, :]
            acc = acc + d / den
        C[b] = acc.to(out_dtype)
    return C


def fused_int8_gemm(A_bf, B_bf):
    """triton/fused_triton_fwd32.py:71-96: A per 128x128 tile, B per (n, 128-k group)."""
    A_bf = A_bf.contiguous()
    qa, sa = tile_quant_additive_eps(A_bf, 128)
    qb, sb = tile_quant_additive_eps(B_bf[None], 1)
    return fused_gemm_from_quant(qa, sa, qb, sb, 1)


def fwd_32(a: torch.Tensor, b: torch.Tensor):
    """triton/fused_triton_fwd32.py:104-108."""
    return fused_int8_gemm(A_bf=a, B_bf=b)
