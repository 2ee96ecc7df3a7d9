"""Shared arithmetic primitives of the oracle (torch-CPU, un-fused IEEE fp32).

TEST INFRASTRUCTURE: see the package docstring.  Every product of two fp32
values and every sum below is a separate torch op, so nothing is contracted
into an FMA; divisions are IEEE-correct fp32 divisions.
"""
import torch

F32 = torch.float32


def f32(v):
    """A python scalar as the fp32 value Triton would materialise for it."""
    return torch.tensor(v, dtype=F32)


def widen(x: torch.Tensor) -> torch.Tensor:
    """bf16/fp16 -> fp32 (exact)."""
    return x.to(F32)


def floor_half_up(xs: torch.Tensor) -> torch.Tensor:
    """``tl.floor(x_scaled + 0.5)``: add then floor, two roundings, ties go up."""
    return torch.floor(xs + f32(0.5))


def to_int8(r: torch.Tensor, clamp: bool) -> torch.Tensor:
    """fp32 integer-valued tensor -> int8, with the optional [-128,127] clamp of
    triton/block_channel_fwd32.py:121,186 (absent in block_channel_bwd33.py:114).
    Values are always inside [-127,127] for finite inputs, so both agree there."""
    if clamp:
        r = torch.minimum(torch.maximum(r, f32(-128.0)), f32(127.0))
    return r.to(torch.int32).to(torch.int8)


def eps_floor(amax: torch.Tensor) -> torch.Tensor:
    """``tl.where(amax > 1e-4, amax, 1e-4)`` with the constant rounded to fp32."""
    e = f32(1e-4)
    return torch.where(amax > e, amax, e)


def int_dot_k128(aq: torch.Tensor, bq: torch.Tensor) -> torch.Tensor:
    """Exact int8 x int8 dot over ONE 128-deep K block, returned as fp32.

    aq: [..., M, 128] int8, bq: [..., N, 128] int8 -> [..., M, N] fp32 holding the
    exact integers (|sum| <= 128*127^2 = 2 064 512 < 2^24, so every partial sum of
    an fp32 GEMM is exactly representable whatever the summation order)."""
    assert aq.shape[-1] <= 1024 and bq.shape[-1] == aq.shape[-1]
    return torch.matmul(aq.to(F32), bq.to(F32).transpose(-1, -2))


def int_matmul_nt(aq: torch.Tensor, bq: torch.Tensor) -> torch.Tensor:
    """Exact int32 ``aq @ bq^T`` over the whole K (2-D operands)."""
    assert aq.dim() == 2 and bq.dim() == 2 and aq.shape[1] == bq.shape[1]
    K = aq.shape[1]
    acc = torch.zeros((aq.shape[0], bq.shape[0]), dtype=torch.int32)
    step = 1024  # 1024*127^2 < 2^24: fp32 sgemm of such a slab is exact
    for k0 in range(0, K, step):
        k1 = min(K, k0 + step)
        acc += torch.matmul(aq[:, k0:k1].to(F32), bq[:, k0:k1].to(F32).t()).to(torch.int32)
    return acc


def calc_diff(x, y):
    """1 - 2<x,y>/(|x|^2+|y|^2) in float64 (triton/block_channel_fwd32.py:244-248)."""
    x, y = x.double(), y.double()
    denominator = (x * x + y * y).sum()
    sim = 2 * (x * y).sum() / denominator
    return 1 - sim
