"""Oracle of the INT8 linear layer built from the reference's fwd_32 / bwd_33
pieces: Y = X W^T, dX = dY W, dW = dY^T X, plus the quantisation modes the
benchmark configurations name.

TEST INFRASTRUCTURE -- torch-CPU, un-fused IEEE fp32.  The reference has no
linear-layer wrapper; its two entry points are NT GEMMs contracting over the last
dim of both operands (triton/block_channel_fwd32.py:252-254,
triton/block_channel_bwd33.py:175-177), so the layer is wired as

    Y  = fwd_32(X [B,M,K],      W   [N,K])
    dX = fwd_32(dY[B,M,N],      W^T [K,N])
    dW = bwd_33(dY^T [1,N,B*M], X^T [1,K,B*M])[0]      (tokens flattened)

``scheme``:
  "block_channel"  reference literal: the 3-D operand in 128x128 blocks, the 2-D
                   operand per row; bwd_33 both in blocks.
  "row_block"      the wording of the benchmark configs ("per-token X, per
                   128x128-block W"): a per row, b per block, for all three GEMMs:
                   acc += (f32(dot_kb) * sA[m]) * sB[nb, kb].
  "double_channel" per-row scales on both operands, full-K int32 accumulation
                   (triton/double-channle_fwd32.py); ``hadamard="full"`` adds the
                   reference's full-length rotation and its 1/K factor.
``hadamard=128`` (block_channel / row_block): block-diagonal H_128 along the
contraction dim of both operands before quantisation, result times exactly 2^-7.
"""
import torch

from ._prims import F32, f32, int_dot_k128
from . import block_channel_fwd32 as bcf
from . import block_channel_bwd33 as bcb
from . import double_channel_fwd32 as dcf
from .hadamard import hadamard128, hadamard_transform

ROW, BLOCK = "row", "block"


def _expand(s, mode, rows, kb):
    """Scale of every row of a 2-D operand at K block ``kb`` as an fp32 vector."""
    if mode == ROW:
        return s.reshape(rows).to(F32)
    return s[:, kb].to(F32).repeat_interleave(128)[:rows]   # row r uses block r // 128 (rows need not fill the last block)


def gemm_scaled(Aq, sA, modeA, Bq, sB, modeB, out_scale=None, out_dtype=torch.bfloat16, with_magnitude=False):
    """2-D NT GEMM with per-K-block promotion, literal association
    ``acc = acc + (f32(dot) * sa) * sb`` for any mix of ROW / BLOCK descriptors.
    ``out_scale`` (a power of two) multiplies the fp32 accumulator before the store.
    ``with_magnitude`` also returns sum_kb |term_kb| (fp32, scaled like the result): what a
    different association of the same fp32 sum can move the result by is a few 2^-24 of it."""
    M, K = Aq.shape
    N = Bq.shape[0]
    acc = torch.zeros((M, N), dtype=F32)
    mag = torch.zeros((M, N), dtype=F32)
    for kb in range(K // 128):
        ks = slice(kb * 128, (kb + 1) * 128)
        d = int_dot_k128(Aq[:, ks], Bq[:, ks])
        t = d * _expand(sA, modeA, M, kb)[:, None]
        t = t * _expand(sB, modeB, N, kb)[None, :]
        acc = acc + t
        if with_magnitude:
            mag = mag + t.abs()
    if out_scale is not None:
        acc = acc * f32(out_scale)
        mag = mag * f32(out_scale)
    return (acc.to(out_dtype), mag) if with_magnitude else acc.to(out_dtype)


def quant2d(x, mode, clamp):
    """2-D operand -> (q, s) with s [rows,1]->[rows] for ROW, [rows/128, K/128] for BLOCK."""
    if mode == ROW:
        q, s = bcf.token_quant(x, clamp)
        return q, s.reshape(-1)
    q, s = bcf.block_quant(x[None], clamp)
    return q[0], s[0]


def nt_gemm(a, b, modeA, modeB, hadamard=None):
    """bf16 a [M,K], b [N,K] -> bf16 a @ b^T through the quantised path."""
    out_scale = None
    if hadamard == 128:
        a, b = hadamard128(a), hadamard128(b)
        out_scale = 2.0 ** -7
    # clamp or not is value-neutral on finite data (see block_channel_bwd33.py:114)
    qa, sa = quant2d(a, modeA, clamp=True)
    qb, sb = quant2d(b, modeB, clamp=True)
    return gemm_scaled(qa, sa, modeA, qb, sb, modeB, out_scale)


def double_channel_nt(a, b, hadamard=None, rcp_mul=False):
    """Per-row x per-row NT GEMM with int32 accumulation (2-D operands)."""
    inv_K = 1.0 / a.shape[-1]
    if hadamard == "full":
        a, b = hadamard_transform(a), hadamard_transform(b)
    # the chunk width only splits the absmax reduction; 128 lifts the reference's
    # multiple-of-2048 restriction without changing any value
    qa, sa = dcf.row_quant(a, BLOCK_N=128, rcp_mul=rcp_mul)
    qb, sb = dcf.row_quant(b, BLOCK_N=128, rcp_mul=rcp_mul)
    C = dcf.dequant_epilogue(dcf.gemm_i32(qa[None], qb), sa[None], sb)[0]
    if hadamard == "full":
        C = dcf.scale_bf16(C, inv_K)
    return C


def _pad_rows(x, multiple=128):
    """Zero-pad rows to the 128-row tile: zeros change no absmax, an all-padding block gets
    the epsilon scale and zero codes, and padded tokens add nothing to dW."""
    T = x.shape[0]
    Tp = -(-T // multiple) * multiple
    if Tp == T:
        return x
    out = x.new_zeros((Tp, x.shape[1]))
    out[:T] = x
    return out


def linear_fwd_bwd(X, W, dY, scheme="block_channel", hadamard=None):
    """Returns (Y, dX, dW) for X [B,M,K] (or [M,K]), W [N,K], dY like Y.  Token counts that
    are not multiples of 128 are zero-padded (skinny / ragged M) and the outputs cut back."""
    squeeze = X.dim() == 2
    if squeeze:
        X, dY = X[None], dY[None]
    B, M, K = X.shape
    N = W.shape[0]
    T = B * M
    Xf, dYf = _pad_rows(X.reshape(T, K)), _pad_rows(dY.reshape(T, N))
    if scheme == "double_channel":
        Y = double_channel_nt(Xf, W, hadamard)
        dX = double_channel_nt(dYf, W.t().contiguous(), hadamard)
        dW = double_channel_nt(dYf.t().contiguous(), Xf.t().contiguous(), hadamard)
    else:
        ma, mb, mbwd = (BLOCK, ROW, BLOCK) if scheme == "block_channel" else (ROW, BLOCK, BLOCK)
        if scheme not in ("block_channel", "row_block"):
            raise ValueError(scheme)
        mabwd = BLOCK if scheme == "block_channel" else ROW
        Y = nt_gemm(Xf, W, ma, mb, hadamard)
        dX = nt_gemm(dYf, W.t().contiguous(), ma, mb, hadamard)
        dW = nt_gemm(dYf.t().contiguous(), Xf.t().contiguous(), mabwd, mbwd, hadamard)
    Y, dX = Y[:T].reshape(B, M, N), dX[:T].reshape(B, M, K)
    if squeeze:
        Y, dX = Y[0], dX[0]
    return Y, dX, dW
