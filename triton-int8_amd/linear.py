"""INT8 linear layer built on the reference's two entry points.

The reference stops at ``fwd_32`` / ``bwd_33`` (NT GEMMs that contract over the last
dim of both operands) and never shows how a linear layer maps onto them.  The wiring
used here is

    Y  = fwd_32(X [B,M,K],       W   [N,K])
    dX = fwd_32(dY[B,M,N],       W^T [K,N])
    dW = bwd_33(dY^T [1,N,B*M],  X^T [1,K,B*M])[0]

``scheme``
  "block_channel"   reference literal (triton/block_channel_fwd32.py:221-222,
                    triton/block_channel_bwd33.py:153-154): the 3-D operand per 128x128
                    block, the 2-D operand per row; bwd_33 both per block.
  "row_block"       "per-token activations, per-128x128-block weights": the first operand
                    of every GEMM per row, the second per block.
  "double_channel"  per-row scales on both operands, int32 accumulation over the whole K
                    (triton/double-channle_fwd32.py), optional full-length Hadamard.
``hadamard=128`` ("block_channel" / "row_block"): both operands of every GEMM are rotated
by a block-diagonal H_128 along the contraction dim before quantisation and the result is
multiplied by 2^-7 (exact) in the GEMM epilogue.

MI355X-specific data flow: a 128x128 block quantisation commutes with transposition, so
X and dY are each read ONCE by a quantiser that writes both the int8 tensor and its
transpose (the K-contiguous operand of the dW GEMM); W^T is quantised per row by a
column-absmax kernel that never materialises W^T in bf16.
"""
import torch

from . import ops
from ._lib import (COMBINE_MUL_MUL, INV_AMAX_DIV_127, INV_RCP_OF_SCALE, SCALE_BLOCK128, SCALE_ROW)

__all__ = ["quantize_weight", "linear_forward", "linear_backward", "linear_fwd_bwd", "pad_tokens", "Int8LinearFunction", "Int8Linear", "SCHEMES"]

SCHEMES = ("block_channel", "row_block", "double_channel")


def _check(scheme, hadamard):
    if scheme not in SCHEMES:
        raise ValueError(f"unknown scheme {scheme!r}; expected one of {SCHEMES}")
    if scheme == "double_channel" and hadamard not in (None, "full"):
        raise ValueError("double_channel supports hadamard=None or 'full'")
    if scheme != "double_channel" and hadamard not in (None, 128):
        raise ValueError(f"{scheme} supports hadamard=None or 128")


def _h128(x2d):
    return ops.fwht(x2d, 128)


def _live_rows(a_q, tokens):
    """Rows of the (zero-padded, 128-row-quantised) token operand that the GEMM has to multiply:
    with few tokens the GEMM takes any multiple of 32 rows, and the padding rows are zeros whose
    products nobody reads."""
    rows = a_q.shape[0]
    if tokens is None or rows > 256 or ops.GEMM_PATH in ("tiled", "large") or a_q.shape[1] > 32768:
        return rows
    return min(rows, -(-tokens // 32) * 32)


def _deferred(gemms, problem):
    """Queue one 2-D GEMM for the launch that ends a whole step (``linear_fwd_bwd``); returns its output tensor,
    which holds the result once that launch has run."""
    M, N = problem["A"].shape[0], problem["B"].shape[0]
    problem["out"] = torch.empty((M, N), dtype=torch.bfloat16, device=problem["A"].device)
    gemms.append(problem)
    return problem["out"]


def _gemm_bc(a_q, a_s, a_mode, b_q, b_s, b_mode, out_scale=1.0, tokens=None, gemms=None):
    """2-D operands through the batched block-channel GEMM (batch of one); with ``gemms`` (a list) the GEMM is
    queued there instead of launched."""
    if gemms is not None:
        return _deferred(gemms, dict(A=a_q, B=b_q, sA=a_s.reshape(-1) if a_mode == SCALE_ROW else a_s, modeA=a_mode,
                                     sB=b_s.reshape(-1) if b_mode == SCALE_ROW else b_s, modeB=b_mode, out_scale=out_scale))
    rows = _live_rows(a_q, tokens)
    a_q = a_q[:rows]
    a_s3 = a_s[:rows].reshape(1, -1) if a_mode == SCALE_ROW else a_s[None]
    return ops.gemm_i8_nt(a_q[None], b_q, a_s3, a_mode, b_s, b_mode, combine=COMBINE_MUL_MUL,
                          out_scale=out_scale)[0]


def _gemm_dc(a_q, a_s, b_q, b_s, post_scale=0.0, tokens=None, gemms=None):
    if gemms is not None:
        return _deferred(gemms, dict(A=a_q, B=b_q, sA=a_s.reshape(-1), modeA=SCALE_ROW, sB=b_s.reshape(-1), modeB=SCALE_ROW,
                                     acc_i32_full=True, post_scale=post_scale))
    rows = _live_rows(a_q, tokens)
    return ops.gemm_i8_nt(a_q[:rows][None], b_q, a_s[:rows].reshape(1, -1), SCALE_ROW, b_s, SCALE_ROW, acc_i32_full=True,
                          post_scale=post_scale)[0]


# Quantise an operand by rows and by columns in one launch sequence (ops.quant_row_col_t) where a
# step needs both; False falls back to separate quant_row / quant_col_t calls (same bits).
FUSE_ROW_COL = True


def _row_col(x, **kw):
    if FUSE_ROW_COL:
        return ops.quant_row_col_t(x, **kw)
    q, s = ops.quant_row(x, **kw)
    qT, sT = ops.quant_col_t(x, **kw)
    return q, s, qT, sT


def _rotated_row_quant(x, hadamard):
    """The double-channel scheme's per-row quantiser, behind the full-length rotation when ``hadamard`` is "full" (one
    pass: the rotated bf16 tensor is not written)."""
    if hadamard == "full":
        return ops.fwht_quant_row(x, clamp=True, inv_mode=INV_AMAX_DIV_127)
    return ops.quant_row(x, clamp=True, inv_mode=INV_AMAX_DIV_127)


def quantize_weight(W, scheme="block_channel", hadamard=None):
    """The forward GEMM's view of W [N, K]: ``(Wq int8 [N, K], scales)`` in the scheme's layout (per
    output channel, or 128x128 blocks for "row_block"; rotated first when ``hadamard`` asks).
    A forward-only caller (inference) computes it once per weight update and hands it to
    :func:`linear_forward` as ``wq``."""
    _check(scheme, hadamard)
    if scheme == "block_channel":
        return ops.quant_row(W, clamp=True, hadamard128=(hadamard == 128))
    if scheme == "row_block":
        wq, ws = ops.quant_block_had128(W[None], clamp=True) if hadamard == 128 else ops.quant_block(W[None], clamp=True)
        return wq[0], ws[0]
    return _rotated_row_quant(W, hadamard)


def linear_forward(X2, W, scheme="block_channel", hadamard=None, need_backward=True, wq=None, tokens=None, xq=None, gemms=None):
    """X2 bf16 [T, K] (tokens flattened), W bf16 [N, K] -> (Y bf16 [T, N], saved) where
    ``saved`` holds what the backward can reuse: operands the forward quantises anyway are
    quantised for the backward GEMMs in the same pass (transposed copies, column-wise scales)
    unless ``need_backward`` is false.  ``wq`` = :func:`quantize_weight` of W computed earlier
    (forward-only use; W itself is then not read).  ``tokens`` = number of real rows of X2 when the
    caller has zero-padded it: with few tokens the GEMM skips the padding rows.  ``xq`` = ``(q, qT, s)`` of
    ``ops.quant_block(X2[None], with_transpose=True)`` computed earlier ("block_channel" without rotation only).
    ``gemms`` = a list: the GEMM is queued there instead of launched (see :func:`linear_fwd_bwd`)."""
    _check(scheme, hadamard)
    saved = {}
    if wq is not None and need_backward:
        raise ValueError("a pre-quantised weight serves the forward only")
    if scheme == "block_channel":
        if hadamard == 128:
            q, s = ops.quant_block_had128(X2[None], clamp=True)
            wq, ws = wq if wq is not None else quantize_weight(W, scheme, hadamard)
            return _gemm_bc(q[0], s[0], SCALE_BLOCK128, wq, ws, SCALE_ROW, 2.0 ** -7, tokens=tokens, gemms=gemms), saved
        if not need_backward:
            q, s = ops.quant_block(X2[None], clamp=True)
            wq, ws = wq if wq is not None else quantize_weight(W, scheme, hadamard)
            return _gemm_bc(q[0], s[0], SCALE_BLOCK128, wq, ws, SCALE_ROW, tokens=tokens, gemms=gemms), saved
        q, qT, s = xq if xq is not None else ops.quant_block(X2[None], clamp=True, with_transpose=True)
        saved["XqT"], saved["Xs"] = qT[0], s[0]
        wq, ws, saved["WtQ"], saved["Wts"] = _row_col(W, clamp=True)   # rows for Y, columns for dX
        return _gemm_bc(q[0], s[0], SCALE_BLOCK128, wq, ws, SCALE_ROW, tokens=tokens, gemms=gemms), saved
    if scheme == "row_block":
        q, s = ops.quant_row(X2, clamp=True, hadamard128=(hadamard == 128))
        if hadamard == 128 or not need_backward:
            wq, ws = wq if wq is not None else quantize_weight(W, scheme, hadamard)
            return _gemm_bc(q, s, SCALE_ROW, wq, ws, SCALE_BLOCK128, 2.0 ** -7 if hadamard == 128 else 1.0, tokens=tokens, gemms=gemms), saved
        wq, wqT, ws = ops.quant_block(W[None], clamp=True, with_transpose=True)
        saved["WqT"], saved["Ws"] = wqT[0], ws[0]
        return _gemm_bc(q, s, SCALE_ROW, wq[0], ws[0], SCALE_BLOCK128, tokens=tokens, gemms=gemms), saved
    # double_channel
    K = X2.shape[1]
    if hadamard == "full" or not need_backward:
        q, s = _rotated_row_quant(X2, hadamard)
        wq, ws = wq if wq is not None else quantize_weight(W, scheme, hadamard)
        return _gemm_dc(q, s, wq, ws, 1.0 / K if hadamard == "full" else 0.0, tokens=tokens, gemms=gemms), saved
    q, s, saved["XtQ"], saved["Xts"] = _row_col(X2, clamp=True, inv_mode=INV_AMAX_DIV_127)
    wq, ws, saved["WtQ"], saved["Wts"] = _row_col(W, clamp=True, inv_mode=INV_AMAX_DIV_127)
    return _gemm_dc(q, s, wq, ws, tokens=tokens, gemms=gemms), saved


def linear_backward(dY2, X2, W, scheme="block_channel", hadamard=None, saved=None, tokens=None, gemms=None):
    """dY2 bf16 [T, N], X2 bf16 [T, K], W bf16 [N, K] -> (dX bf16 [T, K], dW bf16 [N, K])."""
    _check(scheme, hadamard)
    saved = saved or {}
    T, N = dY2.shape
    K = X2.shape[1]
    if scheme == "block_channel":
        if hadamard == 128:
            # H_128 along N for dX, along the tokens for dW: two differently rotated copies
            dq, ds = ops.quant_block_had128(dY2[None], clamp=True)
            wtq, wts = ops.quant_col_t(W, clamp=True, hadamard128=True)   # W^T [K,N] per row, rotated along N
            dX = _gemm_bc(dq[0], ds[0], SCALE_BLOCK128, wtq, wts, SCALE_ROW, 2.0 ** -7, tokens=tokens, gemms=gemms)
            # the token-dim rotation is fused too: one read of dY / X, transposed int8 out
            dyt, dyts = ops.quant_block_had128(dY2[None], along_rows=True, clamp=False)
            xt, xts = ops.quant_block_had128(X2[None], along_rows=True, clamp=False)
            dW = _gemm_bc(dyt[0], dyts[0].t(), SCALE_BLOCK128, xt[0], xts[0].t(), SCALE_BLOCK128, 2.0 ** -7, gemms=gemms)
            return dX, dW
        dq, dqT, ds = saved["dYq"] if "dYq" in saved else ops.quant_block(dY2[None], clamp=True, with_transpose=True)
        if "WtQ" in saved:
            wtq, wts = saved["WtQ"], saved["Wts"]
        else:
            wtq, wts = ops.quant_col_t(W, clamp=True)                # W^T [K,N] per row
        dX = _gemm_bc(dq[0], ds[0], SCALE_BLOCK128, wtq, wts, SCALE_ROW, tokens=tokens, gemms=gemms)
        if "XqT" in saved:
            xqT, xs = saved["XqT"], saved["Xs"]
        else:
            _, xqT3, xs3 = ops.quant_block(X2[None], clamp=True, with_transpose=True)
            xqT, xs = xqT3[0], xs3[0]
        # scales of the transposed operands are the transposed scale grids
        dW = _gemm_bc(dqT[0], ds[0].t(), SCALE_BLOCK128, xqT, xs.t(), SCALE_BLOCK128, gemms=gemms)
        return dX, dW
    if scheme == "row_block":
        if hadamard == 128:
            dq, ds = ops.quant_row(dY2, clamp=True, hadamard128=True)
            wtq, wts = ops.quant_block_had128(W[None], along_rows=True, clamp=True)      # W^T [K,N], groups along N
            dX = _gemm_bc(dq, ds, SCALE_ROW, wtq[0], wts[0].t(), SCALE_BLOCK128, 2.0 ** -7, tokens=tokens, gemms=gemms)
            dytq, dyts = ops.quant_col_t(dY2, clamp=True, hadamard128=True)   # dY^T [N,T] per row, rotated along the tokens
            xtq, xts = ops.quant_block_had128(X2[None], along_rows=True, clamp=True)
            dW = _gemm_bc(dytq, dyts, SCALE_ROW, xtq[0], xts[0].t(), SCALE_BLOCK128, 2.0 ** -7, gemms=gemms)
            return dX, dW
        dq, ds, dytq, dyts = _row_col(dY2, clamp=True)    # rows for dX, columns (dY^T [N,T] per row) for dW
        if "WqT" in saved:
            wqT, ws = saved["WqT"], saved["Ws"]
        else:
            _, wqT3, ws3 = ops.quant_block(W[None], clamp=True, with_transpose=True)
            wqT, ws = wqT3[0], ws3[0]
        dX = _gemm_bc(dq, ds, SCALE_ROW, wqT, ws.t(), SCALE_BLOCK128, tokens=tokens, gemms=gemms)
        _, xqT, xs = ops.quant_block(X2[None], clamp=True, with_transpose=True)
        dW = _gemm_bc(dytq, dyts, SCALE_ROW, xqT[0], xs[0].t(), SCALE_BLOCK128, gemms=gemms)
        return dX, dW
    # double_channel
    if hadamard == "full":
        # the transposed operands are rotated along the rows of the tensors as they lie in memory and quantised per row
        # of the transpose (ops.fwht_t_quant_row: a tiled int16 transposition + the one-pass rotate-and-quantise kernel;
        # the same bits as quant_row(fwht_t(.))).  A length that is no power of two is rotated as the reference's external
        # library rotates it (zero-extended to the next power of two and cut back)
        dq, ds = _rotated_row_quant(dY2, "full")
        wtq, wts = ops.fwht_t_quant_row(W, clamp=True, inv_mode=INV_AMAX_DIV_127)
        dX = _gemm_dc(dq, ds, wtq, wts, 1.0 / N, tokens=tokens, gemms=gemms)
        dytq, dyts = ops.fwht_t_quant_row(dY2, clamp=True, inv_mode=INV_AMAX_DIV_127)
        xtq, xts = ops.fwht_t_quant_row(X2, clamp=True, inv_mode=INV_AMAX_DIV_127)
        dW = _gemm_dc(dytq, dyts, xtq, xts, 1.0 / T, gemms=gemms)
        return dX, dW
    dq, ds, dytq, dyts = _row_col(dY2, clamp=True, inv_mode=INV_AMAX_DIV_127)
    if "WtQ" in saved:
        wtq, wts = saved["WtQ"], saved["Wts"]
    else:
        wtq, wts = ops.quant_col_t(W, clamp=True, inv_mode=INV_AMAX_DIV_127)
    dX = _gemm_dc(dq, ds, wtq, wts, tokens=tokens, gemms=gemms)
    if "XtQ" in saved:
        xtq, xts = saved["XtQ"], saved["Xts"]
    else:
        xtq, xts = ops.quant_col_t(X2, clamp=True, inv_mode=INV_AMAX_DIV_127)
    dW = _gemm_dc(dytq, dyts, xtq, xts, gemms=gemms)
    return dX, dW


def pad_tokens(x2, multiple=128):
    """Zero-pad the token (row) dim of a [T, C] tensor up to a multiple of the 128-row tile.
    Padding rows are zeros, so no absmax (block, row or column) changes, a block made only of
    padding quantises to zeros with the epsilon scale, and padded rows add nothing to dW: this
    is the "zero-pad to the tile, absmax over valid rows only" semantics for skinny / ragged M."""
    T = x2.shape[0]
    Tp = -(-T // multiple) * multiple
    if Tp == T:
        return x2
    out = x2.new_zeros((Tp, x2.shape[1]))
    out[:T] = x2
    return out


# Schemes whose whole step (linear_fwd_bwd with more than 256 tokens and output features) runs its three GEMMs as
# one launch (ops.gemm_i8_nt_multi; same kernels on the same operands, so the same bits as linear_forward +
# linear_backward): one launch of persistent workgroups walks the tiles of all three.
ONE_LAUNCH_SCHEMES = ("block_channel", "row_block", "double_channel")


def _one_launch(scheme, hadamard, padded_tokens, out_features):
    """Whether the GEMMs of a step (or of its backward half) go into one launch.  With up to 256 rows (tokens for Y
    and dX, output features for dW) a GEMM launched alone takes the few-rows kernel, which the one launch does not offer."""
    return scheme in ONE_LAUNCH_SCHEMES and min(padded_tokens, out_features) > 256 and ops.GEMM_PATH in ("auto", "tiled", "large")


# Schemes whose whole step is one library call (ops.linear_step: the same launches, queued from C) when nothing is
# rotated.  False: the step is assembled here from the separate entry points (same bits; the tests run both).
ONE_CALL_STEP = True
ONE_CALL_SCHEMES = ("block_channel", "double_channel")


def linear_fwd_bwd(X, W, dY, scheme="block_channel", hadamard=None, out=None, workspace=None):
    """One forward + backward of the layer: returns (Y, dX, dW) for X [B,M,K] or [M,K].
    Any number of tokens is accepted (zero-padded to a multiple of 128, see :func:`pad_tokens`);
    K and N must be multiples of 128.  ``out`` = (Y [T,N], dX [T,K], dW [N,K]) bf16 tensors to write into and
    ``workspace`` (``ops.linear_step_workspace_bytes``) are taken where the step is one library call and the token
    count a multiple of 128 (else ValueError): a caller that runs many steps of one shape allocates them once."""
    _check(scheme, hadamard)
    lead = X.shape[:-1]
    K, N = X.shape[-1], W.shape[0]
    X2, dY2 = X.reshape(-1, K), dY.reshape(-1, N)
    T = X2.shape[0]
    if T == 0:   # nothing to multiply: empty Y and dX, a zero weight gradient (as torch.nn.functional.linear gives)
        return X.new_empty((*lead, N)), X.new_empty((*lead, K)), W.new_zeros((N, K))
    X2, dY2 = pad_tokens(X2), pad_tokens(dY2)
    one_call = ONE_CALL_STEP and scheme in ONE_CALL_SCHEMES and hadamard is None and ops.GEMM_PATH in ("auto", "tiled", "large")
    if out is not None or workspace is not None:
        if not one_call or X2.shape[0] != T:
            raise ValueError("`out` / `workspace` go with the one-call step: block_channel or double_channel without rotation, "
                             "tokens a multiple of 128")
    if one_call:
        Y, dX, dW = ops.linear_step(X2, W, dY2, scheme, tokens=T, out=out, workspace=workspace)
        return Y[:T].reshape(*lead, N), dX[:T].reshape(*lead, K), dW
    gemms = [] if _one_launch(scheme, hadamard, X2.shape[0], N) else None
    pre = None
    if scheme == "block_channel" and hadamard is None:
        # both activations are at hand: one quantiser launch for X and dY (the forward alone would quantise X, the
        # backward dY, with the same kernel and the same bits)
        pre = ops.quant_block_multi([X2[None], dY2[None]], clamp=True, with_transpose=True)
    Y, saved = linear_forward(X2, W, scheme, hadamard, tokens=T, xq=pre[0] if pre else None, gemms=gemms)
    if pre:
        saved["dYq"] = pre[1]
    dX, dW = linear_backward(dY2, X2, W, scheme, hadamard, saved, tokens=T, gemms=gemms)
    if gemms:
        ops.gemm_i8_nt_multi(gemms)   # Y, dX and dW, into the tensors handed out above
    return Y[:T].reshape(*lead, N), dX[:T].reshape(*lead, K), dW


class Int8LinearFunction(torch.autograd.Function):
    """y = x W^T (+ bias) with every GEMM of forward and backward on the INT8 path."""

    @staticmethod
    def forward(ctx, x, weight, bias, scheme, hadamard):
        K, N = x.shape[-1], weight.shape[0]
        x2 = x.reshape(-1, K)
        ctx.tokens = x2.shape[0]
        ctx.has_bias = bias is not None
        if ctx.tokens == 0:   # an empty batch: empty output, zero gradients
            ctx.save_for_backward(x2, weight)
            return x.new_empty((*x.shape[:-1], N))
        x2 = pad_tokens(x2)
        need_bwd = any(ctx.needs_input_grad[:2])
        y, saved = linear_forward(x2, weight, scheme, hadamard, need_backward=need_bwd, tokens=ctx.tokens)
        ctx.scheme, ctx.hadamard, ctx.saved_q = scheme, hadamard, saved
        ctx.has_bias = bias is not None
        ctx.save_for_backward(x2, weight)
        y = y[:ctx.tokens]
        if bias is not None:
            y = y + bias
        return y.reshape(*x.shape[:-1], N)

    @staticmethod
    def backward(ctx, dy):
        x2, weight = ctx.saved_tensors
        N = weight.shape[0]
        if ctx.tokens == 0:
            return dy.new_empty((*dy.shape[:-1], x2.shape[1])), torch.zeros_like(weight), (dy.new_zeros((N,)) if ctx.has_bias else None), None, None
        dy2 = pad_tokens(dy.reshape(-1, N).contiguous())
        gemms = [] if _one_launch(ctx.scheme, ctx.hadamard, x2.shape[0], N) else None
        dx, dw = linear_backward(dy2, x2, weight, ctx.scheme, ctx.hadamard, ctx.saved_q, tokens=ctx.tokens, gemms=gemms)
        if gemms:
            ops.gemm_i8_nt_multi(gemms)   # dX and dW in one launch
        db = dy2.sum(dim=0).to(dy.dtype) if ctx.has_bias else None
        return dx[:ctx.tokens].reshape(*dy.shape[:-1], x2.shape[1]), dw, db, None, None


class Int8Linear(torch.nn.Module):
    """``torch.nn.Linear`` whose three GEMMs (Y, dX, dW) run through the INT8 path.
    in_features and out_features must be multiples of 128; any number of tokens works
    (zero-padded to the 128-row tile)."""

    def __init__(self, in_features, out_features, bias=False, scheme="block_channel", hadamard=None,
                 device=None, dtype=torch.bfloat16):
        super().__init__()
        _check(scheme, hadamard)
        if in_features % 128 or out_features % 128:
            raise ValueError("in_features and out_features must be multiples of 128")
        self.in_features, self.out_features = in_features, out_features
        self.scheme, self.hadamard = scheme, hadamard
        self.weight = torch.nn.Parameter(torch.empty(out_features, in_features, device=device, dtype=dtype))
        self.bias = torch.nn.Parameter(torch.zeros(out_features, device=device, dtype=dtype)) if bias else None
        torch.nn.init.normal_(self.weight, std=0.02)
        self._wq, self._wq_key = None, None   # quantised weight of the forward-only path and what it was made from

    def forward(self, x):
        if torch.is_grad_enabled() and (x.requires_grad or self.weight.requires_grad):
            return Int8LinearFunction.apply(x, self.weight, self.bias, self.scheme, self.hadamard)
        if x.numel() == 0:
            return x.new_empty((*x.shape[:-1], self.out_features))
        # forward only (inference): the weight is quantised once per weight update, not per call
        key = (self.weight._version, self.weight.data_ptr(), self.scheme, self.hadamard)
        if self._wq_key != key:
            self._wq, self._wq_key = quantize_weight(self.weight.detach(), self.scheme, self.hadamard), key
        K = x.shape[-1]
        x2 = x.reshape(-1, K)
        tokens = x2.shape[0]
        y, _ = linear_forward(pad_tokens(x2), None, self.scheme, self.hadamard, need_backward=False, wq=self._wq, tokens=tokens)
        y = y[:tokens]
        if self.bias is not None:
            y = y + self.bias
        return y.reshape(*x.shape[:-1], self.out_features)

    def extra_repr(self):
        return f"in_features={self.in_features}, out_features={self.out_features}, scheme={self.scheme}, hadamard={self.hadamard}"
