"""Host wrappers (allocate outputs, derive strides, pick the stream) around the C ABI.

Every function takes and returns torch tensors on a HIP device, enqueues on the
current torch stream and never synchronises.  Arguments the kernels cannot take
(wrong dtype/device, sizes that are not multiples of the tile) raise ``ValueError``
here, before anything is launched.
"""
import collections
import threading

import torch

from . import _lib
from ._lib import (COMBINE_DIV_PROD, COMBINE_MUL_MUL, COMBINE_MUL_PROD, GEMM_LARGE_TILES, GEMM_ONE_TILE, GEMM_SKINNY, GEMM_STRICT, GEMM_TILED, INV_AMAX_DIV_127,
                   INV_AMAX_MUL_RCP127, INV_MULTIPLIER, INV_RCP_OF_SCALE, Q_CLAMP, Q_EPS_ADD, Q_HAD128, Q_SCALE_BF16, Q_TORCH_BF16, Q_TORCH_ROUND,
                   Q_WS_PINGPONG, Q_WS_SECOND,
                   SCALE_BLOCK128, SCALE_BLOCK_K256, SCALE_ROW, SCALE_ROW_K128)

__all__ = ["quant_block", "quant_block_multi", "quant_block_had128", "quant_row", "quant_col_t", "quant_row_col_t", "fwht", "fwht_t", "gemm_i8_nt", "gemm_i8_nt_i32",
           "linear_step", "linear_step_workspace_bytes"]


# Which GEMM kernel `gemm_i8_nt` asks for: "auto" (the few-rows kernel for M <= 256, else an
# LDS-tiled one with tiles sized to the shape), "tiled", "large" (LDS-tiled with 256 x 256 tiles
# whatever the shape) or "skinny" (wherever it supports the scale modes).  Tests set it to run
# the same cases through every kernel.
GEMM_PATH = "auto"
# False: one workgroup per output tile also where the block-channel promotion would run on persistent workgroups (same bits)
GEMM_PERSISTENT = True


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _on_gpu(t):
    """Whether a tensor lives in device memory.  One place, so that a host-side model of the launches
    (tests that record the C-ABI calls these wrappers make, without a GPU) can stand in for it."""
    return t.is_cuda


def _need(cond, msg):
    if not cond:
        raise ValueError(msg)


def _check_bf16(x, name):
    _need(isinstance(x, torch.Tensor) and _on_gpu(x), f"{name} must be a tensor on the GPU")
    _need(x.dtype == torch.bfloat16, f"{name} must be bfloat16, got {x.dtype}")


def _qflags(clamp, eps_add, scale_bf16, torch_arith=None):
    _need(torch_arith in (None, "f32", "bf16"), "torch_arith must be None, 'f32' or 'bf16'")
    return ((Q_CLAMP if clamp else 0) | (Q_EPS_ADD if eps_add else 0) | (Q_SCALE_BF16 if scale_bf16 else 0) |
            {None: 0, "f32": Q_TORCH_ROUND, "bf16": Q_TORCH_ROUND | Q_TORCH_BF16}[torch_arith])


def quant_block(x, *, clamp=True, group_c=128, eps_add=False, scale_bf16=False, inv_mode=INV_RCP_OF_SCALE,
                out="like", with_transpose=False, torch_arith=None):
    """Per-128 x group_c-block absmax quantisation of ``x`` [B, M, N] (bf16).

    ``x`` may be row-major (last stride 1) or a transposed view of a row-major
    tensor (stride(1) == 1); it is read in place either way.  ``out``:
      "like"        q has the strides of ``x`` (what ``torch.empty_like`` gives)
      "contiguous"  q is contiguous in the logical [B, M, N] orientation
    ``with_transpose`` additionally returns ``qT`` = contiguous [B, N, M] int8 holding
    ``q`` transposed, written by the same kernel from the same registers.
    ``torch_arith`` "f32" / "bf16": the arithmetic of the reference's pure-torch quantisers (reciprocal
    times 127, round half to even, clamp +-127; "bf16" rounds every intermediate to bf16) instead of
    its kernels'; row-major ``x``, ``q`` only.
    Returns ``(q, s)`` or ``(q, qT, s)``; ``s`` is fp32 [B, M/128, N/group_c]."""
    _check_bf16(x, "x")
    _need(x.dim() == 3, "x must be [B, M, N]")
    B, M, N = x.shape
    _need(B > 0 and M > 0 and N > 0, "empty tensors are not supported")
    if x.stride(2) == 1 or N == 1:
        xc, transposed = x, False
    elif x.stride(1) == 1:
        xc, transposed = x.transpose(1, 2), True
    else:
        xc, transposed = x.contiguous(), False
    if xc.stride(2) != 1 or (B > 1 and xc.stride(0) % 8) or xc.stride(1) % 8 or xc.data_ptr() % 16:
        xc = xc.contiguous()
    _need(group_c in (128, 256), "group_c must be 128 or 256")
    _need(out in ("like", "contiguous"), "out must be 'like' or 'contiguous'")
    _need(not (transposed or with_transpose) or group_c == 128, "transposed layouts need 128 x 128 blocks")
    _need(torch_arith is None or not (transposed or with_transpose), "torch_arith needs a row-major x and no transposed output")
    _need(M % 128 == 0 and N % (group_c if not transposed else 128) == 0,
          f"block quantisation needs M % 128 == 0 and N % {group_c} == 0, got M={M} N={N}")
    R, C = xc.shape[1], xc.shape[2]          # canonical (row-major) view of the memory
    dev = x.device
    s = torch.empty((B, M // 128, N // group_c), dtype=torch.float32, device=dev)
    if transposed:   # canonical tile (rb, cb) is logical tile (mb = cb, nb = rb)
        ssr, ssc = s.stride(2), s.stride(1)
    else:
        ssr, ssc = s.stride(1), s.stride(2)
    # which of the kernel's two outputs are needed: qc in the memory ("canonical")
    # orientation [B, R, C], qct in the transposed one [B, C, R]
    if transposed:
        want_canon, want_canon_t = (out == "like" or with_transpose), (out == "contiguous")
    else:
        want_canon, want_canon_t = True, with_transpose
    qc = torch.empty((B, R, C), dtype=torch.int8, device=dev) if want_canon else None
    qct = torch.empty((B, C, R), dtype=torch.int8, device=dev) if want_canon_t else None
    _lib.call("ti8_quant_block", xc.data_ptr(), xc.stride(0), xc.stride(1),
              qc.data_ptr() if qc is not None else None, R * C, C,
              qct.data_ptr() if qct is not None else None, R * C, R,
              s.data_ptr(), s.stride(0), ssr, ssc, B, R, C, group_c,
              _qflags(clamp, eps_add, scale_bf16, torch_arith), inv_mode, _stream())
    if not transposed:
        q = qc
        qT = qct
    else:
        q = qct if out == "contiguous" else qc.transpose(1, 2)
        qT = qc  # canonical orientation IS the logical transpose
    return (q, qT, s) if with_transpose else (q, s)


def quant_block_multi(xs, *, clamp=True, with_transpose=False, inv_mode=INV_RCP_OF_SCALE):
    """``quant_block`` of several row-major operands [B, M, N] (up to 4) in ONE launch: a list of
    ``(q, s)`` or ``(q, qT, s)``, bit-identical to separate calls.  A training step that has X and dY
    at hand quantises both this way."""
    _need(1 <= len(xs) <= 4, "between 1 and 4 operands")
    descs, outs = (_lib.QBlockOperand * len(xs))(), []
    for i, x in enumerate(xs):
        _check_bf16(x, "x")
        _need(x.dim() == 3 and x.numel() > 0, "every operand must be a non-empty [B, M, N] tensor")
        B, M, N = x.shape
        _need(M % 128 == 0 and N % 128 == 0, f"block quantisation needs M % 128 == 0 and N % 128 == 0, got M={M} N={N}")
        if x.stride(2) != 1 or (B > 1 and x.stride(0) % 8) or x.stride(1) % 8 or x.data_ptr() % 16:
            x = x.contiguous()
        q = torch.empty((B, M, N), dtype=torch.int8, device=x.device)
        qT = torch.empty((B, N, M), dtype=torch.int8, device=x.device) if with_transpose else None
        s = torch.empty((B, M // 128, N // 128), dtype=torch.float32, device=x.device)
        descs[i] = _lib.QBlockOperand(x.data_ptr(), x.stride(0), x.stride(1), q.data_ptr(), M * N, N,
                                      qT.data_ptr() if with_transpose else None, M * N, M,
                                      s.data_ptr(), s.stride(0), s.stride(1), s.stride(2), B, M, N)
        outs.append((q, qT, s) if with_transpose else (q, s))
        xs = list(xs)
        xs[i] = x     # keep a contiguous copy alive until the launch is queued
    _lib.call("ti8_quant_block_multi", descs, len(xs), _qflags(clamp, False, False), inv_mode, _stream())
    return outs


def quant_block_had128(x, *, along_rows=False, clamp=True, inv_mode=INV_RCP_OF_SCALE):
    """Block-diagonal H_128 rotation fused with the 128x128 block quantiser, one read of ``x``
    [B, R, C] (bf16, row-major).  ``along_rows=False``: groups of 128 along the columns,
    returns ``q`` [B, R, C].  ``along_rows=True``: groups along the rows, returns ``q``
    TRANSPOSED, [B, C, R].  ``s`` is fp32 [B, R/128, C/128] (tile grid of ``x``) in both cases."""
    _check_bf16(x, "x")
    _need(x.dim() == 3, "x must be [B, R, C]")
    B, R, C = x.shape
    _need(B > 0 and R % 128 == 0 and C % 128 == 0 and R > 0 and C > 0, f"need R % 128 == 0 and C % 128 == 0, got {R}x{C}")
    if x.stride(2) != 1 or (B > 1 and x.stride(0) % 8) or x.stride(1) % 8 or x.data_ptr() % 16:
        x = x.contiguous()
    q = torch.empty((B, C, R) if along_rows else (B, R, C), dtype=torch.int8, device=x.device)
    s = torch.empty((B, R // 128, C // 128), dtype=torch.float32, device=x.device)
    _lib.call("ti8_quant_block_had128", x.data_ptr(), x.stride(0), x.stride(1), q.data_ptr(), R * C, q.shape[2],
              s.data_ptr(), s.stride(0), s.stride(1), s.stride(2), B, R, C, 1 if along_rows else 0,
              _qflags(clamp, False, False), inv_mode, _stream())
    return q, s


def quant_row(x, *, clamp=True, group=0, eps_add=False, scale_bf16=False, inv_mode=INV_RCP_OF_SCALE, hadamard128=False,
              torch_arith=None):
    """Per-row (``group=0``) or per-(row, 128 columns) absmax quantisation of the last dim.
    ``x``: bf16 [..., cols].  Returns ``(q, s)`` with ``s`` fp32 [...] or [..., cols/128].
    ``hadamard128`` rotates every group of 128 columns by H_128 first (fused, one read)."""
    _check_bf16(x, "x")
    _need(x.dim() >= 1 and x.numel() > 0, "x must be a non-empty tensor")
    cols = x.shape[-1]
    _need(cols % 128 == 0 and cols <= 32768, f"per-row quantisation needs cols % 128 == 0 and cols <= 32768, got {cols}")
    x2 = x.reshape(-1, cols)
    if x2.stride(1) != 1 or x2.stride(0) % 8 or x2.data_ptr() % 16:
        x2 = x2.contiguous()
    rows = x2.shape[0]
    q = torch.empty((rows, cols), dtype=torch.int8, device=x.device)
    s = torch.empty((rows, cols // 128) if group else (rows,), dtype=torch.float32, device=x.device)
    _lib.call("ti8_quant_row", x2.data_ptr(), x2.stride(0), q.data_ptr(), cols, s.data_ptr(), rows, cols, group,
              _qflags(clamp, eps_add, scale_bf16, torch_arith) | (Q_HAD128 if hadamard128 else 0), inv_mode, _stream())
    lead = x.shape[:-1]
    return q.reshape(*lead, cols), s.reshape(*lead, cols // 128) if group else s.reshape(*lead)


def quant_col_t(x, *, clamp=True, inv_mode=INV_RCP_OF_SCALE, hadamard128=False):
    """Per-column absmax quantisation of ``x`` [R, C] with transposed output: the per-row
    quantiser applied to ``x.T``.  Returns ``(qT int8 [C, R], s fp32 [C])``.
    ``hadamard128`` rotates every group of 128 rows by H_128 first (= ``quant_row(x.T, hadamard128=True)``
    without the bf16 transpose)."""
    _check_bf16(x, "x")
    _need(x.dim() == 2, "x must be [R, C]")
    R, C = x.shape
    _need(R % 128 == 0 and C % 128 == 0, f"column quantisation needs R % 128 == 0 and C % 128 == 0, got {R}x{C}")
    if x.stride(1) != 1 or x.stride(0) % 8 or x.data_ptr() % 16:
        x = x.contiguous()
    qT = torch.empty((C, R), dtype=torch.int8, device=x.device)
    s = torch.empty((C,), dtype=torch.float32, device=x.device)
    ws = torch.empty((C,), dtype=torch.float32, device=x.device)
    _lib.call("ti8_quant_col_t", x.data_ptr(), x.stride(0), qT.data_ptr(), R, s.data_ptr(), ws.data_ptr(), R, C,
              _qflags(clamp, False, False) | (Q_HAD128 if hadamard128 else 0), inv_mode, _stream())
    return qT, s


def quant_row_col_t(x, *, clamp=True, inv_mode=INV_RCP_OF_SCALE):
    """Per-row AND per-column (transposed) quantisation of x [R, C] in one go:
    returns (q [R, C], s_row [R], qT [C, R], s_col [C]), the same bits as
    ``quant_row(x)`` and ``quant_col_t(x)``."""
    _check_bf16(x, "x")
    _need(x.dim() == 2, "x must be [R, C]")
    R, C = x.shape
    _need(R % 128 == 0 and C % 128 == 0, f"R and C must be multiples of 128, got {R} x {C}")
    if x.stride(1) != 1 or x.stride(0) % 8 or x.data_ptr() % 16:
        x = x.contiguous()
    q = torch.empty((R, C), dtype=torch.int8, device=x.device)
    qT = torch.empty((C, R), dtype=torch.int8, device=x.device)
    s_row = torch.empty((R,), dtype=torch.float32, device=x.device)
    s_col = torch.empty((C,), dtype=torch.float32, device=x.device)
    flags = _qflags(clamp, False, False)
    stream = _stream()
    args = (x.data_ptr(), x.stride(0), q.data_ptr(), C, s_row.data_ptr(), qT.data_ptr(), R, s_col.data_ptr())
    if torch.cuda.is_current_stream_capturing():
        # a replayed call cannot alternate: plain workspace, cleared by the library on every replay
        ws = torch.empty((R + C,), dtype=torch.float32, device=x.device)
        _lib.call("ti8_quant_row_col_t", *args, ws.data_ptr(), R, C, flags, inv_mode, stream)
    else:
        with _PINGPONG_LOCK:
            slot = _pingpong_workspace(x.device, stream, R, C)
            _lib.call("ti8_quant_row_col_t", *args, slot[0].data_ptr(), R, C,
                      flags | Q_WS_PINGPONG | (Q_WS_SECOND if slot[1] else 0), inv_mode, stream)
            slot[1] ^= 1   # only once the launches are queued: a rejected call leaves both parts as they were
    return q, s_row, qT, s_col


# Two-part workspaces of quant_row_col_t: a call collects its maxima in one part and clears the
# other for the next call, so no call needs a launch that clears memory.  One buffer (and the part
# to use next) per device, stream and shape: calls on one stream run in order and can share it;
# calls on different streams may overlap and get different buffers.  The cache holds the
# _PINGPONG_SLOTS most recently used buffers (a training step alternates between a handful of
# shapes); a buffer that drops out is released once the work queued on it has run (torch's
# allocator keeps the memory of a freed tensor until the stream has passed the free), and a
# shape that comes back starts again from a zero-filled buffer.  Lookup, launch and the flip of
# the part happen under one lock, so that threads sharing a stream enqueue their calls in the
# order in which they were handed the parts.
_PINGPONG_SLOTS = 16
_PINGPONG_WS = collections.OrderedDict()
_PINGPONG_LOCK = threading.Lock()


def _pingpong_workspace(device, stream, R, C):
    """The slot [buffer of 2 * (R + C) floats, part the next call works in]; call with the lock held."""
    key = (device.index, stream, R, C)
    slot = _PINGPONG_WS.pop(key, None)
    if slot is None:
        slot = [torch.zeros((2 * (R + C),), dtype=torch.float32, device=device), 0]
        while len(_PINGPONG_WS) >= _PINGPONG_SLOTS:
            _PINGPONG_WS.popitem(last=False)
    _PINGPONG_WS[key] = slot          # most recently used last
    return slot


def fwht(x, n=None, scale=1.0):
    """Un-normalised Walsh-Hadamard transform over groups of ``n`` (default: all) of the last dim.
    Without ``n``, a last dim that is no power of two is transformed as the reference's external library
    transforms it: zero-extended to the next power of two, multiplied by H, cut back to its own length
    (a multiple of 16 in (64, 32768))."""
    _check_bf16(x, "x")
    cols = x.shape[-1]
    n = (1 << max(cols - 1, 1).bit_length()) if n is None else n
    _need(n >= 128 and n <= 32768 and (n & (n - 1)) == 0, f"n must be a power of two in [128, 32768], got {n}")
    _need(cols % n == 0 or (n // 2 < cols < n and cols % 16 == 0), f"last dim {cols} is neither a multiple of n={n} nor a multiple of 16 in ({n // 2}, {n})")
    x2 = x.reshape(-1, cols)
    if x2.stride(1) != 1 or x2.stride(0) % 8 or x2.data_ptr() % 16:
        x2 = x2.contiguous()
    y = torch.empty((x2.shape[0], cols), dtype=torch.bfloat16, device=x.device)
    _lib.call("ti8_fwht", x2.data_ptr(), x2.stride(0), y.data_ptr(), cols, x2.shape[0], cols, n, float(scale), _stream())
    return y.reshape(x.shape)


def fwht_quant_row(x, *, clamp=True, eps_add=False, inv_mode=INV_RCP_OF_SCALE):
    """``quant_row(fwht(x))`` in one pass over ``x`` (bf16 [..., cols], the rotation over the whole last dim, zero-extended
    when ``cols`` is no power of two): the rotated bf16 tensor is never written.  Returns ``(q, s)``, the same bits."""
    _check_bf16(x, "x")
    _need(x.dim() >= 1 and x.numel() > 0, "x must be a non-empty tensor")
    cols = x.shape[-1]
    n = 1 << max(cols - 1, 1).bit_length()
    _need(128 <= n <= 32768 and cols % 128 == 0, f"the last dim must be a multiple of 128 in (64, 32768], got {cols}")
    x2 = x.reshape(-1, cols)
    if x2.stride(1) != 1 or x2.stride(0) % 8 or x2.data_ptr() % 16:
        x2 = x2.contiguous()
    rows = x2.shape[0]
    q = torch.empty((rows, cols), dtype=torch.int8, device=x.device)
    s = torch.empty((rows,), dtype=torch.float32, device=x.device)
    _lib.call("ti8_fwht_quant_row", x2.data_ptr(), x2.stride(0), q.data_ptr(), cols, s.data_ptr(), rows, cols, n,
              _qflags(clamp, eps_add, False), inv_mode, _stream())
    lead = x.shape[:-1]
    return q.reshape(*lead, cols), s.reshape(*lead)


def fwht_t_quant_row(x, *, clamp=True, eps_add=False, inv_mode=INV_RCP_OF_SCALE):
    """``quant_row(fwht_t(x))`` for x bf16 [R, C]: the rotation along the rows of ``x`` and the per-row quantiser of the
    rotated transpose, ``(q int8 [C, R], s fp32 [C])``, the same bits; a tiled transposition into a scratch tensor and the
    one-pass rotate + quantise kernel on it."""
    _check_bf16(x, "x")
    _need(x.dim() == 2, "x must be [R, C]")
    R, C = x.shape
    _need(128 <= R <= 32768 and R % 128 == 0 and C > 0 and C % 64 == 0, f"need R a multiple of 128 in [128, 32768] and C % 64 == 0, got {R} x {C}")
    if x.stride(1) != 1 or x.stride(0) % 8 or x.data_ptr() % 16:
        x = x.contiguous()
    scratch = torch.empty((C, R), dtype=torch.bfloat16, device=x.device)
    q = torch.empty((C, R), dtype=torch.int8, device=x.device)
    s = torch.empty((C,), dtype=torch.float32, device=x.device)
    _lib.call("ti8_fwht_t_quant_row", x.data_ptr(), x.stride(0), scratch.data_ptr(), q.data_ptr(), R, s.data_ptr(), R, C,
              _qflags(clamp, eps_add, False), inv_mode, _stream())
    return q, s


def fwht_t(x, scale=1.0):
    """Walsh-Hadamard transform of ``x.T`` along its rows, i.e. along the ROWS of ``x`` [R, C], without
    the bf16 transpose: returns y [C, R] = ``fwht(x.T.contiguous())``, bit for bit."""
    _check_bf16(x, "x")
    _need(x.dim() == 2, "x must be [R, C]")
    R, C = x.shape
    if R & (R - 1) and R % 16 == 0 and 64 < R < 32768:
        # a length that is no power of two: the zero-extended transform, on the transposed copy
        return fwht(x.t().contiguous(), None, scale)
    _need(R >= 128 and R <= 32768 and (R & (R - 1)) == 0, f"R must be a power of two in [128, 32768] or a multiple of 16 in (64, 32768), got {R}")
    _need(C > 0 and C % 8 == 0, f"C must be a positive multiple of 8, got {C}")
    if x.stride(1) != 1 or x.stride(0) % 8 or x.data_ptr() % 16:
        x = x.contiguous()
    y = torch.empty((C, R), dtype=torch.bfloat16, device=x.device)
    _lib.call("ti8_fwht_t", x.data_ptr(), x.stride(0), y.data_ptr(), R, R, C, float(scale), _stream())
    return y


def _k_contig(t):
    if t.stride(-1) != 1 or any(st % 16 for st in t.stride()[:-1]) or t.data_ptr() % 16:
        t = t.contiguous()
    return t


def _scale_desc(s, mode, rows, nkb, batch, batched, who):
    """(ptr, batch stride, row stride, k stride) of a scale tensor for operand `who`."""
    _need(s.dtype == torch.float32 and _on_gpu(s), f"{who} scale must be a float32 GPU tensor")
    if mode == SCALE_ROW:
        shape = (batch, rows) if batched else (rows,)
        _need(s.numel() == batch * rows if batched else s.numel() == rows,
              f"{who} per-row scale must have {shape} elements, got {tuple(s.shape)}")
        v = s.reshape(shape)
        return v, (v.stride(0) if batched else 0), v.stride(-1), 0
    if mode == SCALE_BLOCK128:
        shape = (-(-rows // 128), nkb)
    elif mode == SCALE_ROW_K128:
        shape = (rows, nkb)
    else:
        shape = (-(-rows // 128), nkb // 2)
    full = ((batch,) + shape) if batched else shape
    _need(tuple(s.shape) == full or (not batched and tuple(s.shape) == (1,) + shape),
          f"{who} scale must have shape {full}, got {tuple(s.shape)}")
    v = s.reshape(full)
    return v, (v.stride(0) if batched else 0), v.stride(-2), v.stride(-1)


def gemm_i8_nt(A, B, sA, modeA, sB, modeB, *, acc_i32_full=False, combine=COMBINE_MUL_MUL, out_scale=1.0,
               post_scale=0.0, strict=False, out=None):
    """C[b] = dequant(A[b] @ B[b]^T): A int8 [batch, M, K]; B int8 [N, K] (shared) or [batch, N, K]."""
    _need(A.dtype == torch.int8 and B.dtype == torch.int8 and _on_gpu(A) and _on_gpu(B), "A and B must be int8 GPU tensors")
    _need(A.dim() == 3 and B.dim() in (2, 3), "A must be [batch, M, K]; B [N, K] or [batch, N, K]")
    batch, M, K = A.shape
    N = B.shape[-2]
    _need(B.shape[-1] == K, f"K mismatch: A has {K}, B has {B.shape[-1]}")
    _need(B.dim() == 2 or B.shape[0] == batch, "batch mismatch between A and B")
    _need((M % 128 == 0 or (M % 32 == 0 and M <= 256)) and N % 128 == 0 and K % 128 == 0 and batch > 0,
          f"N, K must be positive multiples of 128 and M one of 128 (of 32 up to 256 rows), got M={M} N={N} K={K}")
    A, B = _k_contig(A), _k_contig(B)
    nkb = K // 128
    sAv, sa_bs, sa_rs, sa_ks = _scale_desc(sA, modeA, M, nkb, batch, True, "A")
    sBv, sb_bs, sb_rs, sb_ks = _scale_desc(sB, modeB, N, nkb, batch, B.dim() == 3, "B")
    if out is None:
        out = torch.empty((batch, M, N), dtype=torch.bfloat16, device=A.device)
    else:
        _need(out.shape == (batch, M, N) and out.dtype == torch.bfloat16 and out.stride(2) == 1, "bad `out` tensor")
    _lib.call("ti8_gemm_i8_nt", A.data_ptr(), A.stride(0), A.stride(1),
              B.data_ptr(), B.stride(0) if B.dim() == 3 else 0, B.stride(-2),
              out.data_ptr(), out.stride(0), out.stride(1),
              sAv.data_ptr(), modeA, sa_bs, sa_rs, sa_ks, sBv.data_ptr(), modeB, sb_bs, sb_rs, sb_ks,
              batch, M, N, K, 1 if acc_i32_full else 0, combine, float(out_scale), float(post_scale),
              (GEMM_STRICT if strict else 0) | {"auto": 0, "tiled": GEMM_TILED, "skinny": GEMM_SKINNY, "large": GEMM_LARGE_TILES}[GEMM_PATH]
              | (0 if GEMM_PERSISTENT else GEMM_ONE_TILE),
              _stream())
    return out


def gemm_i8_nt_multi(problems):
    """Up to 3 GEMMs ``dequant(A @ B^T)`` with A int8 [M, K] and B int8 [N, K] in ONE launch; `problems`
    is a list of dicts with the keys A, B, sA, modeA, sB, modeB and optionally acc_i32_full, combine,
    out_scale, post_scale, out (meaning as in ``gemm_i8_nt``).  Returns the bf16 outputs [M, N],
    bit-identical to separate calls.  The GEMMs must select the same kernel (else RuntimeError)."""
    _need(1 <= len(problems) <= 3, "between 1 and 3 GEMMs")
    descs, outs, keep = (_lib.GemmProblem * len(problems))(), [], []
    for i, p in enumerate(problems):
        A, B = p["A"], p["B"]
        _need(A.dtype == torch.int8 and B.dtype == torch.int8 and _on_gpu(A) and _on_gpu(B), "A and B must be int8 GPU tensors")
        _need(A.dim() == 2 and B.dim() == 2, "A must be [M, K] and B [N, K]")
        M, K = A.shape
        N = B.shape[0]
        _need(B.shape[1] == K, f"K mismatch: A has {K}, B has {B.shape[1]}")
        _need(M % 128 == 0 and N % 128 == 0 and K % 128 == 0 and M > 0 and N > 0 and K > 0,
              f"M, N, K must be positive multiples of 128, got M={M} N={N} K={K}")
        A, B = _k_contig(A), _k_contig(B)
        sAv, _, sa_rs, sa_ks = _scale_desc(p["sA"], p["modeA"], M, K // 128, 1, False, "A")
        sBv, _, sb_rs, sb_ks = _scale_desc(p["sB"], p["modeB"], N, K // 128, 1, False, "B")
        out = p.get("out")
        if out is None:
            out = torch.empty((M, N), dtype=torch.bfloat16, device=A.device)
        else:
            _need(out.shape == (M, N) and out.dtype == torch.bfloat16 and out.stride(1) == 1, "bad `out` tensor")
        descs[i] = _lib.GemmProblem(A.data_ptr(), 0, A.stride(0), B.data_ptr(), 0, B.stride(0), out.data_ptr(), 0, out.stride(0),
                                    sAv.data_ptr(), p["modeA"], 0, sa_rs, sa_ks, sBv.data_ptr(), p["modeB"], 0, sb_rs, sb_ks,
                                    1, M, N, K, 1 if p.get("acc_i32_full") else 0, p.get("combine", COMBINE_MUL_MUL),
                                    float(p.get("out_scale", 1.0)), float(p.get("post_scale", 0.0)))
        outs.append(out)
        keep.append((A, B, sAv, sBv))     # contiguous copies stay alive until the launch is queued
    _lib.call("ti8_gemm_i8_nt_multi", descs, len(problems), {"auto": 0, "tiled": GEMM_TILED, "large": GEMM_LARGE_TILES}.get(GEMM_PATH, 0) | (0 if GEMM_PERSISTENT else GEMM_ONE_TILE), _stream())
    return outs


def gemm_i8_nt_i32(A, B):
    """Raw int32 accumulators of A[b] @ B[b]^T over the whole K."""
    _need(A.dtype == torch.int8 and B.dtype == torch.int8 and _on_gpu(A) and _on_gpu(B), "A and B must be int8 GPU tensors")
    _need(A.dim() == 3 and B.dim() in (2, 3), "A must be [batch, M, K]; B [N, K] or [batch, N, K]")
    batch, M, K = A.shape
    N = B.shape[-2]
    _need(B.shape[-1] == K and (B.dim() == 2 or B.shape[0] == batch), "shape mismatch between A and B")
    _need(M % 128 == 0 and N % 128 == 0 and K % 128 == 0 and batch > 0,
          f"M, N, K must be positive multiples of 128, got M={M} N={N} K={K}")
    A, B = _k_contig(A), _k_contig(B)
    C = torch.empty((batch, M, N), dtype=torch.int32, device=A.device)
    _lib.call("ti8_gemm_i8_nt_i32", A.data_ptr(), A.stride(0), A.stride(1),
              B.data_ptr(), B.stride(0) if B.dim() == 3 else 0, B.stride(-2),
              C.data_ptr(), C.stride(0), C.stride(1), batch, M, N, K, _stream())
    return C


_STEP_SCHEMES = {"block_channel": _lib.SCHEME_BLOCK_CHANNEL, "double_channel": _lib.SCHEME_DOUBLE_CHANNEL}


def linear_step_workspace_bytes(T, K, N, scheme):
    """Bytes of workspace that :func:`linear_step` needs for T tokens (a multiple of 128), K inputs and N outputs."""
    _need(scheme in _STEP_SCHEMES, f"linear_step serves the schemes {sorted(_STEP_SCHEMES)}")
    n = _lib.lib().ti8_linear_fwd_bwd_workspace(T, K, N, _STEP_SCHEMES[scheme])
    _need(n >= 0, f"T, K and N must be positive multiples of 128, got T={T} K={K} N={N}")
    return n


def linear_step(X2, W, dY2, scheme, *, tokens=None, out=None, workspace=None):
    """A whole forward + backward of the layer in ONE library call (``ti8_linear_fwd_bwd``): X2 bf16 [T, K],
    W bf16 [N, K], dY2 bf16 [T, N] -> (Y [T, N], dX [T, K], dW [N, K]), the quantisers and GEMMs of
    ``linear.linear_forward`` + ``linear.linear_backward`` enqueued from C with the same bits.
    T, K, N multiples of 128; ``tokens`` = rows that hold data when the caller has zero-padded X2 and dY2 (with up to
    256 rows Y and dX are then computed for the first ceil(tokens / 32) * 32 rows only).  ``out`` = (Y, dX, dW) to write into; ``workspace`` = a uint8 tensor of at least
    :func:`linear_step_workspace_bytes` bytes (both allocated here when absent)."""
    for t, name in ((X2, "X"), (W, "W"), (dY2, "dY")):
        _check_bf16(t, name)
        _need(t.dim() == 2, f"{name} must be 2-D")
    T, K = X2.shape
    N = W.shape[0]
    _need(W.shape[1] == K and tuple(dY2.shape) == (T, N), f"shapes do not fit: X {tuple(X2.shape)}, W {tuple(W.shape)}, dY {tuple(dY2.shape)}")
    need = linear_step_workspace_bytes(T, K, N, scheme)

    def rows(t):
        if t.stride(1) != 1 or t.stride(0) % 8 or t.data_ptr() % 16:
            t = t.contiguous()
        return t
    X2, W, dY2 = rows(X2), rows(W), rows(dY2)
    dev = X2.device
    if out is None:
        out = (torch.empty((T, N), dtype=torch.bfloat16, device=dev), torch.empty((T, K), dtype=torch.bfloat16, device=dev),
               torch.empty((N, K), dtype=torch.bfloat16, device=dev))
    else:
        for o, shape in zip(out, ((T, N), (T, K), (N, K))):
            _need(tuple(o.shape) == shape and o.dtype == torch.bfloat16 and o.stride(1) == 1 and _on_gpu(o), "bad `out` tensor")
    if workspace is None:
        workspace = torch.empty((need + 256,), dtype=torch.uint8, device=dev)
        workspace = workspace[(-workspace.data_ptr()) % 256:][:need]    # device allocations are aligned already: a no-op there
    else:
        _need(workspace.dtype == torch.uint8 and workspace.is_contiguous() and workspace.numel() >= need and _on_gpu(workspace)
              and workspace.data_ptr() % 256 == 0, f"`workspace` must be a contiguous, 256-byte aligned uint8 GPU tensor of at least {need} bytes")
    Y, dX, dW = out
    _lib.call("ti8_linear_fwd_bwd", X2.data_ptr(), X2.stride(0), W.data_ptr(), W.stride(0), dY2.data_ptr(), dY2.stride(0),
              Y.data_ptr(), Y.stride(0), dX.data_ptr(), dX.stride(0), dW.data_ptr(), dW.stride(0), T, T if tokens is None else tokens, K, N,
              _STEP_SCHEMES[scheme],
              {"auto": 0, "tiled": GEMM_TILED, "large": GEMM_LARGE_TILES}.get(GEMM_PATH, 0) | (0 if GEMM_PERSISTENT else GEMM_ONE_TILE),
              workspace.data_ptr(), workspace.numel(), _stream())
    return Y, dX, dW
