"""ctypes access to ``oracle/c/libti8_ref.so``, the scalar C restatement.

TEST INFRASTRUCTURE: an independent, element-at-a-time evaluation of the same
formulas, used by the tests to pin the vectorised torch oracle bit-for-bit.
"""
import ctypes
import os
import subprocess

import numpy as np
import torch

_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "c")
_SO = os.path.join(_DIR, "libti8_ref.so")
_lib = None


def build(force: bool = False):
    """Compile the C restatement with gcc (seconds)."""
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(os.path.join(_DIR, "ti8_ref.c")):
        subprocess.check_call(["make", "-s", "-B", "-C", _DIR, "CC=gcc"])
    return _SO


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(_SO)
    return _lib


def _p(a):
    return ctypes.c_void_p(a.ctypes.data)


def _bits(x: torch.Tensor) -> np.ndarray:
    """bf16 tensor -> contiguous uint16 bit pattern array."""
    return np.ascontiguousarray(x.contiguous().view(torch.int16).numpy().view(np.uint16))


def _from_bits(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)


I64 = ctypes.c_int64


def group_quant(x, bm, bn, clamp, eps_mode=0, inv_mode=0, scale_bf16=False):
    """x bf16 [B,M,N] -> (q int8 [B,M,N], s f32 [B,M/bm,N/bn])."""
    B, M, N = x.shape
    q = np.empty((B, M, N), np.int8)
    s = np.empty((B, M // bm, N // bn), np.float32)
    xb = _bits(x)
    lib().ti8ref_group_quant(_p(xb), I64(B), I64(M), I64(N), I64(bm), I64(bn), int(clamp), int(eps_mode),
                             int(inv_mode), int(scale_bf16), _p(q), _p(s))
    return torch.from_numpy(q), torch.from_numpy(s)


def gemm_i32(A, Bm):
    A = np.ascontiguousarray(A.numpy())
    Bm = np.ascontiguousarray(Bm.numpy())
    M, K = A.shape
    N = Bm.shape[0]
    C = np.empty((M, N), np.int32)
    lib().ti8ref_gemm_i32(_p(A), _p(Bm), I64(M), I64(N), I64(K), _p(C))
    return torch.from_numpy(C)


def gemm_promote(A, Bm, sA, modeA, sB, modeB, combine=0, out_scale=1.0):
    A = np.ascontiguousarray(A.numpy())
    Bm = np.ascontiguousarray(Bm.numpy())
    sA = np.ascontiguousarray(sA.numpy().astype(np.float32))
    sB = np.ascontiguousarray(sB.numpy().astype(np.float32))
    M, K = A.shape
    N = Bm.shape[0]
    C = np.empty((M, N), np.uint16)
    accf = np.empty((M, N), np.float32)
    lib().ti8ref_gemm_promote(_p(A), _p(Bm), _p(sA), int(modeA), _p(sB), int(modeB), I64(M), I64(N), I64(K),
                              int(combine), ctypes.c_float(out_scale), _p(C), _p(accf))
    return _from_bits(C), torch.from_numpy(accf)


def dequant_rows(acc, sA, sB, inv_k=0.0):
    acc = np.ascontiguousarray(acc.numpy().astype(np.int32))
    sA = np.ascontiguousarray(sA.numpy().astype(np.float32))
    sB = np.ascontiguousarray(sB.numpy().astype(np.float32))
    M, N = acc.shape
    C = np.empty((M, N), np.uint16)
    lib().ti8ref_dequant_rows(_p(acc), _p(sA), _p(sB), I64(M), I64(N), ctypes.c_float(np.float32(inv_k)), _p(C))
    return _from_bits(C)


def fwht_f32(x: torch.Tensor, n: int) -> torch.Tensor:
    a = np.ascontiguousarray(x.to(torch.float32).numpy()).copy()
    rows = a.size // n
    lib().ti8ref_fwht_f32(_p(a), I64(rows), I64(n))
    return torch.from_numpy(a)
