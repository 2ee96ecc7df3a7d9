"""Helpers shared by the per-scheme modules."""
import time

import torch


def calc_diff(x, y):
    """1 - 2<x,y>/(|x|^2 + |y|^2) in float64: the reference's acceptance metric
    (triton/block_channel_fwd32.py:244-248, identical in every reference script)."""
    x, y = x.double(), y.double()
    denominator = (x * x + y * y).sum()
    sim = 2 * (x * y).sum() / denominator
    return 1 - sim


def need_bf16_out(out_dtype):
    if out_dtype != torch.bfloat16:
        raise ValueError(f"only out_dtype=torch.bfloat16 is supported, got {out_dtype}")


class StageTimer:
    """Opt-in reproduction of the reference pipelines' per-call `int8 time` / `kernel time`
    prints (triton/block_channel_fwd32.py:219-238).  The reference synchronises the device
    and prints on every call; here that only happens with ``verbose=True``."""

    def __init__(self, device, verbose):
        self.device, self.verbose = device, verbose

    def start(self):
        if self.verbose:
            torch.cuda.synchronize(self.device)
            self.t0 = time.time()

    def stop(self, label):
        if self.verbose:
            torch.cuda.synchronize(self.device)
            print(f"{label}:{(time.time() - self.t0) * 1000} ms")


def bf16_reference_nt(a, b):
    """bf16 ``a @ b^T`` over the last two dims, the product the reference's self-checks compare with
    (``torch.matmul(a, b.T)`` / ``torch.bmm(a, b.transpose(1, 2))``).  With a 3-D ``b`` it is
    evaluated batch by batch as 2-D products rather than as one batched call."""
    if b.dim() == 2:
        return torch.matmul(a, b.t())
    return torch.stack([torch.matmul(a[i], b[i].t()) for i in range(a.shape[0])])


def ceildiv(a, b):
    """tilelang/block_channel_bwd.py:91-92."""
    return (a + b - 1) // b
