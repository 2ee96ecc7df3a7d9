"""Oracle of the Walsh-Hadamard rotation used by the double-channel scripts.

TEST INFRASTRUCTURE.  The reference calls ``hadamard_transform`` from the external
fast_hadamard_transform CUDA extension (Dao-AILab, version unpinned; call sites
triton/double-channle_fwd32.py:273-274,299-300 and
triton/double_channel_bwd33.py:189-190,208-209).  Its published contract is
``hadamard_transform(x, scale=1.0) == x @ H_n * scale`` along the last dim with
H_n the Sylvester-ordered +-1 matrix, computed in fp32 and returned in the dtype
of ``x``.  That contract is restated here with a fixed butterfly schedule --
stage strides 1, 2, 4, ..., n/2, each stage ``(a, b) -> (a + b, a - b)`` with
``a`` the element whose index has the stride bit clear -- shared with the HIP
kernels.  The rounding order inside the external kernel is unavailable, so
results are **parity unpinned** against it beyond fp32 rounding error.
"""
import torch

from ._prims import F32, widen


def fwht_f32(xf: torch.Tensor, n: int) -> torch.Tensor:
    """Un-normalised FWHT over contiguous groups of ``n`` along the last dim, fp32."""
    assert n & (n - 1) == 0 and xf.shape[-1] % n == 0
    shape = xf.shape
    y = xf.reshape(-1, n).clone()
    h = 1
    while h < n:
        v = y.reshape(-1, n // (2 * h), 2, h)
        a = v[:, :, 0, :]
        b = v[:, :, 1, :]
        y = torch.stack((a + b, a - b), dim=2).reshape(-1, n)
        h *= 2
    return y.reshape(shape)


def hadamard_transform(x: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """Full-length transform along the last dim; bf16 in -> bf16 out (one rounding).

    A last dim that is no power of two is handled as the external library documents it
    ("if dim is not a power of 2, we implicitly pad x with zero so that dim is the next
    power of 2"; the result has the input's shape): zero-extended to the next power of two,
    transformed, cut back to the first ``dim`` elements."""
    dim = x.shape[-1]
    n = 1 << (dim - 1).bit_length()
    xf = widen(x)
    if n != dim:
        xf = torch.nn.functional.pad(xf, (0, n - dim))
    y = fwht_f32(xf, n)[..., :dim]
    if scale != 1.0:
        y = y * torch.tensor(scale, dtype=F32)
    return y.to(x.dtype)


def hadamard128(x: torch.Tensor, dim: int = -1) -> torch.Tensor:
    """Block-diagonal H_128 along ``dim`` (groups of 128 consecutive indices),
    un-normalised, rounded once to the input dtype."""
    xt = x.transpose(dim, -1)
    y = fwht_f32(widen(xt), 128).to(x.dtype)
    return y.transpose(dim, -1)
