import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def dev():
    return torch.device("cuda:0")


def make_gen(seed):
    return torch.Generator().manual_seed(seed)


def randn_bf16(gen, *shape, std=1.0):
    return (torch.randn(*shape, generator=gen) * std).to(torch.bfloat16)


def bits_equal(a, b):
    """Bit equality of two tensors of the same dtype (bf16 compared on its bit pattern)."""
    a, b = a.cpu(), b.cpu()
    if a.dtype != b.dtype or a.shape != b.shape:
        return False
    if a.dtype == torch.bfloat16:
        return bool((a.contiguous().view(torch.int16) == b.contiguous().view(torch.int16)).all())
    return bool((a == b).all())


def rel_err(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return float((a - b).norm() / b.norm().clamp_min(1e-300))


def bf16_ulp(v):
    """Spacing of bf16 numbers at |v| (as an fp32 tensor)."""
    _, e = torch.frexp(v.float().abs().clamp_min(2.0 ** -126))
    return torch.ldexp(torch.ones_like(v, dtype=torch.float32), e - 8)


def assert_promoted_close(got, want, mag, K, what=""):
    """The bar for the default (re-associated) block-channel promotion, per element:
        |got - want| <= 1 bf16 ulp of want + (K/128 + 4) * 2^-23 * mag
    with mag >= sum over the K blocks of |term|: what summing the same K/128 fp32 terms in another order, or with an
    fma, can move an element by.  It scales with the magnitudes that went into THAT element, so a small output next to
    large ones gets no extra room; a wrong scale, a dropped K tile or a misplaced tile is off by orders of magnitude more."""
    got, want, mag = got.float().cpu(), want.float().cpu(), mag.float().cpu()
    assert got.shape == want.shape == mag.shape, what
    bound = bf16_ulp(want) + (K // 128 + 4) * 2.0 ** -23 * mag
    bad = (got - want).abs() > bound
    assert not bool(bad.any()), f"{what}: {int(bad.sum())} of {bad.numel()} elements outside one bf16 ulp, first at {bad.nonzero()[0].tolist()}"
    assert torch.isfinite(got).all(), what


def product_magnitude(a, b, out_scale=1.0):
    """An upper bound of sum_kb |term_kb| of the quantised product a @ b^T from the bf16 operands themselves
    (a [..., M, K], b [..., N, K]): a dequantised code differs from its element by at most half a quantisation step,
    and no step exceeds max|operand| / 127, so sum_k (|a| + max|a|/254) (|b| + max|b|/254) bounds the sum of the
    magnitudes of all products, hence of the K-block terms.  For `assert_promoted_close` where the int8 operands and
    scales of the oracle are not at hand."""
    a, b = a.float().abs(), b.float().abs()
    a, b = a + a.max() / 254.0, b + b.max() / 254.0
    return (a @ b.transpose(-1, -2)) * (1.0 + 2.0 ** -10) * out_scale


def linear_magnitudes(X, W, dY, hadamard=None):
    """[(magnitude bound, contraction length)] for Y, dX, dW of the layer (X [..., K], W [N, K], dY [..., N]; tokens
    flattened), for `assert_promoted_close`.  With ``hadamard=128`` the operands are rotated as the layer rotates
    them (oracle.hadamard.hadamard128 along the contraction dim, zero-padded to 128) and the result carries 2^-7."""
    from oracle.hadamard import hadamard128
    X2, dY2 = X.reshape(-1, X.shape[-1]), dY.reshape(-1, dY.shape[-1])
    out = []
    for a, b in ((X2, W), (dY2, W.t()), (dY2.t(), X2.t())):
        pad = (-a.shape[1]) % 128
        a = torch.nn.functional.pad(a.contiguous(), (0, pad))
        b = torch.nn.functional.pad(b.contiguous(), (0, pad))
        if hadamard == 128:
            out.append((product_magnitude(hadamard128(a), hadamard128(b), 2.0 ** -7), a.shape[1]))
        else:
            out.append((product_magnitude(a, b), a.shape[1]))
    return out
