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


def assert_one_ulp(got, want, what="", slack=2.0 ** -18):
    """Every element of `got` within one bf16 ulp of `want`, plus `slack` x max|want| for the elements
    whose K-block terms cancel (re-associating the fp32 sum moves those by a few 2^-24 of the terms,
    which are of the size of the large elements, not of the result)."""
    got, want = got.float().cpu(), want.float().cpu()
    assert got.shape == want.shape, what
    bad = (got - want).abs() > bf16_ulp(want) + slack * want.abs().max()
    assert not bool(bad.any()), f"{what}: {int(bad.sum())} of {bad.numel()} elements off by more than one bf16 ulp, first at {bad.nonzero()[0].tolist()}"
