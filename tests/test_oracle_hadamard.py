"""Pins the oracle's Walsh-Hadamard transform against what the mathematics fixes:
scipy's Sylvester matrix, H(H(x)) = n x, one-hot rows, exactness on small integers."""
import numpy as np
import pytest
import scipy.linalg
import torch

from conftest import bits_equal, make_gen, randn_bf16
from oracle import cref
from oracle.hadamard import fwht_f32, hadamard128, hadamard_transform


@pytest.mark.parametrize("n", [128, 256, 2048])
def test_equals_sylvester_matrix_on_integers(n):
    g = make_gen(n)
    x = torch.randint(-8, 9, (5, n), generator=g).float()        # sums stay far below 2^24: exact
    H = torch.from_numpy(scipy.linalg.hadamard(n).astype(np.float32))
    assert torch.equal(fwht_f32(x, n), x @ H)
    # H[i, j] = (-1)^popcount(i & j): the transform of a one-hot is a row of H
    e = torch.zeros(1, n)
    e[0, 37] = 1
    row = fwht_f32(e, n)[0]
    expect = torch.tensor([(-1.0) ** bin(37 & j).count("1") for j in range(n)])
    assert torch.equal(row, expect)


def test_involution_and_orthogonality():
    x = torch.randint(-4, 5, (3, 512), generator=make_gen(1)).float()
    assert torch.equal(fwht_f32(fwht_f32(x, 512), 512), 512 * x)
    # Parseval: |Hx|^2 = n |x|^2
    y = fwht_f32(x, 128)
    assert float((y * y).sum()) == 128 * float((x * x).sum())


def test_matches_scalar_c_butterflies_bit_for_bit():
    x = torch.randn(7, 4096, generator=make_gen(2))
    for n in (128, 1024, 4096):
        assert bits_equal(fwht_f32(x, n), cref.fwht_f32(x, n).reshape(7, 4096))


def test_bf16_interface_and_block_diagonal():
    x = randn_bf16(make_gen(3), 4, 1024)
    y = hadamard_transform(x)
    assert y.dtype == torch.bfloat16 and y.shape == x.shape
    H = torch.from_numpy(scipy.linalg.hadamard(1024).astype(np.float64))
    ref = x.double() @ H
    assert float((y.double() - ref).norm() / ref.norm()) < 4e-3          # one bf16 rounding
    yb = hadamard128(x)
    H128 = torch.from_numpy(scipy.linalg.hadamard(128).astype(np.float64))
    refb = (x.double().reshape(4, 8, 128) @ H128).reshape(4, 1024)
    assert float((yb.double() - refb).norm() / refb.norm()) < 4e-3
    # along another dim = transpose, transform, transpose back
    assert bits_equal(hadamard128(x.t().contiguous(), dim=0), hadamard128(x).t().contiguous())


@pytest.mark.parametrize("dim", [96, 384, 1792])
def test_a_length_that_is_no_power_of_two_is_zero_extended_and_cut_back(dim):
    """The external library's documented rule for such a length (the reference hands it K = 14336 of the Llama MLP
    unchanged, triton/double-channle_fwd32.py:299-300): pad with zeros to the next power of two, multiply by H, keep the
    first `dim` outputs.  Against scipy's matrix on small integers (exact), and NOT an orthogonal map."""
    n = 1 << (dim - 1).bit_length()
    g = make_gen(dim)
    x = torch.zeros(5, dim)
    for r in range(5):      # 40 small integers per row: every output is an integer below 128 in magnitude, exact also in bf16
        x[r, torch.randperm(dim, generator=g)[:40]] = torch.randint(1, 4, (40,), generator=g).float() * (torch.randint(0, 2, (40,), generator=g) * 2 - 1)
    x = x.to(torch.bfloat16)
    H = torch.from_numpy(scipy.linalg.hadamard(n).astype(np.float32))
    want = (torch.nn.functional.pad(x.float(), (0, n - dim)) @ H)[:, :dim]
    assert float(want.abs().max()) < 256                                      # representable in bf16
    assert torch.equal(hadamard_transform(x).float(), want)
    # = the first `dim` columns of the first `dim` rows of H_n: a one-hot gives that row of H, cut
    e = torch.zeros(1, dim, dtype=torch.bfloat16)
    e[0, dim - 1] = 1
    assert torch.equal(hadamard_transform(e)[0].float(), H[dim - 1, :dim])
    # power-of-two lengths are untouched by the rule
    y = randn_bf16(g, 3, 256)
    assert bits_equal(hadamard_transform(y), fwht_f32(y.float(), 256).to(torch.bfloat16))
