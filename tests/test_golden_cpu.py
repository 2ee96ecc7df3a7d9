"""The oracle (and the scalar C restatement) reproduce the committed golden vectors, so a
later change of either cannot silently redefine what the GPU kernels are checked against."""
import torch

from conftest import bits_equal
from golden_util import bf16, load, t
from oracle import block_channel_bwd33 as obb
from oracle import block_channel_fwd32 as obf
from oracle import cref
from oracle import double_channel_fwd32 as odf
from oracle import fused_fwd32 as off
from oracle import linear as olin
from oracle import tilelang_block_channel_fwd as otf
from oracle.hadamard import fwht_f32, hadamard_transform


def test_quant_vectors():
    z = load("quant_256x256.npz")
    x = bf16(z["x"])
    for got, q, s in ((obf.triton_per_block_quant(x), "block_q", "block_s"),
                      (obf.triton_per_token_quant(x[0]), "token_q", "token_s"),
                      (odf.row_quant(x[0], BLOCK_N=128), "row_q", "row_s"),
                      (otf.triton_per_block_quant(x), "tl_block_q", "tl_block_s"),
                      (off.tile_quant_additive_eps(x, 128), "fused_a_q", "fused_a_s"),
                      (off.tile_quant_additive_eps(x, 1), "fused_b_q", "fused_b_s")):
        assert bits_equal(got[0], t(z[q])) and bits_equal(got[1], t(z[s])), q
    # the planted ties in the scale-1 block: round half up
    q = t(z["block_q"])[0, 130, 130:140]
    assert q.tolist() == [127, 1, 0, 2, -1, 3, -2, 64, -63, 127]
    assert float(t(z["block_s"])[0, 1, 1]) == 1.0
    # scalar C agrees with the fixture too
    qc, sc = cref.group_quant(x, 128, 128, True)
    assert bits_equal(qc, t(z["block_q"])) and bits_equal(sc, t(z["block_s"]))


def test_gemm_vectors():
    z = load("gemm_128x128x512.npz")
    A, B = t(z["A"]), t(z["B"])
    acc = odf.gemm_i32(A[None], B)[0]
    assert bits_equal(acc, t(z["acc_i32"]))
    assert int(acc[0, 0]) == -512 * 127 * 127
    assert torch.equal(acc.double(), A.double() @ B.double().t())
    sAb, sBb, sAr, sBr = t(z["sA_block"]), t(z["sB_block"]), t(z["sA_row"]), t(z["sB_row"])
    assert bits_equal(obf.triton_gemm(A[None], B, sAb[None], sBr.reshape(-1, 1))[0], bf16(z["C_block_row"]))
    assert bits_equal(obb.triton_gemm(A[None], B[None], sAb[None], sBb[None])[0], bf16(z["C_block_block"]))
    assert bits_equal(odf.triton_gemm(A[None], B, sAr[None], sBr)[0], bf16(z["C_row_row"]))
    assert bits_equal(cref.gemm_promote(A, B, sAb, 1, sBr, 0)[0], bf16(z["C_block_row"]))
    assert bits_equal(cref.dequant_rows(acc, sAr, sBr, 1.0 / 512), bf16(z["C_row_row_invk"]))
    assert bits_equal(cref.gemm_promote(A, B, sAr, 0, sBb, 1)[0], bf16(z["C_row_block"]))


def test_fwht_vectors():
    z = load("fwht.npz")
    xi, xr = bf16(z["x_int"]), bf16(z["x_rand"])
    assert bits_equal(fwht_f32(xi.float(), 128).to(torch.bfloat16), bf16(z["h128_int"]))
    assert bits_equal(hadamard_transform(xi), bf16(z["h256_int"]))
    assert bits_equal(hadamard_transform(xr), bf16(z["h2048_rand"]))
    assert bits_equal(cref.fwht_f32(xr.float(), 128).reshape(8, 2048).to(torch.bfloat16), bf16(z["h128_rand"]))


def test_linear_vectors():
    z = load("linear_128x256x128.npz")
    X, W, dY = bf16(z["X"]), bf16(z["W"]), bf16(z["dY"])
    for scheme, h in (("block_channel", None), ("row_block", None), ("double_channel", None), ("block_channel", 128)):
        tag = scheme + ("_h128" if h else "")
        Y, dX, dW = olin.linear_fwd_bwd(X, W, dY, scheme, h)
        assert bits_equal(Y, bf16(z[tag + "_Y"])) and bits_equal(dX, bf16(z[tag + "_dX"])) and bits_equal(dW, bf16(z[tag + "_dW"]))
