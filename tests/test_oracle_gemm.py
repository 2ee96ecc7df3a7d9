"""Pins the oracle's GEMMs: the integer part is exact by definition (checked against
float64 matmul, torch._int_mm and special cases); the promotion / epilogue against the
scalar C restatement bit for bit and against a float64 evaluation within fp32 rounding."""
import numpy as np
import pytest
import torch

from conftest import bits_equal, make_gen, randn_bf16, rel_err
from oracle import block_channel_bwd33 as obb
from oracle import block_channel_fwd32 as obf
from oracle import cref
from oracle import double_channel_bwd33 as odb
from oracle import double_channel_fwd32 as odf
from oracle import fused_bwd33 as ofb
from oracle import fused_fwd32 as off
from oracle import linear as olin
from oracle import tilelang_block_channel_bwd as otb
from oracle import tilelang_block_channel_fwd as otf
from oracle._prims import calc_diff, int_dot_k128, int_matmul_nt


def rand_i8(g, *shape):
    return torch.randint(-127, 128, shape, generator=g, dtype=torch.int8)


def test_integer_gemm_is_exact():
    g = make_gen(0)
    A, B = rand_i8(g, 192, 2304), rand_i8(g, 160, 2304)
    C = int_matmul_nt(A, B)
    assert torch.equal(C.double(), A.double() @ B.double().t())           # exact to 2^53
    assert torch.equal(C, torch._int_mm(A, B.t().contiguous()))
    assert torch.equal(C[:64, :48], cref.gemm_i32(A[:64], B[:48]))
    d = int_dot_k128(A[:, :128], B[:, :128])
    assert torch.equal(d.double(), A[:, :128].double() @ B[:, :128].double().t())


def test_integer_gemm_special_cases():
    K = 14336
    A = torch.full((128, K), 127, dtype=torch.int8)
    B = torch.full((128, K), -127, dtype=torch.int8)
    C = int_matmul_nt(A, B)
    assert int(C[0, 0]) == -K * 127 * 127 and bool((C == C[0, 0]).all())   # saturation, fits int32
    eye = torch.zeros(128, 128, dtype=torch.int8)
    eye[torch.arange(128), torch.arange(128)] = 1
    X = rand_i8(make_gen(1), 128, 128)
    assert torch.equal(int_matmul_nt(X, eye), X.int())                     # X @ I^T = X
    one = torch.zeros(128, 256, dtype=torch.int8)
    one[5, 77] = 3
    Y = rand_i8(make_gen(2), 128, 256)
    C = int_matmul_nt(one, Y)
    assert torch.equal(C[5], 3 * Y[:, 77].int()) and int(C.abs().sum()) == int(C[5].abs().sum())
    # transposing the operands transposes the result
    P, Q = rand_i8(make_gen(3), 128, 384), rand_i8(make_gen(4), 256, 384)
    assert torch.equal(int_matmul_nt(P, Q), int_matmul_nt(Q, P).t())


def quantised_operands(seed, B=1, M=128, N=256, K=512):
    g = make_gen(seed)
    a, b2, b3 = randn_bf16(g, B, M, K), randn_bf16(g, N, K), randn_bf16(g, B, N, K)
    return a, b2, b3


def test_block_channel_promotion_matches_scalar_c():
    a, b2, b3 = quantised_operands(5)
    qa, sa = obf.triton_per_block_quant(a)
    qb, sb = obf.triton_per_token_quant(b2)
    C = obf.triton_gemm(qa, qb, sa, sb)
    Cc, accf = cref.gemm_promote(qa[0], qb, sa[0], 1, sb.flatten(), 0, combine=0)
    assert bits_equal(C[0], Cc)
    qb3, sb3 = obb.triton_per_block_quant(b3)
    C = obb.triton_gemm(qa, qb3, sa, sb3)
    Cc, _ = cref.gemm_promote(qa[0], qb3[0], sa[0], 1, sb3[0], 1, combine=0)
    assert bits_equal(C[0], Cc)
    # float64 evaluation of the same sum: fp32 result within a few ulps of K/128 additions
    d64 = torch.zeros(128, 256, dtype=torch.float64)
    for kb in range(4):
        ks = slice(kb * 128, (kb + 1) * 128)
        d = qa[0, :, ks].double() @ qb[:, ks].double().t()
        d64 += d * sa[0, :, kb].double().repeat_interleave(128)[:, None] * sb.double().reshape(1, -1)
    assert rel_err(accf, d64) < 1e-6


def test_tilelang_and_fused_match_scalar_c():
    a, b2, b3 = quantised_operands(6)
    qa, sa = otf.triton_per_block_quant(a)
    qb, sb = otf.triton_per_token_quant(b2)
    C = otf.tl_gemm(qa, qb, torch.zeros(1, 128, 256, dtype=torch.bfloat16), sa, sb)
    Cc, _ = cref.gemm_promote(qa[0], qb, sa[0], 3, sb.flatten(), 0, combine=1)
    assert bits_equal(C[0], Cc)
    qa2, sa2 = otb.triton_per_block_quant(a)
    qb3, sb3 = otb.triton_per_block_quant(b3)
    C = otb.tl_gemm(qa2, qb3, torch.zeros(1, 128, 256, dtype=torch.bfloat16), sa2, sb3)
    Cc, _ = cref.gemm_promote(qa2[0], qb3[0], sa2[0], 1, sb3[0], 1, combine=1)
    assert bits_equal(C[0], Cc)
    # fused: quantisers with additive eps, division by the multiplier product
    qf, sf = off.tile_quant_additive_eps(a, 128)
    qg, sg = off.tile_quant_additive_eps(b2[None], 1)
    C = off.fused_gemm_from_quant(qf, sf, qg, sg, 1)
    Cc, _ = cref.gemm_promote(qf[0], qg[0], sf[0], 1, sg[0], 2, combine=2)
    assert bits_equal(C[0], Cc)
    assert bits_equal(C, off.fwd_32(a, b2))
    qh, sh = off.tile_quant_additive_eps(b3, 128)
    C = ofb.bwd_33(a, b3)
    Cc, _ = cref.gemm_promote(qf[0], qh[0], sf[0], 1, sh[0], 1, combine=2)
    assert bits_equal(C[0], Cc)


def test_double_channel_epilogue_matches_scalar_c():
    g = make_gen(7)
    a, b2 = randn_bf16(g, 1, 128, 2048), randn_bf16(g, 256, 2048)
    qa, sa = odf.triton_per_row_quant_3d(a)
    qb, sb = odf.triton_per_row_quant_2d(b2)
    acc = odf.gemm_i32(qa, qb)
    assert torch.equal(acc[0], cref.gemm_i32(qa[0], qb))
    C = odf.triton_gemm(qa, qb, sa, sb)
    assert bits_equal(C[0], cref.dequant_rows(acc[0], sa[0], sb))
    # with the pipeline's C * inv_K second rounding
    C2 = odf.scale_bf16(C, 1.0 / 2048)
    assert bits_equal(C2[0], cref.dequant_rows(acc[0], sa[0], sb, inv_k=1.0 / 2048))
    # int32 -> fp32 is inexact above 2^24: the epilogue must round to nearest even there
    big = torch.tensor([[2 ** 24 + 1, 2 ** 24 + 3, -(2 ** 25 + 2), 123456789]], dtype=torch.int32)
    one = torch.ones(1)
    out = odf.dequant_epilogue(big[None], one[None], torch.ones(4), torch.float32)
    assert out[0, 0].tolist() == [float(2 ** 24), float(2 ** 24 + 4), -float(2 ** 25 + 4 - 4), 123456792.0]


@pytest.mark.parametrize("mod,three_d", [(obf, False), (obb, True), (odf, False), (odb, True), (off, False),
                                         (ofb, True), (otf, False), (otb, True)])
def test_reference_acceptance_bar(mod, three_d):
    """The reference's only self-check: calc_diff(C, bf16 matmul) < 1e-3 on N(0,1)
    (triton/block_channel_fwd32.py:257-272 and the same block in every script)."""
    g = make_gen(8)
    a = randn_bf16(g, 2, 256, 2048)
    b = randn_bf16(g, 2, 384, 2048) if three_d else randn_bf16(g, 384, 2048)
    fn = mod.bwd_33 if three_d else mod.fwd_32
    C = fn(a, b)
    ref = torch.matmul(a.float(), b.float().transpose(-1, -2))
    assert C.dtype == torch.bfloat16 and C.shape == (2, 256, 384)
    assert float(calc_diff(C, ref)) < 1e-3


def test_linear_wiring_reduces_to_the_entry_points():
    g = make_gen(9)
    X, W = randn_bf16(g, 256, 512), randn_bf16(g, 384, 512, std=0.02)
    dY = randn_bf16(g, 256, 384, std=1e-3)
    Y, dX, dW = olin.linear_fwd_bwd(X, W, dY, "block_channel")
    assert bits_equal(Y, obf.fwd_32(X[None], W)[0])
    assert bits_equal(dX, obf.fwd_32(dY[None], W.t().contiguous())[0])
    assert bits_equal(dW, obb.bwd_33(dY.t()[None], X.t()[None])[0])
    for scheme, h in (("block_channel", None), ("row_block", None), ("double_channel", None),
                      ("block_channel", 128), ("row_block", 128)):
        Y, dX, dW = olin.linear_fwd_bwd(X, W, dY, scheme, h)
        assert float(calc_diff(Y, X.float() @ W.float().t())) < 1e-3
        assert float(calc_diff(dX, dY.float() @ W.float())) < 1e-3
        assert float(calc_diff(dW, dY.float().t() @ X.float())) < 1e-3


def test_config1_plumbing_forward_as_worded():
    """BASELINE config 1 as worded, on the CPU: block-channel INT8 linear forward, X 2048 x 4096 bf16
    ~N(0,1) with 1 % of the input channels x20, W 4096 x 4096 ~N(0,0.02), per-token scale on X,
    per-128x128-block scale on W, round to nearest, int32 matmul, bf16 out = acc * sx * sw, seed 0."""
    import numpy as np
    from oracle import linear as olin
    g = torch.Generator().manual_seed(0)
    M, K, N = 2048, 4096, 4096
    X = torch.randn(M, K, generator=g)
    X[:, torch.randperm(K, generator=g)[: K // 100 + 1]] *= 20.0
    X = X.to(torch.bfloat16)
    W = (torch.randn(N, K, generator=g) * 0.02).to(torch.bfloat16)
    xq, xs = olin.quant2d(X, olin.ROW, clamp=True)
    wq, ws = olin.quant2d(W, olin.BLOCK, clamp=True)
    # quantiser invariants: every group reaches 127, codes reconstruct x within half a step
    assert int(xq.abs().amax(dim=1).min()) == 127 and xs.shape == (M,)
    assert int(wq.reshape(N // 128, 128, K // 128, 128).abs().amax(dim=(1, 3)).min()) == 127 and ws.shape == (N // 128, K // 128)
    assert bool(((X.float() - xq.float() * xs[:, None]).abs() <= xs[:, None] * (0.5 + 1e-4)).all())
    wsx = ws.repeat_interleave(128, 0).repeat_interleave(128, 1)
    assert bool(((W.float() - wq.float() * wsx).abs() <= wsx * (0.5 + 1e-4)).all())
    Y = olin.gemm_scaled(xq, xs, olin.ROW, wq, ws, olin.BLOCK)
    assert Y.dtype == torch.bfloat16 and Y.shape == (M, N)
    # the whole path equals the layer entry point of that scheme, and a sampled block of the integer
    # GEMM equals an int64 evaluation
    assert torch.equal(Y, olin.linear_fwd_bwd(X, W, torch.zeros(M, N, dtype=torch.bfloat16), "row_block")[0])
    r, c = slice(1024, 1088), slice(512, 640)
    acc = (xq[r, :128].long() @ wq[c, :128].long().t())
    part = olin.gemm_scaled(xq[r, :128], xs[r], olin.ROW, wq[c, :128], ws[4:5, :1], olin.BLOCK, out_dtype=torch.float32)
    want = (acc.double() * xs[r, None].double() * float(ws[4, 0])).float()
    assert np.allclose(part.numpy(), want.numpy(), rtol=3e-7, atol=0)
    # against the bf16 product: 1 % of the channels x20 costs int8 resolution, well inside 1e-2
    ref = X.float() @ W.float().t()
    from oracle._prims import calc_diff
    assert float(calc_diff(Y, ref)) < 2e-3
