"""Pins the oracle's quantisers: against the independent scalar C restatement (bit for
bit), against planted ties / zero groups / outliers whose answers follow from the
formula by hand, and against invariants any correct absmax quantiser satisfies."""
import numpy as np
import pytest
import torch

from conftest import bits_equal, make_gen, randn_bf16
from oracle import block_channel_bwd33 as obb
from oracle import block_channel_fwd32 as obf
from oracle import cref
from oracle import double_channel_fwd32 as odf
from oracle import fused_fwd32 as off
from oracle import tilelang_block_channel_fwd as otf

F32 = np.float32


def planted(gen, B=2, M=256, N=384):
    x = randn_bf16(gen, B, M, N)
    x[0, :128, :128] = 0                      # an all-zero block: amax falls back to 1e-4
    x[0, 128:, 128:256] *= 1e-6               # a block below the 1e-4 floor
    x[1, 3, 200] = 1000.0                     # an outlier that squashes its block
    x[1, 130:140, :] = -x[1, 130:140, :].abs()  # negative absmax
    return x


def test_block_quant_matches_scalar_c():
    x = planted(make_gen(1))
    for clamp in (True, False):
        q, s = obf.block_quant(x, clamp)
        qc, sc = cref.group_quant(x, 128, 128, clamp)
        assert bits_equal(q, qc) and bits_equal(s, sc)
    q, s = otf.triton_per_block_quant(x[:, :, :256])
    qc, sc = cref.group_quant(x[:, :, :256].contiguous(), 128, 256, False, scale_bf16=True)
    assert bits_equal(q, qc) and bits_equal(s, sc)


def test_token_and_row_quant_match_scalar_c():
    x = planted(make_gen(2))[0]
    q, s = obf.triton_per_token_quant(x)
    qc, sc = cref.group_quant(x[None], 1, x.shape[1], True)
    assert bits_equal(q, qc[0]) and bits_equal(s.flatten(), sc.flatten())
    x2 = randn_bf16(make_gen(3), 16, 4096)
    q, s = odf.triton_per_row_quant_2d(x2)
    qc, sc = cref.group_quant(x2[None], 1, 4096, True, inv_mode=1)
    assert bits_equal(q, qc[0]) and bits_equal(s, sc.flatten())
    q, s = odf.row_quant(x2, rcp_mul=True)
    qc, sc = cref.group_quant(x2[None], 1, 4096, True, inv_mode=2)
    assert bits_equal(q, qc[0]) and bits_equal(s, sc.flatten())


def test_fused_quant_matches_scalar_c():
    x = planted(make_gen(4))
    q, s = off.tile_quant_additive_eps(x, 128)
    qc, sc = cref.group_quant(x, 128, 128, False, eps_mode=1, inv_mode=3)
    assert bits_equal(q, qc) and bits_equal(s, sc)
    q, s = off.tile_quant_additive_eps(x, 1)
    qc, sc = cref.group_quant(x, 1, 128, False, eps_mode=1, inv_mode=3)
    assert bits_equal(q, qc) and bits_equal(s, sc)


def test_known_answers_by_hand():
    # one block whose absmax is exactly 127: scale = 127/127 = 1, so q = floor(x + 0.5)
    x = torch.zeros(1, 128, 128)
    x[0, 0, 0] = 127.0
    vals = torch.tensor([0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 0.49, -0.51, 126.5, -126.5, -127.0])
    x[0, 1, :vals.numel()] = vals
    q, s = obf.block_quant(x.to(torch.bfloat16), clamp=True)
    # ties round UP (toward +inf): 0.5->1, -0.5->0, 1.5->2, -1.5->-1, 2.5->3, -2.5->-2
    # bf16(0.49)=0.490234.. -> 0 ; bf16(-0.51)=-0.5117.. -> floor(-0.0117)= -1
    expect = torch.tensor([1, 0, 2, -1, 3, -2, 0, -1, 127, -126, -127], dtype=torch.int8)
    assert torch.equal(q[0, 1, :vals.numel()], expect)
    assert q[0, 0, 0] == 127 and float(s[0, 0, 0]) == 1.0
    # all-zero block: amax -> fp32(1e-4); scale = 127/1e-4; stored 1/scale
    z = torch.zeros(1, 128, 128, dtype=torch.bfloat16)
    q, s = obf.block_quant(z, clamp=True)
    scale = F32(127.0) / F32(1e-4)
    assert int(q.abs().max()) == 0 and F32(s[0, 0, 0].item()) == F32(1.0) / scale
    # two-pass row quantiser stores amax/127 (one division), block kernel 1/(127/amax)
    r = torch.full((1, 2048), 3.0, dtype=torch.bfloat16)
    _, s_row = odf.triton_per_row_quant_2d(r)
    assert F32(s_row[0].item()) == F32(3.0) / F32(127.0)
    _, s_tok = obf.triton_per_token_quant(r)
    assert F32(s_tok[0, 0].item()) == F32(1.0) / (F32(127.0) / F32(3.0))
    # fused: additive eps
    _, s_f = off.tile_quant_additive_eps(r.reshape(1, 1, 2048)[:, :, :128].expand(1, 128, 128).contiguous(), 128)
    assert F32(s_f[0, 0, 0].item()) == F32(127.0) / (F32(3.0) + F32(1e-5))


@pytest.mark.parametrize("seed", [0, 1])
def test_invariants(seed):
    g = make_gen(10 + seed)
    x = randn_bf16(g, 2, 256, 256) * 3
    q, s = obf.block_quant(x, clamp=True)
    qv = q.reshape(2, 2, 128, 2, 128).float()
    # every block reaches +-127 at its absmax element and nowhere exceeds it
    assert torch.equal(qv.abs().amax(dim=(2, 4)), torch.full((2, 2, 2), 127.0))
    # reconstruction error is at most half a step (plus fp32 rounding of the product)
    sx = s.repeat_interleave(128, 1).repeat_interleave(128, 2)
    err = (x.float() - q.float() * sx).abs()
    assert bool((err <= sx * (0.5 + 1e-4)).all())  # half a step + fp32 rounding of x*scale, 1/scale
    # a 128x128 block quantisation commutes with transposition
    qt, st = obb.triton_per_block_quant(x.transpose(1, 2))
    assert torch.equal(qt, q.transpose(1, 2)) and torch.equal(st, s.transpose(1, 2))
    # clamped and unclamped agree on finite data
    q2, s2 = obf.block_quant(x, clamp=False)
    assert torch.equal(q, q2) and torch.equal(s, s2)
    # sign symmetry away from ties: q(-x) == -q(x) unless x*scale is a half-integer
    qn, _ = obf.block_quant(-x, clamp=True)
    scale = (np.float32(127.0) / s.numpy().astype(np.float32))  # ~ multiplier, only to find ties
    frac = (x.float() * (127.0 / x.float().reshape(2, 2, 128, 2, 128).abs().amax(dim=(2, 4), keepdim=True)
                         ).expand(2, 2, 128, 2, 128).reshape(2, 256, 256))
    tie = (frac - torch.floor(frac) - 0.5).abs() < 1e-3
    assert bool(((qn == -q) | tie).all())


def test_row_quant_brute_force_python():
    """Element-at-a-time numpy float32 evaluation of the formula on a tiny input."""
    g = make_gen(21)
    x = randn_bf16(g, 3, 128)
    q, s = obf.triton_per_token_quant(x)
    xf = x.float().numpy()
    for r in range(3):
        amax = F32(0)
        for v in xf[r]:
            amax = max(amax, F32(abs(v)))
        amax = amax if amax > F32(1e-4) else F32(1e-4)
        scale = F32(127.0) / amax
        for c in range(128):
            e = int(np.floor(F32(F32(xf[r, c]) * scale) + F32(0.5)))
            e = min(max(e, -128), 127)
            assert int(q[r, c]) == e
        assert F32(s[r, 0].item()) == F32(1.0) / scale


def test_reference_torch_quantisers_differ_only_on_ties():
    """The author's pure-torch quantiser (round-half-even, +-127 clamp, bf16 math) is kept
    for documentation; it must stay close to the kernel formula (|dq| <= 1)."""
    x = randn_bf16(make_gen(5), 64, 256)
    q_ref, _ = otf.per_token_cast_to_int8(x)
    q, _ = obf.triton_per_token_quant(x)
    assert int((q_ref.int() - q.int()).abs().max()) <= 1


def _bf16_round(a):
    """fp32 numpy array -> nearest bf16 (ties to even), as fp32."""
    u = np.asarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32)


def test_torch_cast_quantisers_closed_form():
    """The reference's pure-torch quantisers, pinned against a numpy evaluation with every rounding
    written out: torch turns ``127.0 / amax`` into reciprocal(amax) * 127 (two roundings), rounds half
    to even, and on a bf16 tensor rounds every intermediate (x * scale included) to bf16.  This is
    the arithmetic the HIP kernels implement for TI8_Q_TORCH_ROUND / TI8_Q_TORCH_BF16."""
    from oracle import tilelang_block_channel_bwd as otb
    x = randn_bf16(make_gen(31), 2, 256, 384)
    x[0, :128, :128] = 0                       # all-zero block: the 1e-4 floor
    x[1, 130, 200] = 37.25
    # planted exact ties of x * scale: the block maximum 127 makes scale exactly 1
    x[1, 128:256, 256:384] = torch.tensor([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 127.0, 3.0] * 16).to(torch.bfloat16)
    xf = x.float().numpy()
    blocks = xf.reshape(2, 2, 128, 3, 128)
    amax = np.abs(blocks).max(axis=(2, 4), keepdims=True)
    # fp32 variant (tilelang/block_channel_bwd.py:96-104)
    a32 = np.maximum(amax, np.float32(1e-4))
    scale = (np.float32(1.0) / a32) * np.float32(127.0)
    q = np.clip(np.rint(blocks * scale), -127, 127).astype(np.int8).reshape(2, 256, 384)
    s = (np.float32(1.0) / scale).reshape(2, 2, 3)
    qo, so = otb.per_block_cast_to_int8(x)
    assert so.dtype == torch.float32 and np.array_equal(qo.numpy(), q) and np.array_equal(so.numpy().view(np.uint32), s.view(np.uint32))
    assert qo[1, 128, 256:264].tolist() == [0, 2, 2, 0, -2, -2, 127, 3]       # half to even (the kernels' floor(x + 0.5): 1, 2, 3, 0, -1, -2)
    # bf16 variant (tilelang/block_channel_fwd.py:222-230)
    ab = np.maximum(amax, _bf16_round(np.float32(1e-4)))
    scale = _bf16_round(_bf16_round(np.float32(1.0) / ab) * np.float32(127.0))
    q = np.clip(np.rint(_bf16_round(blocks * scale)), -127, 127).astype(np.int8).reshape(2, 256, 384)
    s = _bf16_round(np.float32(1.0) / scale).reshape(2, 2, 3)
    qo, so = otf.per_block_cast_to_int8(x)
    assert so.dtype == torch.bfloat16 and np.array_equal(qo.numpy(), q) and np.array_equal(so.float().numpy(), s)
    # per row, bf16 (tilelang/block_channel_fwd.py:215-220)
    rows = xf[1]
    ab = np.maximum(np.abs(rows).max(axis=1, keepdims=True), _bf16_round(np.float32(1e-4)))
    scale = _bf16_round(_bf16_round(np.float32(1.0) / ab) * np.float32(127.0))
    q = np.clip(np.rint(_bf16_round(rows * scale)), -127, 127).astype(np.int8)
    qo, so = otf.per_token_cast_to_int8(x[1])
    assert np.array_equal(qo.numpy(), q) and np.array_equal(so.float().numpy(), _bf16_round(np.float32(1.0) / scale))
