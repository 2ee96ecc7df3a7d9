"""Writes the small golden fixtures under tests/golden/ from the CPU oracle.

The reference ships no golden vectors (its only checks are run-time random
self-tests), so these are produced by this repository's oracle, which the
``test_oracle_*`` tests pin independently.  Inputs are seeded and planted with the
edge cases of the domain (ties, all-zero groups, sub-epsilon groups, outliers,
+-127 saturation).  Run from the repository root:

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import block_channel_bwd33 as obb  # noqa: E402
from oracle import block_channel_fwd32 as obf  # noqa: E402
from oracle import double_channel_fwd32 as odf  # noqa: E402
from oracle import fused_fwd32 as off  # noqa: E402
from oracle import linear as olin  # noqa: E402
from oracle import tilelang_block_channel_fwd as otf  # noqa: E402
from oracle.hadamard import fwht_f32, hadamard_transform  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def bits(x):
    return x.contiguous().view(torch.int16).numpy().view(np.uint16)


def planted_input(seed, M=256, N=256):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(1, M, N, generator=g)
    x[0, :128, :128] = 0.0                        # all-zero block
    x[0, 128:, :128] *= 1e-6                      # block under the 1e-4 floor
    x[0, 7, 200] = 977.0                          # outlier
    x[0, 130, 130:140] = torch.tensor([127.0, 0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 63.5, -63.5, 126.5])
    x[0, 128:, 128:] = x[0, 128:, 128:].clamp(-127, 127)   # block absmax exactly 127 -> scale 1, exact ties
    x[0, 130, 130] = 127.0
    return x.to(torch.bfloat16)


def main():
    x = planted_input(0)
    out = {"x": bits(x)}
    q, s = obf.triton_per_block_quant(x)
    out["block_q"], out["block_s"] = q.numpy(), s.numpy()
    q, s = obf.triton_per_token_quant(x[0])
    out["token_q"], out["token_s"] = q.numpy(), s.numpy()
    q, s = odf.row_quant(x[0], BLOCK_N=128)
    out["row_q"], out["row_s"] = q.numpy(), s.numpy()
    q, s = otf.triton_per_block_quant(x)
    out["tl_block_q"], out["tl_block_s"] = q.numpy(), s.numpy()
    q, s = off.tile_quant_additive_eps(x, 128)
    out["fused_a_q"], out["fused_a_s"] = q.numpy(), s.numpy()
    q, s = off.tile_quant_additive_eps(x, 1)
    out["fused_b_q"], out["fused_b_s"] = q.numpy(), s.numpy()
    q, s = obf.token_quant(x[0].t().contiguous(), True)
    out["col_qT"], out["col_s"] = q.numpy(), s.numpy().reshape(-1)
    np.savez_compressed(os.path.join(HERE, "quant_256x256.npz"), **out)

    g = torch.Generator().manual_seed(1)
    A = torch.randint(-127, 128, (128, 512), generator=g, dtype=torch.int8)
    B = torch.randint(-127, 128, (128, 512), generator=g, dtype=torch.int8)
    A[0, :] = 127
    B[0, :] = -127                                 # one saturated accumulator: -512*127^2
    sAb = (torch.rand(1, 4, generator=g) * 0.05 + 1e-3)
    sBb = (torch.rand(1, 4, generator=g) * 0.05 + 1e-3)
    sAr = (torch.rand(128, generator=g) * 0.05 + 1e-3)
    sBr = (torch.rand(128, generator=g) * 0.05 + 1e-3)
    out = {"A": A.numpy(), "B": B.numpy(), "sA_block": sAb.numpy(), "sB_block": sBb.numpy(),
           "sA_row": sAr.numpy(), "sB_row": sBr.numpy()}
    out["acc_i32"] = odf.gemm_i32(A[None], B)[0].numpy()
    out["C_block_row"] = bits(obf.triton_gemm(A[None], B, sAb[None], sBr.reshape(-1, 1))[0])
    out["C_block_block"] = bits(obb.triton_gemm(A[None], B[None], sAb[None], sBb[None])[0])
    out["C_row_row"] = bits(odf.triton_gemm(A[None], B, sAr[None], sBr)[0])
    out["C_row_row_invk"] = bits(odf.scale_bf16(odf.triton_gemm(A[None], B, sAr[None], sBr), 1.0 / 512)[0])
    out["C_row_block"] = bits(olin.gemm_scaled(A, sAr, olin.ROW, B, sBb, olin.BLOCK))
    np.savez_compressed(os.path.join(HERE, "gemm_128x128x512.npz"), **out)

    g = torch.Generator().manual_seed(2)
    xi = torch.randint(-16, 17, (8, 256), generator=g).to(torch.bfloat16)     # exact in fp32 and bf16
    xr = torch.randn(8, 2048, generator=g).to(torch.bfloat16)
    out = {"x_int": bits(xi), "h128_int": bits(fwht_f32(xi.float(), 128).to(torch.bfloat16)),
           "h256_int": bits(hadamard_transform(xi)), "x_rand": bits(xr), "h2048_rand": bits(hadamard_transform(xr)),
           "h128_rand": bits(fwht_f32(xr.float(), 128).to(torch.bfloat16))}
    np.savez_compressed(os.path.join(HERE, "fwht.npz"), **out)

    g = torch.Generator().manual_seed(3)
    X = torch.randn(128, 256, generator=g).to(torch.bfloat16)
    X[:, torch.randperm(256, generator=g)[:3]] *= 20                         # outlier channels
    W = (torch.randn(128, 256, generator=g) * 0.02).to(torch.bfloat16)
    dY = (torch.randn(128, 128, generator=g) * 1e-3).to(torch.bfloat16)
    out = {"X": bits(X), "W": bits(W), "dY": bits(dY)}
    for scheme, h in (("block_channel", None), ("row_block", None), ("double_channel", None),
                      ("block_channel", 128)):
        Y, dX, dW = olin.linear_fwd_bwd(X, W, dY, scheme, h)
        tag = scheme + ("_h128" if h else "")
        out[tag + "_Y"], out[tag + "_dX"], out[tag + "_dW"] = bits(Y), bits(dX), bits(dW)
    np.savez_compressed(os.path.join(HERE, "linear_128x256x128.npz"), **out)
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")


if __name__ == "__main__":
    main()
