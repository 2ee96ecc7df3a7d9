"""Build ``libti8.so`` (every HIP kernel + the C ABI) for gfx950 with hipcc.

Run as ``python triton-int8_amd/build.py`` or call :func:`build`.  The library is
written next to this file; it is cross-compiled, so no GPU is needed to build.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libti8.so")
SOURCES = ["api.hip", "quant.hip", "fwht.hip", "gemm.hip", "gemm_chain.hip", "gemm_skinny.hip", "step.hip", "probe.hip"]

# -ffp-contract=off: x*scale+0.5 must round twice (bit-exact quantisation); kernels
#   that want an fma ask for one explicitly.
# -packed-fp32-ops disabled: keep hipcc from forming v_pk_*_f32 from scalar float code.
# -amdgpu-mfma-vgpr-form: MFMA accumulators in ordinary VGPRs, so the block-channel promotion
#   (convert + fma on every 128-deep partial) reads them without v_accvgpr_read copies.
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-ffp-contract=off",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument",
         "-mllvm", "-amdgpu-mfma-vgpr-form"]


def build(verbose: bool = False) -> str:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc] + FLAGS + ["-o", LIB] + [os.path.join(CSRC, s) for s in SOURCES]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out:
        print(out)
    return LIB


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
