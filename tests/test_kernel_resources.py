"""The hot GEMM kernels must fit the register file: a kernel that spills keeps running, only slower (its scratch
reloads wait behind the operand loads in flight), so nothing else would notice.  Compiles the two GEMM sources to
gfx950 assembly with the library's own flags (no GPU needed) and reads the kernel descriptors."""
import importlib.util
import os
import re
import shutil
import subprocess

import pytest

from conftest import ROOT

PKG = os.path.join(ROOT, "triton-int8_amd")


def _build_module():
    spec = importlib.util.spec_from_file_location("ti8_build", os.path.join(PKG, "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def kernel_resources(source, tmp_path):
    b = _build_module()
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    if not (os.path.exists(hipcc) or shutil.which(hipcc)):
        pytest.skip("hipcc not available")
    out = str(tmp_path / (source + ".s"))
    flags = [f for f in b.FLAGS if f not in ("-shared", "-fPIC")]
    res = subprocess.run([hipcc] + flags + ["--cuda-device-only", "-S", "-o", out, os.path.join(b.CSRC, source)],
                         stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert res.returncode == 0, res.stdout[-2000:]
    kernels = {}
    for m in re.finditer(r"\.amdhsa_kernel (\S+)(.*?)\.end_amdhsa_kernel", open(out).read(), flags=re.S):
        body = m.group(2)
        kernels[m.group(1)] = {k: int(re.search(r"\.amdhsa_" + k + r" (\d+)", body).group(1))
                               for k in ("private_segment_fixed_size", "next_free_vgpr", "next_free_sgpr")}
    return kernels


def test_persistent_chain_kernel_does_not_spill(tmp_path):
    kernels = kernel_resources("gemm_chain.hip", tmp_path)
    chain = [v for k, v in kernels.items() if "gemm_i8_chain_kernel" in k]
    assert len(chain) == 1
    assert chain[0]["private_segment_fixed_size"] == 0, chain[0]     # no scratch
    assert chain[0]["next_free_vgpr"] <= 256                          # two waves per SIMD


def test_tiled_gemm_kernels_do_not_spill(tmp_path):
    kernels = kernel_resources("gemm.hip", tmp_path)
    # 256 x 256 and 256 x 128 tiles run 8 waves of up to 256 registers; only the literal-arithmetic kernel (not tuned) may spill
    hot = {k: v for k, v in kernels.items() if "gemm_i8" in k and "ELi3EEE" not in k}
    assert len(hot) >= 8
    for name, v in hot.items():
        assert v["private_segment_fixed_size"] == 0, (name, v)
        assert v["next_free_vgpr"] <= 256, (name, v)
