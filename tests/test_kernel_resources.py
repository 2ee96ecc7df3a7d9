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


def compile_to_asm(source, tmp_path):
    """Path of the gfx950 assembly of one kernel source, compiled with the library's own flags."""
    b = _build_module()
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    if not (os.path.exists(hipcc) or shutil.which(hipcc)):
        pytest.skip("hipcc not available")
    out = str(tmp_path / (source + ".s"))
    flags = [f for f in b.FLAGS if f not in ("-shared", "-fPIC")]
    res = subprocess.run([hipcc] + flags + ["--cuda-device-only", "-S", "-o", out, os.path.join(b.CSRC, source)],
                         stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert res.returncode == 0, res.stdout[-2000:]
    return out


def kernel_resources(source, tmp_path):
    out = compile_to_asm(source, tmp_path)
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


def test_persistent_chain_kernel_waits_match_its_stores(tmp_path):
    """The persistent kernel lets its epilogue stores drain under the next tile's first K tile: it waits with
    `s_waitcnt vmcnt(n)`, n = the stores a wave issued last, for everything issued BEFORE them (the next tile's operand
    and factor loads).  That is only safe while n does not exceed the stores really emitted, so the count in the source
    (EPILOGUE_STORES = 16: one 16-byte store per lane and row) is checked against the code the toolchain produces:
    every variant of the epilogue must hold exactly 16 global stores, all of them 16 bytes wide, and the two waits
    must carry that count (plus the 4 operand loads issued behind the factor loads)."""
    text = open(compile_to_asm("gemm_chain.hip", tmp_path)).read()
    body = text[text.index("gemm_i8_chain_kernel"):]
    body = body[:body.index(".end_amdhsa_kernel")]
    src = open(os.path.join(PKG, "csrc", "gemm_chain.hip")).read()
    m = re.search(r"static_assert\(RPI == 8 && STORES_PER_PASS == 2 && EPILOGUE_STORES == (\d+)", src)
    assert m, "the source no longer pins EPILOGUE_STORES"
    stores_per_wave = int(m.group(1))
    stores = re.findall(r"^\s*(global_store_\w+|buffer_store_\w+|flat_store_\w+|scratch_store_\w+)", body, flags=re.M)
    assert stores and set(stores) == {"global_store_dwordx4"}, sorted(set(stores))
    variants = 8          # extra factor x row scales x column scales, each a compile-time copy of the store loop
    assert len(stores) == variants * stores_per_wave, (len(stores), stores_per_wave)
    # straight-line check: between two branch targets / branches no more than one variant's stores
    for block in re.split(r"^\.LBB\S+:|^\s*s_cbranch\w+|^\s*s_branch", body, flags=re.M):
        n = len(re.findall(r"^\s*global_store_dwordx4", block, flags=re.M))
        assert n in (0, stores_per_wave), n
    waits = set(re.findall(r"s_waitcnt vmcnt\((\d+)\)", body))
    assert str(stores_per_wave) in waits, waits              # first K tile of a tile: everything but the stores
    assert str(stores_per_wave + 4) in waits, waits          # next tile's factors: behind 4 operand loads and the stores
    assert all(int(w) <= stores_per_wave + 4 for w in waits), waits
