"""The C ABI library loads without a GPU, exports every symbol include/ti8.h declares,
and rejects bad arguments on the host (status code + message) before launching anything."""
import ctypes
import os
import re

import pytest

from conftest import ROOT

HEADER = os.path.join(ROOT, "include", "ti8.h")


@pytest.fixture(scope="module")
def lib():
    import triton_int8_amd
    return triton_int8_amd._lib.lib()


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ti8_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported(lib):
    names = declared_functions()
    assert {"ti8_quant_block", "ti8_quant_row", "ti8_quant_col_t", "ti8_fwht", "ti8_gemm_i8_nt",
            "ti8_gemm_i8_nt_i32", "ti8_version", "ti8_last_error", "ti8_arch"} <= set(names)
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in ti8.h but not exported by libti8.so"
    import triton_int8_amd
    assert sorted(triton_int8_amd._lib.EXPORTS) == names       # the binding covers the whole header


def test_version_and_arch(lib):
    assert lib.ti8_version() >= 100
    assert lib.ti8_arch() == b"gfx950"


def test_missing_library_fails_loudly(monkeypatch):
    import triton_int8_amd
    L = triton_int8_amd._lib
    monkeypatch.setattr(L, "_lib", None)
    monkeypatch.setattr(L, "LIB_PATH", "/nonexistent/libti8.so")
    with pytest.raises(ImportError, match="no fallback"):
        L.lib()


FAKE = 0x10000  # a 16-byte aligned non-null "device pointer"; validation never dereferences it


@pytest.mark.parametrize("call,code,msg", [
    (("ti8_quant_block", None, 0, 128, FAKE, 0, 128, None, 0, 0, FAKE, 0, 1, 1, 1, 128, 128, 128, 0, 0, None), 1, "required"),
    (("ti8_quant_block", FAKE, 0, 128, FAKE, 0, 128, None, 0, 0, FAKE, 0, 1, 1, 1, 100, 128, 128, 0, 0, None), 2, "R%128"),
    (("ti8_quant_block", FAKE, 0, 128, FAKE, 0, 128, None, 0, 0, FAKE, 0, 1, 1, 1, 128, 128, 64, 0, 0, None), 4, "group_c"),
    (("ti8_quant_block", FAKE, 0, 128, FAKE, 0, 128, FAKE, 0, 128, FAKE, 0, 1, 1, 1, 128, 256, 256, 0, 0, None), 4, "transposed"),
    (("ti8_quant_block", FAKE + 2, 0, 128, FAKE, 0, 128, None, 0, 0, FAKE, 0, 1, 1, 1, 128, 128, 128, 0, 0, None), 3, "aligned"),
    (("ti8_quant_block", FAKE, 0, 128, FAKE, 0, 128, None, 0, 0, FAKE, 0, 1, 1, 1, 128, 128, 128, 256, 0, None), 4, "flag"),
    (("ti8_quant_block", FAKE, 0, 256, FAKE, 0, 256, None, 0, 0, FAKE, 0, 1, 1, 1, 128, 256, 256, 64, 0, None), 4, "torch arithmetic"),
    (("ti8_quant_block", FAKE, 0, 128, FAKE, 0, 128, FAKE, 0, 128, FAKE, 0, 1, 1, 1, 128, 128, 128, 128, 0, None), 4, "torch arithmetic"),
    (("ti8_quant_row", FAKE, 4096, FAKE, 4096, FAKE, 4, 4096, 128, 64, 0, None), 4, "torch arithmetic"),
    (("ti8_quant_row", FAKE, 4096, FAKE, 4096, FAKE, 4, 4096, 0, 64, 1, None), 4, "torch arithmetic"),
    (("ti8_quant_col_t", FAKE, 256, FAKE, 128, FAKE, FAKE, 128, 256, 64, 0, None), 4, "unknown quantiser flag"),
    (("ti8_quant_block", FAKE, 0, 128, FAKE, 0, 128, None, 0, 0, FAKE, 0, 1, 1, 1, 128, 128, 128, 8, 0, None), 4, "had128"),
    (("ti8_quant_block_had128", FAKE, 0, 128, FAKE, 0, 128, FAKE, 0, 1, 1, 1, 128, 100, 0, 1, 0, None), 2, "C%128"),
    (("ti8_quant_block_had128", FAKE, 0, 128, None, 0, 128, FAKE, 0, 1, 1, 1, 128, 128, 1, 1, 0, None), 1, "required"),
    (("ti8_quant_row", FAKE, 4096, FAKE, 4096, FAKE, 4, 65536, 0, 0, 0, None), 2, "cols<=32768"),
    (("ti8_quant_row", FAKE, 4096, FAKE, 4096, FAKE, 4, 4096, 64, 0, 0, None), 4, "group"),
    (("ti8_quant_row", FAKE, 4096, FAKE, 4096, FAKE, 4, 4096, 0, 0, 7, None), 4, "inv_mode"),
    (("ti8_fwht_quant_row", FAKE, 4096, None, 4096, FAKE, 4, 4096, 4096, 1, 1, None), 1, "required"),
    (("ti8_fwht_quant_row", FAKE, 4096, FAKE, 4096, FAKE, 4, 4096, 3000, 1, 1, None), 2, "power of two"),
    (("ti8_fwht_quant_row", FAKE, 8192, FAKE, 8192, FAKE, 4, 8192, 4096, 1, 1, None), 2, "cols==n"),       # several transforms per row
    (("ti8_fwht_quant_row", FAKE, 2048, FAKE, 2048, FAKE, 4, 2048, 4096, 1, 1, None), 2, "cols==n"),       # cols = n / 2: not zero-extended
    (("ti8_fwht_quant_row", FAKE, 3000, FAKE, 3008, FAKE, 4, 3000, 4096, 1, 1, None), 2, "cols%16"),
    (("ti8_fwht_quant_row", FAKE, 4096, FAKE, 4096, FAKE, 0, 4096, 4096, 1, 1, None), 2, "rows>0"),
    (("ti8_fwht_quant_row", FAKE, 4096, FAKE, 4000, FAKE, 4, 4096, 4096, 1, 1, None), 2, "leading dimension"),
    (("ti8_fwht_quant_row", FAKE + 8, 4096, FAKE, 4096, FAKE, 4, 4096, 4096, 1, 1, None), 3, "aligned"),
    (("ti8_fwht_quant_row", FAKE, 4096, FAKE, 4096, FAKE, 4, 4096, 4096, 8, 1, None), 4, "apply here"),     # TI8_Q_HAD128
    (("ti8_fwht_quant_row", FAKE, 4096, FAKE, 4096, FAKE, 4, 4096, 4096, 4, 1, None), 4, "apply here"),     # TI8_Q_SCALE_BF16
    (("ti8_fwht_quant_row", FAKE, 4096, FAKE, 4096, FAKE, 4, 4096, 4096, 1, 9, None), 4, "inv_mode"),
    (("ti8_fwht_t_quant_row", FAKE, 256, None, FAKE, 4096, FAKE, 4096, 256, 1, 1, None), 1, "required"),
    (("ti8_fwht_t_quant_row", FAKE, 256, FAKE + 4096, FAKE, 4096, FAKE, 4096, 200, 1, 1, None), 2, "C % 64"),
    (("ti8_fwht_t_quant_row", FAKE, 256, FAKE + 4096, FAKE, 4096, FAKE, 65536, 256, 1, 1, None), 2, "R <= 32768"),
    (("ti8_fwht_t_quant_row", FAKE, 256, FAKE + 4096, FAKE, 2048, FAKE, 2048 + 64, 256, 1, 1, None), 2, "leading dimension of q"),
    (("ti8_fwht_t_quant_row", FAKE, 200, FAKE + 4096, FAKE, 4096, FAKE, 4096, 256, 1, 1, None), 2, "leading dimension"),
    (("ti8_fwht_t_quant_row", FAKE, 256, FAKE, FAKE, 4096, FAKE, 4096, 256, 1, 1, None), 4, "must not be the input"),
    (("ti8_fwht_t_quant_row", FAKE, 256, FAKE + 4096, FAKE, 4096, FAKE, 4096, 256, 8, 1, None), 4, "apply here"),
    (("ti8_quant_col_t", FAKE, 256, FAKE, 128, FAKE, None, 128, 256, 0, 0, None), 1, "required"),
    (("ti8_quant_col_t", FAKE, 256, FAKE, 128, FAKE, FAKE, 100, 256, 0, 0, None), 2, "R%128"),
    (("ti8_quant_row_col_t", FAKE, 256, FAKE, 256, FAKE, FAKE, 128, FAKE, None, 128, 256, 0, 0, None), 1, "required"),
    (("ti8_quant_row_col_t", FAKE, 256, FAKE, 256, FAKE, FAKE, 128, FAKE, FAKE, 128, 200, 0, 0, None), 2, "C%128"),
    (("ti8_quant_row_col_t", FAKE, 256, FAKE, 128, FAKE, FAKE, 128, FAKE, FAKE, 128, 256, 0, 0, None), 2, "leading dimension"),
    (("ti8_quant_row_col_t", FAKE, 256, FAKE, 256, FAKE, FAKE, 128, FAKE, FAKE, 128, 200, 16, 0, None), 2, "C%128"),
    (("ti8_quant_row_col_t", FAKE, 256, FAKE, 256, FAKE, FAKE, 128, FAKE, FAKE, 128, 256, 32, 0, None), 4, "TI8_Q_WS_PINGPONG"),
    (("ti8_quant_row_col_t", FAKE, 256, FAKE, 256, FAKE, FAKE, 128, FAKE, FAKE, 128, 256, 8, 0, None), 4, "Hadamard"),
    (("ti8_quant_row", FAKE, 4096, FAKE, 4096, FAKE, 4, 4096, 0, 16, 0, None), 4, "unknown quantiser flag"),
    (("ti8_quant_row_col_t_noalloc", FAKE, 65536, FAKE, 65536, FAKE, FAKE, 128, FAKE, 128, 65536, 0, 0, None), 2, "exceeds"),
    (("ti8_quant_row_col_t_noalloc", FAKE, 256, FAKE, 256, FAKE, FAKE, 128, FAKE, 128, 256, 16, 0, None), 4, "workspace flags"),
    (("ti8_fwht", FAKE, 384, FAKE, 384, 4, 384, 384, 1.0, None), 2, "power of two"),
    (("ti8_fwht", FAKE, 256, FAKE, 256, 4, 256, 64, 1.0, None), 2, "power of two"),
    (("ti8_fwht_t", FAKE, 256, FAKE + 0x100000, 384, 384, 256, 1.0, None), 2, "power of two"),
    (("ti8_fwht_t", FAKE, 260, FAKE + 0x100000, 256, 256, 260, 1.0, None), 2, "C % 8"),
    (("ti8_fwht_t", FAKE, 256, FAKE, 256, 256, 256, 1.0, None), 4, "in place"),
    (("ti8_fwht_t", FAKE, 256, FAKE + 0x100000, 128, 256, 256, 1.0, None), 2, "leading dimension"),
    (("ti8_gemm_i8_nt", FAKE, 0, 128, FAKE, 0, 128, FAKE, 0, 128, FAKE, 0, 0, 1, 0, FAKE, 0, 0, 1, 0,
      1, 128, 128, 100, 0, 0, 1.0, 0.0, 0, None), 2, "multiples of 128"),
    (("ti8_gemm_i8_nt", FAKE, 0, 128, FAKE, 0, 128, FAKE, 0, 128, None, 0, 0, 1, 0, FAKE, 0, 0, 1, 0,
      1, 128, 128, 128, 0, 0, 1.0, 0.0, 0, None), 1, "scale pointer"),
    (("ti8_gemm_i8_nt", FAKE, 0, 128, FAKE, 0, 128, FAKE, 0, 128, FAKE, 1, 0, 1, 1, FAKE, 0, 0, 1, 0,
      1, 128, 128, 128, 1, 0, 1.0, 0.0, 0, None), 4, "per-row scales"),
    (("ti8_gemm_i8_nt", FAKE, 0, 128, FAKE, 0, 128, FAKE, 0, 128, FAKE, 0, 0, 1, 0, FAKE, 0, 0, 1, 0,
      1, 128, 128, 128, 0, 9, 1.0, 0.0, 0, None), 4, "combine"),
    (("ti8_gemm_i8_nt_i32", FAKE, 0, 64, FAKE, 0, 128, FAKE, 0, 128, 1, 128, 128, 128, None), 2, "leading dimension"),
])
def test_argument_validation(lib, call, code, msg):
    import triton_int8_amd
    name, args = call[0], call[1:]
    rc = getattr(lib, name)(*args)
    assert rc == code, lib.ti8_last_error()
    assert msg in lib.ti8_last_error().decode()
    with pytest.raises(triton_int8_amd._lib.Ti8Error):
        triton_int8_amd._lib.call(name, *args)


def test_python_surface_rejects_bad_inputs_without_gpu():
    import torch
    import triton_int8_amd as T
    x = torch.zeros(1, 128, 128, dtype=torch.bfloat16)          # CPU tensor
    with pytest.raises(ValueError, match="GPU"):
        T.ops.quant_block(x)
    with pytest.raises(ValueError):
        T.linear.linear_forward(x[0], x[0], scheme="nope")
    with pytest.raises(AssertionError):
        T.block_channel_fwd32.triton_per_token_quant(torch.zeros(4, 100, dtype=torch.bfloat16))
    with pytest.raises(ValueError, match="bfloat16"):
        T.block_channel_fwd32.triton_gemm(None, None, None, None, out_dtype=torch.float16)


def test_latency_harness_shape_rules():
    """No GPU needed: the shape check comes before anything touches the device, and the bf16 product of
    two large 3-D operands is never one batched matmul call (that call faulted the GPU twice)."""
    import torch
    import triton_int8_amd as T
    lat = T.latency
    with pytest.raises(ValueError, match="beyond the largest shape"):
        lat.main(["--batch", "8", "--m", "8192", "--n", "8192", "--k", "8192"])
    with pytest.raises(ValueError, match="multiples of 128"):
        lat.check_shape(1, 100, 128, 128)
    lat.check_shape(4, 8192, 8192, 8192)
    meta = lambda *shape: torch.empty(*shape, dtype=torch.bfloat16, device="meta")
    assert lat.batched_matmul_allowed(meta(4, 8192, 8192), meta(8192, 8192))            # 3-D x 2-D: always one call
    assert lat.batched_matmul_allowed(meta(2, 256, 2048), meta(2, 512, 2048))
    assert not lat.batched_matmul_allowed(meta(2, 8192, 4096), meta(2, 4096, 4096))
    assert not lat.batched_matmul_allowed(meta(4, 8192, 8192), meta(4, 8192, 8192))
    a, b = torch.randn(3, 16, 8).to(torch.bfloat16), torch.randn(3, 4, 8).to(torch.bfloat16)
    assert torch.equal(T._common.bf16_reference_nt(a, b), torch.matmul(a, b.transpose(-2, -1)))


def test_gemm_kernel_id_text():
    """The text for a value of ti8_last_gemm_kernel (kind | epilogue << 8 | rows / 64 << 16 | columns / 64 << 20)."""
    import triton_int8_amd
    L = triton_int8_amd._lib
    t = L.describe_gemm_kernel(L.KERNEL_PERSISTENT_CHAIN | 5 << 8 | 4 << 16 | 4 << 20)
    assert "gemm_i8_chain_kernel" in t and "256x256" in t and "chained" in t
    t = L.describe_gemm_kernel(L.KERNEL_ONE_TILE_MULTI | 1 << 8 | 4 << 16 | 4 << 20)
    assert "gemm_i8_multi_kernel" in t and "256x256" in t and "int32 over the whole K" in t
    t = L.describe_gemm_kernel(L.KERNEL_ONE_TILE | 2 << 8 | 4 << 16 | 2 << 20)
    assert "gemm_i8_kernel" in t and "256x128" in t
    assert L.describe_gemm_kernel(L.KERNEL_FEW_ROWS) == "gemm_i8_wavering_kernel (few rows)"
    assert L.describe_gemm_kernel(0) == "none"


def test_linear_step_validation(lib):
    """ti8_linear_fwd_bwd rejects bad arguments before it launches anything (no GPU here: a launch would fail differently)."""
    T_, K, N = 256, 128, 384
    need = lib.ti8_linear_fwd_bwd_workspace(T_, K, N, 0)
    assert need > 0 and need % 256 == 0
    ws = 0x100000   # 256-byte aligned, never dereferenced
    good = dict(X=FAKE, ldx=K, W=FAKE, ldw=K, dY=FAKE, lddy=N, Y=FAKE, ldy=N, dX=FAKE, lddx=K, dW=FAKE, lddw=K, T=T_, tokens=T_, K=K, N=N,
                scheme=0, gemm_flags=0, workspace=ws, workspace_bytes=need, stream=None)
    cases = [(dict(scheme=1), 4, "scheme must be"), (dict(scheme=7), 4, "scheme must be"),
             (dict(X=None), 1, "required"), (dict(dW=None), 1, "required"),
             (dict(T=200, tokens=200), 2, "multiples of 128"), (dict(K=100, ldx=128, ldw=128, lddx=128, lddw=128), 2, "multiples of 128"),
             (dict(N=0), 2, "multiples of 128"),
             (dict(tokens=0), 2, "tokens must be"), (dict(tokens=T_ + 1), 2, "tokens must be"),
             (dict(ldx=K - 8), 2, "leading dimension"), (dict(ldy=N - 8), 2, "leading dimension"),
             (dict(X=FAKE + 8), 3, "16-byte aligned"), (dict(dW=FAKE + 4), 3, "16-byte aligned"), (dict(lddy=N + 4), 3, "16-byte aligned"),
             (dict(workspace=None), 2, "workspace"), (dict(workspace=ws + 16), 2, "workspace"), (dict(workspace_bytes=need - 1), 2, "workspace"),
             (dict(gemm_flags=1), 4, "apply here"), (dict(gemm_flags=4), 4, "apply here")]     # TI8_GEMM_STRICT, TI8_GEMM_SKINNY
    for change, code, msg in cases:
        a = {**good, **change}
        rc = lib.ti8_linear_fwd_bwd(*a.values())
        assert rc == code and msg in lib.ti8_last_error().decode(), (change, rc, lib.ti8_last_error())
    for scheme in (0, 2):
        assert lib.ti8_linear_fwd_bwd_workspace(T_, K, N, scheme) > 0
    for bad in ((T_ + 1, K, N, 0), (T_, 0, N, 0), (T_, K, N, 1), (T_, K, N, -1)):
        assert lib.ti8_linear_fwd_bwd_workspace(*bad) == -1


def test_quant_block_multi_validation(lib):
    """ti8_quant_block_multi takes a host array of operand descriptors; bad ones are rejected before any launch."""
    import triton_int8_amd
    L = triton_int8_amd._lib
    good = dict(x=FAKE, bsx=0, ldx=128, q=FAKE, bsq=0, ldq=128, qT=None, bsqt=0, ldqt=0, s=FAKE, ssb=0, ssr=1, ssc=1, B=1, R=128, C=128)
    arr = lambda *ds: (L.QBlockOperand * len(ds))(*[L.QBlockOperand(**d) for d in ds])
    cases = [((None, 1), 1, "operands is required"),
             ((arr(good), 0), 2, "between 1 and 4"),
             ((arr(good, good, good, good, good), 5), 2, "between 1 and 4"),
             ((arr({**good, "R": 100}), 1), 2, "R%128"),
             ((arr({**good, "x": None}), 1), 1, "required"),
             ((arr(good, {**good, "qT": FAKE, "ldqt": 128}), 2), 4, "same outputs"),
             ((arr({**good, "q": FAKE + 4}), 1), 3, "aligned")]
    for (ops_, n), code, msg in cases:
        rc = lib.ti8_quant_block_multi(ops_, n, 1, 0, None)
        assert rc == code and msg in lib.ti8_last_error().decode(), (lib.ti8_last_error(), msg)
    assert lib.ti8_quant_block_multi(arr(good), 1, 8, 0, None) == 4      # TI8_Q_HAD128


def test_gemm_multi_validation(lib):
    """ti8_gemm_i8_nt_multi takes a host array of GEMM descriptors; a bad one is rejected before any launch, with
    the checks of ti8_gemm_i8_nt."""
    import triton_int8_amd
    L = triton_int8_amd._lib
    good = dict(A=FAKE, bsa=0, lda=128, B=FAKE, bsb=0, ldb=128, C=FAKE, bsc=0, ldc=512, sA=FAKE, modeA=1, sa_bs=0, sa_rs=1, sa_ks=1,
                sB=FAKE, modeB=0, sb_bs=0, sb_rs=1, sb_ks=0, batch=1, M=512, N=512, K=128, acc_i32_full=0, combine=0,
                out_scale=1.0, post_scale=0.0)
    arr = lambda *ds: (L.GemmProblem * len(ds))(*[L.GemmProblem(**d) for d in ds])
    cases = [((None, 1, 0), 1, "problems is required"),
             ((arr(good), 0, 0), 2, "between 1 and 3"),
             ((arr(good, good, good, good), 4, 0), 2, "between 1 and 3"),
             ((arr(good), 1, 4), 4, "few-rows kernel"),                      # TI8_GEMM_SKINNY
             ((arr(good), 1, 256), 4, "unknown flag"),
             ((arr(good, {**good, "batch": 2}), 2, 0), 2, "batch = 1, GEMM 1"),
             ((arr({**good, "M": 64}), 1, 0), 2, "multiple of 128"),
             ((arr({**good, "K": 100}), 1, 0), 2, "multiples of 128"),
             ((arr(good, {**good, "sB": None}), 2, 0), 1, "scale pointer of B"),
             ((arr({**good, "acc_i32_full": 1}), 1, 0), 4, "per-row scales on both"),
             ((arr({**good, "A": FAKE + 4}), 1, 0), 3, "aligned"),
             ((arr({**good, "ldc": 64}), 1, 0), 2, "leading dimension")]
    for (p, n, flags), code, msg in cases:
        rc = lib.ti8_gemm_i8_nt_multi(p, n, flags, None)
        assert rc == code and msg in lib.ti8_last_error().decode(), (rc, lib.ti8_last_error(), msg)


def test_empty_batch_needs_no_kernel():
    """Zero tokens: empty Y and dX, a zero weight gradient, as torch.nn.functional.linear gives; no launch, so it runs here."""
    import torch
    import triton_int8_amd as T
    W = torch.randn(256, 128).to(torch.bfloat16)
    for lead in ((0,), (3, 0), (0, 5)):
        X, dY = torch.empty(*lead, 128, dtype=torch.bfloat16), torch.empty(*lead, 256, dtype=torch.bfloat16)
        for scheme in T.linear.SCHEMES:
            Y, dX, dW = T.linear_fwd_bwd(X, W, dY, scheme)
            assert Y.shape == (*lead, 256) and dX.shape == (*lead, 128) and dW.shape == W.shape and not dW.any()
    lin = T.Int8Linear(128, 256, bias=True, device="cpu")
    x = torch.empty(2, 0, 128, dtype=torch.bfloat16, requires_grad=True)
    y = lin(x)
    assert y.shape == (2, 0, 256)
    y.sum().backward()
    assert x.grad.shape == x.shape and not lin.weight.grad.any() and not lin.bias.grad.any()
    with torch.no_grad():
        assert lin(x.detach()).shape == (2, 0, 256)
