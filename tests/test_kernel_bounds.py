"""Host-side bounds model of the kernels (no GPU).

The kernels take every global-memory offset from triton-int8_amd/csrc/index_math.h, which also
compiles with g++.  tests/kernel_bounds/walk.cpp walks (workgroup, wave, lane, iteration) of the
launch an entry point would make and checks every access against the allocation it goes to.  Here
the Python pipelines (fwd_32 / bwd_33 of every scheme) run on host tensors with the C-ABI calls
RECORDED instead of executed, so the geometry, strides and allocation sizes are the ones the
wrappers of ops.py produce; each recorded call is then walked.

Shapes: the reference's own acceptance / latency shape B = 4, M = N = K = 8192
(triton/block_channel_fwd32.py:257-272, test.py:32-45) and smaller ragged ones."""
import ctypes
import os
import subprocess

import pytest
import torch

from conftest import ROOT

CSRC = os.path.join(ROOT, "triton-int8_amd", "csrc")
SRC = os.path.join(ROOT, "tests", "kernel_bounds", "walk.cpp")
LDS_LIMIT = 160 * 1024     # bytes of LDS per workgroup on gfx950
NUM_CU = 256


class ScaleArg(ctypes.Structure):
    _fields_ = [("mode", ctypes.c_int), ("bs", ctypes.c_int64), ("rs", ctypes.c_int64), ("ks", ctypes.c_int64),
                ("elems", ctypes.c_int64)]


@pytest.fixture(scope="module")
def walker(tmp_path_factory):
    so = str(tmp_path_factory.mktemp("bounds") / "libwalk.so")
    subprocess.run(["g++", "-O2", "-std=c++17", "-shared", "-fPIC", "-I", CSRC, "-o", so, SRC], check=True)
    lib = ctypes.CDLL(so)
    i64, ci, cp = ctypes.c_int64, ctypes.c_int, ctypes.c_char_p
    p64 = ctypes.POINTER(ctypes.c_int64)
    lib.walk_fwht.argtypes = [i64] * 8 + [p64, cp, ci]
    lib.walk_fwht_quant_row.argtypes = [i64] * 9 + [p64, cp, ci]
    lib.walk_transpose_bf16.argtypes = [i64] * 6 + [p64, cp, ci]
    lib.walk_fwht_t.argtypes = [i64] * 7 + [p64, cp, ci]
    lib.walk_quant_row.argtypes = [i64] * 4 + [ci] + [i64] * 3 + [p64, cp, ci]
    lib.walk_quant_block.argtypes = [i64, i64, ci, i64, i64, ci, i64, i64, i64, i64, i64, i64, i64, i64, ci, i64, i64, i64, i64, p64, cp, ci]
    lib.walk_gemm.argtypes = [i64] * 6 + [ctypes.POINTER(ScaleArg)] * 2 + [i64] * 4 + [ci] * 5 + [i64] * 3 + [ctypes.POINTER(ci), p64, cp, ci]
    lib.walk_gemm_chain.argtypes = [i64] * 6 + [ctypes.POINTER(ScaleArg)] * 2 + [i64] * 4 + [ci] + [i64] * 3 + [p64, cp, ci]
    lib.walk_gemm_multi_map.argtypes = [ctypes.POINTER(ci), ci, p64, cp, ci]
    return lib


class Allocations:
    """Host stand-ins for device allocations: start address -> bytes."""

    def __init__(self):
        self.blocks = []
        self.keep = []

    def add(self, t):
        self.blocks.append((t.data_ptr(), t.numel() * t.element_size()))
        self.keep.append(t)
        return t

    def room(self, ptr, elem_size):
        """Elements of `elem_size` bytes between `ptr` and the end of the allocation that holds it."""
        if ptr is None:
            return 0
        for start, nbytes in self.blocks:
            if start <= ptr < start + nbytes:
                return (start + nbytes - ptr) // elem_size
        raise AssertionError(f"pointer {ptr:#x} belongs to no recorded allocation")


@pytest.fixture
def recorded(monkeypatch):
    """Run the Python surface on host tensors with every C-ABI call recorded instead of executed."""
    import triton_int8_amd as T
    allocs, calls = Allocations(), []
    real_empty = torch.empty
    monkeypatch.setattr(torch, "empty", lambda *a, **k: allocs.add(real_empty(*a, **k)))
    monkeypatch.setattr(torch, "zeros", lambda *a, **k: allocs.add(real_empty(*a, **k)))   # untouched pages: no memory used
    monkeypatch.setattr(T.ops, "_on_gpu", lambda t: True)
    monkeypatch.setattr(T.ops, "_stream", lambda: None)
    monkeypatch.setattr(torch.cuda, "set_device", lambda d: None)
    monkeypatch.setattr(torch.cuda, "is_current_stream_capturing", lambda: False)
    monkeypatch.setattr(torch.Tensor, "cuda", lambda self, *a, **k: self)
    monkeypatch.setattr(T._lib, "call", lambda name, *args: calls.append((name, args)))
    yield T, allocs, calls


def walk(lib, allocs, name, a):
    """Walk one recorded call; returns the number of accesses checked."""
    msg = ctypes.create_string_buffer(512)
    n = ctypes.c_int64(0)
    if name == "ti8_fwht":
        x, ldx, y, ldy, rows, cols, nn = a[:7]
        rc = lib.walk_fwht(ldx, ldy, rows, cols, nn, allocs.room(x, 2), allocs.room(y, 2), LDS_LIMIT, ctypes.byref(n), msg, 512)
    elif name == "ti8_fwht_quant_row":
        x, ldx, q, ldq, sc, rows, cols, nn = a[:8]
        rc = lib.walk_fwht_quant_row(ldx, ldq, rows, cols, nn, allocs.room(x, 2), allocs.room(q, 1), allocs.room(sc, 4), LDS_LIMIT,
                                     ctypes.byref(n), msg, 512)
    elif name == "ti8_fwht_t_quant_row":
        # the transposition into the scratch buffer (the long-column path of ti8_fwht_t), then ti8_fwht_quant_row on it
        x, ldx, scratch, q, ldq, sc, R, C = a[:8]
        nn = 1 << (R - 1).bit_length()
        rc = lib.walk_transpose_bf16(ldx, R, R, C, allocs.room(x, 2), allocs.room(scratch, 2), ctypes.byref(n), msg, 512)
        assert rc == 0, f"{name} (transposition): {msg.value.decode()}"
        first = n.value
        rc = lib.walk_fwht_quant_row(R, ldq, C, R, nn, allocs.room(scratch, 2), allocs.room(q, 1), allocs.room(sc, 4), LDS_LIMIT,
                                     ctypes.byref(n), msg, 512)
        n.value += first
    elif name == "ti8_fwht_t":
        x, ldx, y, ldy, R, C = a[:6]
        rc = lib.walk_fwht_t(ldx, ldy, R, C, allocs.room(x, 2), allocs.room(y, 2), LDS_LIMIT, ctypes.byref(n), msg, 512)
    elif name == "ti8_quant_row":
        x, ldx, q, ldq, s, rows, cols, group = a[:8]
        rc = lib.walk_quant_row(ldx, ldq, rows, cols, group, allocs.room(x, 2), allocs.room(q, 1), allocs.room(s, 4), ctypes.byref(n), msg, 512)
    elif name == "ti8_quant_block":
        x, bsx, ldx, q, bsq, ldq, qT, bsqt, ldqt, s, ssb, ssr, ssc, B, R, C, group_c = a[:17]
        rc = lib.walk_quant_block(bsx, ldx, q is not None, bsq, ldq, qT is not None, bsqt, ldqt, ssb, ssr, ssc, B, R, C, group_c,
                                  allocs.room(x, 2), allocs.room(q, 1), allocs.room(qT, 1), allocs.room(s, 4), ctypes.byref(n), msg, 512)
    elif name in ("ti8_gemm_i8_nt", "ti8_gemm_i8_nt_i32"):
        picked = (ctypes.c_int * 3)()
        if name == "ti8_gemm_i8_nt":
            (A, bsa, lda, B, bsb, ldb, C, bsc, ldc, sA, mA, sa_bs, sa_rs, sa_ks, sB, mB, sb_bs, sb_rs, sb_ks,
             batch, M, N, K, acc, combine, out_scale, post_scale, flags) = a[:28]
            sa = ScaleArg(mA, sa_bs, sa_rs, sa_ks, allocs.room(sA, 4))
            sb = ScaleArg(mB, sb_bs, sb_rs, sb_ks, allocs.room(sB, 4))
            rc = lib.walk_gemm(bsa, lda, bsb, ldb, bsc, ldc, ctypes.byref(sa), ctypes.byref(sb), batch, M, N, K, acc, flags & 1, (flags >> 3) & 1, 0,
                               NUM_CU, allocs.room(A, 1), allocs.room(B, 1), allocs.room(C, 2), picked, ctypes.byref(n), msg, 512)
            if rc == 0 and picked[2] == 5 and 2 <= K // 128 <= 256 and K % 256 == 0:   # the chained promotion runs on persistent workgroups
                first = n.value
                tiles = -(-M // 256) * -(-N // 256) * batch
                rc = lib.walk_gemm_chain(bsa, lda, bsb, ldb, bsc, ldc, ctypes.byref(sa), ctypes.byref(sb), batch, M, N, K, min(tiles, NUM_CU),
                                         allocs.room(A, 1), allocs.room(B, 1), allocs.room(C, 2), ctypes.byref(n), msg, 512)
                n.value += first
        else:
            A, bsa, lda, B, bsb, ldb, C, bsc, ldc, batch, M, N, K = a[:13]
            rc = lib.walk_gemm(bsa, lda, bsb, ldb, bsc, ldc, None, None, batch, M, N, K, 0, 0, 0, 1,
                               NUM_CU, allocs.room(A, 1), allocs.room(B, 1), allocs.room(C, 4), picked, ctypes.byref(n), msg, 512)
    elif name == "ti8_gemm_i8_nt_multi":
        # every GEMM of the launch as the tiled kernel walks it alone, then the workgroup -> (GEMM, tile) map
        problems, count, flags = a[:3]
        total, tiles = 0, (ctypes.c_int * count)()
        for i in range(count):
            p = problems[i]
            picked = (ctypes.c_int * 3)()
            sa = ScaleArg(p.modeA, p.sa_bs, p.sa_rs, p.sa_ks, allocs.room(p.sA, 4))
            sb = ScaleArg(p.modeB, p.sb_bs, p.sb_rs, p.sb_ks, allocs.room(p.sB, 4))
            rc = lib.walk_gemm(p.bsa, p.lda, p.bsb, p.ldb, p.bsc, p.ldc, ctypes.byref(sa), ctypes.byref(sb), 1, p.M, p.N, p.K, p.acc_i32_full,
                               flags & 1, (flags >> 3) & 1, 0, NUM_CU, allocs.room(p.A, 1), allocs.room(p.B, 1), allocs.room(p.C, 2),
                               picked, ctypes.byref(n), msg, 512)
            assert rc == 0, f"{name}, GEMM {i}: {msg.value.decode()}"
            total += n.value
            tiles[i] = -(-p.M // picked[0]) * -(-p.N // picked[1])
            if picked[2] == 5 and 2 <= p.K // 128 <= 256 and p.K % 256 == 0:   # persistent workgroups: each GEMM's tiles as one workgroup list walks them
                rc = lib.walk_gemm_chain(p.bsa, p.lda, p.bsb, p.ldb, p.bsc, p.ldc, ctypes.byref(sa), ctypes.byref(sb), 1, p.M, p.N, p.K,
                                         min(tiles[i], NUM_CU), allocs.room(p.A, 1), allocs.room(p.B, 1), allocs.room(p.C, 2), ctypes.byref(n), msg, 512)
                assert rc == 0, f"{name}, GEMM {i} (persistent): {msg.value.decode()}"
                total += n.value
        rc = lib.walk_gemm_multi_map(tiles, count, ctypes.byref(n), msg, 512)
        n.value += total
    else:
        raise AssertionError(f"no walker for {name}")
    assert rc == 0, f"{name}: {msg.value.decode()}"
    assert n.value > 0
    return n.value


PIPELINES = [("double_channel_fwd32", "fwd_32", False), ("double_channel_bwd33", "bwd_33", True),
             ("block_channel_fwd32", "fwd_32", False), ("block_channel_bwd33", "bwd_33", True),
             ("fused_fwd32", "fwd_32", False), ("fused_bwd33", "bwd_33", True),
             ("tilelang_block_channel_fwd", "fwd_32", False), ("tilelang_block_channel_bwd", "bwd_33", True)]


@pytest.mark.parametrize("module,fn,three_d", PIPELINES)
@pytest.mark.parametrize("B,M,N,K", [(4, 8192, 8192, 8192), (2, 384, 640, 2048)])
def test_every_access_of_a_pipeline_is_in_bounds(walker, recorded, module, fn, three_d, B, M, N, K):
    """Every kernel launch of fwd_32 / bwd_33: all global accesses inside their allocations, every
    tile computed once, every element of C stored once.  B = 4, M = N = K = 8192 is the shape of
    the reference's self-checks and of its latency script."""
    T, allocs, calls = recorded
    a = torch.empty(B, M, K, dtype=torch.bfloat16)
    b = torch.empty(B, N, K, dtype=torch.bfloat16) if three_d else torch.empty(N, K, dtype=torch.bfloat16)
    out = getattr(getattr(T, module), fn)(a, b)
    assert tuple(out.shape) == (B, M, N)
    names = [c[0] for c in calls]
    assert "ti8_gemm_i8_nt" in names and len(names) >= 3
    total = sum(walk(walker, allocs, name, args) for name, args in calls)
    assert total > 1000


def test_walker_sees_an_access_past_the_end(walker):
    """The model is not vacuous: the same launches against buffers one row too short fail."""
    msg = ctypes.create_string_buffer(512)
    n = ctypes.c_int64(0)
    rows, cols = 512, 8192
    assert walker.walk_fwht(cols, cols, rows, cols, cols, rows * cols, rows * cols, LDS_LIMIT, ctypes.byref(n), msg, 512) == 0
    assert walker.walk_fwht(cols, cols, rows, cols, cols, rows * cols - 8, rows * cols, LDS_LIMIT, ctypes.byref(n), msg, 512) == 1
    assert b"fwht x" in msg.value
    # LDS: a 2048-element segment needs 8.5 KiB (lengths from 4096 on use a fixed 34 KiB exchange buffer instead)
    assert walker.walk_fwht(2048, 2048, rows, 2048, 2048, rows * 2048, rows * 2048, 4 * 1024, ctypes.byref(n), msg, 512) == 1
    assert walker.walk_quant_row(cols, cols, rows, cols, 0, rows * cols, rows * cols, rows, ctypes.byref(n), msg, 512) == 0
    assert walker.walk_quant_row(cols, cols, rows, cols, 0, rows * cols, rows * cols, rows - 1, ctypes.byref(n), msg, 512) == 1
    assert b"quant_row s" in msg.value
    M = N = K = 512
    sa, sb = ScaleArg(0, M, 1, 0, M), ScaleArg(0, 0, 1, 0, N)
    picked = (ctypes.c_int * 3)()
    ok = lambda a_el, c_el, large: walker.walk_gemm(M * K, K, 0, K, M * N, N, ctypes.byref(sa), ctypes.byref(sb), 1, M, N, K, 1, 0, large, 0, NUM_CU,
                                                    a_el, N * K, c_el, picked, ctypes.byref(n), msg, 512)
    assert ok(M * K, M * N, 0) == 0 and tuple(picked) == (128, 128, 1)
    assert ok(M * K, M * N, 1) == 0 and tuple(picked) == (256, 256, 1)
    assert ok(M * K - 16, M * N, 1) == 1 and b"gemm A" in msg.value
    assert ok(M * K, M * N - 4, 0) == 1 and b"gemm C" in msg.value


@pytest.mark.parametrize("M,N,K,batch,mA,mB,acc,flags", [
    (8192, 4096, 4096, 1, 1, 0, 0, 0),      # config 2 Y / dX: chained promotion kernel on 256 x 256 tiles
    (4096, 4096, 8192, 1, 1, 1, 0, 0),      # config 2 dW: block x block
    (16384, 14336, 4096, 1, 0, 0, 1, 0),    # config 3 gate/up: int32 kernel
    (14336, 4096, 16384, 1, 1, 1, 0, 0),    # config 5 down_proj dW: K = 16384
    (1536, 1024, 1024, 1, 1, 0, 0, 8),      # incomplete group of tile rows + XCD remap, 256 x 256 tiles
    (4608, 2048, 512, 1, 0, 1, 0, 0),       # 256 x 128 tiles
    (640, 384, 640, 3, 1, 1, 0, 0),         # 128 x 128 tiles, tiles that hang over M and N
    (640, 384, 640, 3, 1, 1, 0, 8),         # the same on 256 x 256 tiles: the re-read of the valid half
    (384, 256, 33024, 2, 1, 0, 0, 0),       # K > 32768: literal kernel
    (256, 384, 1024, 2, 1, 2, 0, 2),        # per-(column, K tile) scales of B
])
def test_gemm_launch_geometries(walker, M, N, K, batch, mA, mB, acc, flags):
    """The GEMM kernels at the benchmark shapes and at shapes whose tiles hang over the edges."""
    nkb = K // 128
    def desc(mode, rows, batched):
        per_batch = {0: rows, 1: -(-rows // 128) * nkb, 2: rows * nkb, 3: -(-rows // 128) * (nkb // 2)}[mode]
        rs = {0: 1, 1: nkb, 2: nkb, 3: nkb // 2}[mode]
        return ScaleArg(mode, per_batch if batched else 0, rs, 0 if mode == 0 else 1, per_batch * (batch if batched else 1))
    sa, sb = desc(mA, M, True), desc(mB, N, False)
    msg = ctypes.create_string_buffer(512)
    n = ctypes.c_int64(0)
    picked = (ctypes.c_int * 3)()
    rc = walker.walk_gemm(M * K, K, 0, K, M * N, N, ctypes.byref(sa), ctypes.byref(sb), batch, M, N, K, acc, flags & 1, (flags >> 3) & 1, 0,
                          NUM_CU, batch * M * K, N * K, batch * M * N, picked, ctypes.byref(n), msg, 512)
    assert rc == 0, msg.value.decode()


@pytest.mark.parametrize("R,C", [(128, 8), (128, 520), (2048, 72), (4096, 512), (8192, 1024), (16384, 2048), (32768, 4096), (32768, 64),
                                 (16384, 96)])
def test_transposed_hadamard_launches(walker, recorded, R, C):
    """ti8_fwht_t as ops.fwht_t launches it: every read of x, every LDS index and every write of y in
    bounds, and the XCD-aware column-block map a bijection (with and without the sibling grouping)."""
    T, allocs, calls = recorded
    y = T.ops.fwht_t(torch.empty(R, C, dtype=torch.bfloat16))
    assert tuple(y.shape) == (C, R) and [c[0] for c in calls] == ["ti8_fwht_t"]
    assert walk(walker, allocs, *calls[0]) > R * C // 8
    msg = ctypes.create_string_buffer(512)
    n = ctypes.c_int64(0)
    assert walker.walk_fwht_t(C, R, R, C, R * C - 1, R * C, LDS_LIMIT, ctypes.byref(n), msg, 512) == 1 and msg.value.split(b":")[0].endswith(b" x")
    assert walker.walk_fwht_t(C, R, R, C, R * C, R * C - 8, LDS_LIMIT, ctypes.byref(n), msg, 512) == 1 and msg.value.split(b":")[0].endswith(b" y")


@pytest.mark.parametrize("R,C", [(128, 64), (4096, 192), (8192, 128), (14336, 64), (32768, 64)])
def test_rotate_and_quantise_of_the_transpose(walker, recorded, R, C):
    """ti8_fwht_t_quant_row as the wrapper launches it (scratch tensor included): the transposition and the fused kernel
    behind it stay inside their buffers."""
    T, allocs, calls = recorded
    q, s = T.ops.fwht_t_quant_row(torch.empty(R, C, dtype=torch.bfloat16))
    assert tuple(q.shape) == (C, R) and tuple(s.shape) == (C,) and [c[0] for c in calls] == ["ti8_fwht_t_quant_row"]
    assert walk(walker, allocs, *calls[0]) >= R * C // 4


@pytest.mark.parametrize("rows,cols", [(5, 128), (3, 2048), (2, 8192), (2, 14336), (1, 16384), (1, 32768), (2, 28672)])
def test_rotate_and_quantise_launch(walker, recorded, rows, cols):
    """ti8_fwht_quant_row as the wrapper launches it: every global and LDS access in bounds, every chunk of a row kept by
    one thread; and the walker notices an allocation that is too small."""
    T, allocs, calls = recorded
    q, s = T.ops.fwht_quant_row(torch.empty(rows, cols, dtype=torch.bfloat16))
    assert tuple(q.shape) == (rows, cols) and tuple(s.shape) == (rows,) and [c[0] for c in calls] == ["ti8_fwht_quant_row"]
    nn = 1 << (cols - 1).bit_length()
    assert calls[0][1][7] == nn
    assert walk(walker, allocs, *calls[0]) >= rows * cols // 8
    msg, n = ctypes.create_string_buffer(512), ctypes.c_int64(0)
    args = lambda x_el, q_el, s_el: (cols, cols, rows, cols, nn, x_el, q_el, s_el, LDS_LIMIT, ctypes.byref(n), msg, 512)
    assert walker.walk_fwht_quant_row(*args(rows * cols, rows * cols, rows)) == 0
    assert walker.walk_fwht_quant_row(*args(rows * cols - 8, rows * cols, rows)) == 1 and b"fwht x" in msg.value
    assert walker.walk_fwht_quant_row(*args(rows * cols, rows * cols - 8, rows)) == 1 and b"fwht q" in msg.value
    assert walker.walk_fwht_quant_row(*args(rows * cols, rows * cols, rows - 1)) == 1 and b"fwht s" in msg.value


@pytest.mark.parametrize("rows,cols", [(3, 96), (5, 1792), (4, 14336), (2, 24576)])
def test_zero_extended_hadamard_launch(walker, recorded, rows, cols):
    """ti8_fwht on a length that is no power of two: one zero-extended row per workgroup, nothing read or stored beyond
    the row's own elements."""
    T, allocs, calls = recorded
    y = T.ops.fwht(torch.empty(rows, cols, dtype=torch.bfloat16))
    assert tuple(y.shape) == (rows, cols) and [c[0] for c in calls] == ["ti8_fwht"]
    assert calls[0][1][6] == 1 << (cols - 1).bit_length()
    assert walk(walker, allocs, *calls[0]) >= rows * cols // 8
    msg, n = ctypes.create_string_buffer(512), ctypes.c_int64(0)
    nn = 1 << (cols - 1).bit_length()
    assert walker.walk_fwht(cols, cols, rows, cols, nn, rows * cols - 8, rows * cols, LDS_LIMIT, ctypes.byref(n), msg, 512) == 1 and b"fwht x" in msg.value
    assert walker.walk_fwht(cols, cols, rows, cols, nn, rows * cols, rows * cols - 8, LDS_LIMIT, ctypes.byref(n), msg, 512) == 1 and b"fwht y" in msg.value


@pytest.mark.parametrize("M,K,N", [(1024, 512, 768), (8192, 4096, 4096)])
def test_one_launch_step_is_in_bounds(walker, recorded, monkeypatch, M, K, N):
    """The three GEMMs of a block-channel step in one launch: each GEMM's accesses stay inside its operands, and the
    launch's workgroups cover every tile of every GEMM exactly once."""
    T, allocs, calls = recorded
    monkeypatch.setattr(T.linear, "ONE_CALL_STEP", False)    # the step assembled from the separate entry points
    X, W, dY = (allocs.add(torch.empty(s, dtype=torch.bfloat16)) for s in ((M, K), (N, K), (M, N)))
    T.linear_fwd_bwd(X, W, dY, "block_channel")
    names = [c[0] for c in calls]
    assert names.count("ti8_gemm_i8_nt_multi") == 1 and "ti8_gemm_i8_nt" not in names
    name, a = next(c for c in calls if c[0] == "ti8_gemm_i8_nt_multi")
    assert a[1] == 3 and walk(walker, allocs, name, a) > 3


@pytest.mark.parametrize("scheme", ["block_channel", "double_channel"])
@pytest.mark.parametrize("M,K,N", [(1024, 512, 768), (8192, 4096, 4096), (16384, 4096, 14336)])
def test_one_call_step_workspace(recorded, scheme, M, K, N):
    """The whole step as one library call: the wrapper hands over the three operands, three outputs and a workspace
    of the size the library asks for, and that size holds every piece the step carves out of it (int8 copies and
    transposes of the three operands, their scales, the maxima), each on a 256-byte boundary."""
    T, allocs, calls = recorded
    X, W, dY = (allocs.add(torch.empty(s, dtype=torch.bfloat16)) for s in ((M, K), (N, K), (M, N)))
    Y, dX, dW = T.linear_fwd_bwd(X, W, dY, scheme)
    assert [c[0] for c in calls] == ["ti8_linear_fwd_bwd"]
    a = calls[0][1]
    assert (a[12], a[13], a[14], a[15]) == (M, M, K, N) and (a[1], a[3], a[5], a[7], a[9], a[11]) == (K, K, N, N, K, K)
    for ptr, elems in ((a[0], M * K), (a[2], N * K), (a[4], M * N), (a[6], M * N), (a[8], M * K), (a[10], N * K)):
        assert allocs.room(ptr, 2) >= elems
    ws_ptr, ws_bytes = a[18], a[19]
    assert ws_ptr % 256 == 0 and allocs.room(ws_ptr, 1) >= ws_bytes == T.ops.linear_step_workspace_bytes(M, K, N, scheme)
    int8_bytes = 2 * (M * K + M * N + N * K)                     # q and qT of every operand
    if scheme == "block_channel":
        floats = (M // 128) * (K // 128) + (M // 128) * (N // 128) + 2 * (N + K)
        pieces = 11
    else:
        floats = 2 * ((M + K) + (N + K) + (M + N))
        pieces = 13
    assert int8_bytes + 4 * floats <= ws_bytes <= int8_bytes + 4 * floats + 256 * pieces
    assert T._lib.lib().ti8_linear_fwd_bwd_workspace(M + 1, K, N, 0) == -1 and T._lib.lib().ti8_linear_fwd_bwd_workspace(M, K, N, 1) == -1


@pytest.mark.parametrize("tiles", [[512, 512, 512], [1, 1, 1], [7, 300, 2], [5], [9, 4]])
def test_multi_launch_map(walker, tiles):
    msg, n = ctypes.create_string_buffer(512), ctypes.c_int64(0)
    arr = (ctypes.c_int * len(tiles))(*tiles)
    assert walker.walk_gemm_multi_map(arr, len(tiles), ctypes.byref(n), msg, 512) == 0, msg.value.decode()
    assert n.value == sum(tiles)


@pytest.mark.parametrize("M,N,K,batch,mA,mB,grid", [(8192, 4096, 4096, 1, 1, 0, 256), (4096, 4096, 8192, 1, 1, 1, 256), (4224, 4480, 256, 1, 1, 0, 256),
                                                    (2048, 2304, 1024, 3, 0, 1, 256), (1152, 1408, 512, 2, 3, 0, 7), (8192, 8192, 512, 1, 0, 0, 256), (4096, 4096, 16384, 1, 1, 1, 256), (1280, 768, 32768, 1, 1, 0, 15)])
def test_persistent_chain_kernel_geometries(walker, M, N, K, batch, mA, mB, grid):
    """gemm_i8_chain_kernel: tile lists of persistent workgroups, tiles that hang over M or N, batches, every scale layout."""
    def desc(mode, rows):
        if mode == 0:
            return ScaleArg(0, rows, 1, 0, batch * rows)
        g = (rows // 128, K // 128 // (2 if mode == 3 else 1))
        return ScaleArg(mode, g[0] * g[1], g[1], 1, batch * g[0] * g[1])
    sa, sb = desc(mA, M), desc(mB, N)
    msg, n = ctypes.create_string_buffer(512), ctypes.c_int64(0)
    rc = walker.walk_gemm_chain(M * K, K, N * K, K, M * N, N, ctypes.byref(sa), ctypes.byref(sb), batch, M, N, K, grid,
                                batch * M * K, batch * N * K, batch * M * N, ctypes.byref(n), msg, 512)
    assert rc == 0, msg.value.decode()
    assert n.value > 0
    # one row less of A than the kernel assumes must be noticed
    rc = walker.walk_gemm_chain(M * K, K, N * K, K, M * N, N, ctypes.byref(sa), ctypes.byref(sb), batch, M, N, K, grid,
                                batch * M * K - K, batch * N * K, batch * M * N, ctypes.byref(n), msg, 512)
    assert rc != 0 and b"gemm chain A" in msg.value
