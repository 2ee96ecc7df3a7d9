"""The entry point that allocates nothing (ti8_quant_row_col_t_noalloc) against the entry point it
is a variant of (ti8_quant_row_col_t with a caller-provided workspace): same bits, called through
the C ABI, on two calls in a row that share the library's fixed scratch array, the second with a
smaller input (so it meets the first call's leftovers in the array)."""
import pytest
import torch

from conftest import make_gen, randn_bf16

pytestmark = pytest.mark.gpu


def _call(T, name, x, ws=None):
    R, C = x.shape
    dev = x.device
    q = torch.empty((R, C), dtype=torch.int8, device=dev)
    qT = torch.empty((C, R), dtype=torch.int8, device=dev)
    s_row = torch.empty(R, dtype=torch.float32, device=dev)
    s_col = torch.empty(C, dtype=torch.float32, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    head = (x.data_ptr(), x.stride(0), q.data_ptr(), C, s_row.data_ptr(), qT.data_ptr(), R, s_col.data_ptr())
    tail = (R, C, T._lib.Q_CLAMP, 0, stream)
    if ws is None:
        T._lib.call(name, *head, *tail)
    else:
        T._lib.call(name, *head, ws.data_ptr(), *tail)
    return q, s_row, qT, s_col


def test_no_alloc_entry_point_matches_workspace_entry_point(dev):
    import triton_int8_amd as T
    for R, C, seed in ((1024, 14336, 1), (384, 640, 2), (128, 128, 3)):   # second and third smaller than the one before
        x = randn_bf16(make_gen(seed), R, C)
        x[3] = 0
        x[:, 5] = 0
        x[7, 9] = 250.0
        x = x.to(dev)
        ws = torch.full((R + C,), float("nan"), dtype=torch.float32, device=dev)
        want = _call(T, "ti8_quant_row_col_t", x, ws)
        torch.cuda.synchronize()
        before = torch.cuda.memory_stats(dev)["allocation.all.allocated"]
        stream = torch.cuda.current_stream().cuda_stream
        outs = [torch.empty((R, C), dtype=torch.int8, device=dev), torch.empty(R, dtype=torch.float32, device=dev),
                torch.empty((C, R), dtype=torch.int8, device=dev), torch.empty(C, dtype=torch.float32, device=dev)]
        n_alloc = torch.cuda.memory_stats(dev)["allocation.all.allocated"]
        T._lib.call("ti8_quant_row_col_t_noalloc", x.data_ptr(), x.stride(0), outs[0].data_ptr(), C, outs[1].data_ptr(),
                    outs[2].data_ptr(), R, outs[3].data_ptr(), R, C, T._lib.Q_CLAMP, 0, stream)
        assert torch.cuda.memory_stats(dev)["allocation.all.allocated"] == n_alloc > before   # torch's allocator untouched by the call
        torch.cuda.synchronize()
        for got, exp in zip(outs, want):
            assert got.dtype == exp.dtype and torch.equal(got.view(torch.int32) if got.dtype == torch.float32 else got,
                                                          exp.view(torch.int32) if exp.dtype == torch.float32 else exp)


def test_no_alloc_entry_point_rejects_what_it_cannot_hold(dev):
    import triton_int8_amd as T
    x = torch.zeros((128, 128), dtype=torch.bfloat16, device=dev)
    q = torch.empty((128, 128), dtype=torch.int8, device=dev)
    s = torch.empty(128, dtype=torch.float32, device=dev)
    big = T._lib.NOALLOC_MAX_ROWS_PLUS_COLS
    with pytest.raises(T._lib.Ti8Error, match="exceeds"):
        T._lib.call("ti8_quant_row_col_t_noalloc", x.data_ptr(), big, q.data_ptr(), big, s.data_ptr(), q.data_ptr(), 128,
                    s.data_ptr(), 128, big, 1, 0, None)
    with pytest.raises(T._lib.Ti8Error, match="workspace flags"):
        T._lib.call("ti8_quant_row_col_t_noalloc", x.data_ptr(), 128, q.data_ptr(), 128, s.data_ptr(), q.data_ptr(), 128,
                    s.data_ptr(), 128, 128, 1 | T._lib.Q_WS_PINGPONG, 0, None)
