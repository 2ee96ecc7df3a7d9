"""ctypes binding of ``libti8.so`` (the C ABI declared in ``include/ti8.h``).

The library is the product: there is no fallback.  If it has not been built
(``python triton-int8_amd/build.py``) importing any operator raises.
"""
import contextlib
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libti8.so")

_i64, _int, _f32, _vp = ctypes.c_int64, ctypes.c_int, ctypes.c_float, ctypes.c_void_p

class QBlockOperand(ctypes.Structure):
    """ti8_qblock_operand of include/ti8.h."""
    _fields_ = [("x", _vp), ("bsx", _i64), ("ldx", _i64), ("q", _vp), ("bsq", _i64), ("ldq", _i64),
                ("qT", _vp), ("bsqt", _i64), ("ldqt", _i64), ("s", _vp), ("ssb", _i64), ("ssr", _i64), ("ssc", _i64),
                ("B", _i64), ("R", _i64), ("C", _i64)]

class GemmProblem(ctypes.Structure):
    """ti8_gemm_problem of include/ti8.h."""
    _fields_ = [("A", _vp), ("bsa", _i64), ("lda", _i64), ("B", _vp), ("bsb", _i64), ("ldb", _i64),
                ("C", _vp), ("bsc", _i64), ("ldc", _i64),
                ("sA", _vp), ("modeA", _int), ("sa_bs", _i64), ("sa_rs", _i64), ("sa_ks", _i64),
                ("sB", _vp), ("modeB", _int), ("sb_bs", _i64), ("sb_rs", _i64), ("sb_ks", _i64),
                ("batch", _i64), ("M", _i64), ("N", _i64), ("K", _i64), ("acc_i32_full", _int), ("combine", _int),
                ("out_scale", _f32), ("post_scale", _f32)]


# name -> argument types, in the order of include/ti8.h
PROTOTYPES = {
    "ti8_quant_block": [_vp, _i64, _i64, _vp, _i64, _i64, _vp, _i64, _i64, _vp, _i64, _i64, _i64,
                        _i64, _i64, _i64, _int, _int, _int, _vp],
    "ti8_quant_block_multi": [ctypes.POINTER(QBlockOperand), _int, _int, _int, _vp],
    "ti8_quant_block_had128": [_vp, _i64, _i64, _vp, _i64, _i64, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _int, _int, _int, _vp],
    "ti8_quant_row": [_vp, _i64, _vp, _i64, _vp, _i64, _i64, _int, _int, _int, _vp],
    "ti8_quant_col_t": [_vp, _i64, _vp, _i64, _vp, _vp, _i64, _i64, _int, _int, _vp],
    "ti8_quant_row_col_t": [_vp, _i64, _vp, _i64, _vp, _vp, _i64, _vp, _vp, _i64, _i64, _int, _int, _vp],
    "ti8_quant_row_col_t_noalloc": [_vp, _i64, _vp, _i64, _vp, _vp, _i64, _vp, _i64, _i64, _int, _int, _vp],
    "ti8_fwht": [_vp, _i64, _vp, _i64, _i64, _i64, _i64, _f32, _vp],
    "ti8_fwht_t": [_vp, _i64, _vp, _i64, _i64, _i64, _f32, _vp],
    "ti8_fwht_quant_row": [_vp, _i64, _vp, _i64, _vp, _i64, _i64, _i64, _int, _int, _vp],
    "ti8_fwht_t_quant_row": [_vp, _i64, _vp, _vp, _i64, _vp, _i64, _i64, _int, _int, _vp],
    "ti8_gemm_i8_nt": [_vp, _i64, _i64, _vp, _i64, _i64, _vp, _i64, _i64,
                       _vp, _int, _i64, _i64, _i64, _vp, _int, _i64, _i64, _i64,
                       _i64, _i64, _i64, _i64, _int, _int, _f32, _f32, _int, _vp],
    "ti8_gemm_i8_nt_multi": [ctypes.POINTER(GemmProblem), _int, _int, _vp],
    "ti8_gemm_i8_nt_i32": [_vp, _i64, _i64, _vp, _i64, _i64, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _vp],
    "ti8_linear_fwd_bwd": [_vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _i64, _i64, _i64, _i64, _int, _int, _vp, _i64, _vp],
    "ti8_probe_mfma": [_vp, _i64, _vp, _int, _int, _int, _int, _vp],
}
EXPORTS = ["ti8_version", "ti8_last_error", "ti8_arch", "ti8_init", "ti8_last_gemm_kernel", "ti8_linear_fwd_bwd_workspace"] + list(PROTOTYPES)

# enums of include/ti8.h
Q_CLAMP, Q_EPS_ADD, Q_SCALE_BF16, Q_HAD128, Q_WS_PINGPONG, Q_WS_SECOND, Q_TORCH_ROUND, Q_TORCH_BF16, Q_WS_IS_ZERO = 1, 2, 4, 8, 16, 32, 64, 128, 256
INV_RCP_OF_SCALE, INV_AMAX_DIV_127, INV_AMAX_MUL_RCP127, INV_MULTIPLIER = 0, 1, 2, 3
SCALE_ROW, SCALE_BLOCK128, SCALE_ROW_K128, SCALE_BLOCK_K256 = 0, 1, 2, 3
COMBINE_MUL_MUL, COMBINE_MUL_PROD, COMBINE_DIV_PROD = 0, 1, 2
GEMM_STRICT, GEMM_TILED, GEMM_SKINNY, GEMM_LARGE_TILES, GEMM_ONE_TILE = 1, 2, 4, 8, 16
NOALLOC_MAX_ROWS_PLUS_COLS = 65536
SCHEME_BLOCK_CHANNEL, SCHEME_DOUBLE_CHANNEL = 0, 2
KERNEL_NONE, KERNEL_ONE_TILE, KERNEL_ONE_TILE_MULTI, KERNEL_PERSISTENT_CHAIN, KERNEL_FEW_ROWS = 0, 1, 2, 3, 4

_lib = None


class Ti8Error(RuntimeError):
    """A libti8 entry point returned a non-zero status."""

    def __init__(self, fn, code, msg):
        super().__init__(f"{fn} failed with status {code}: {msg}")
        self.code = code


def lib():
    """The loaded library (loaded once).  Raises if it was never built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python triton-int8_amd/build.py` "
                "(hipcc, gfx950).  There is no fallback implementation.")
        l = ctypes.CDLL(LIB_PATH)
        l.ti8_version.restype = _int
        l.ti8_last_error.restype = ctypes.c_char_p
        l.ti8_arch.restype = ctypes.c_char_p
        l.ti8_init.restype = _int
        l.ti8_init.argtypes = []
        l.ti8_last_gemm_kernel.restype = _int
        l.ti8_last_gemm_kernel.argtypes = []
        l.ti8_linear_fwd_bwd_workspace.restype = _i64
        l.ti8_linear_fwd_bwd_workspace.argtypes = [_i64, _i64, _i64, _int]
        for name, args in PROTOTYPES.items():
            fn = getattr(l, name)
            fn.argtypes = args
            fn.restype = _int
        _lib = l
    return _lib


_timing = None  # {entry point: [(start event, end event), ...]} while `timed_launches` is active


@contextlib.contextmanager
def timed_launches():
    """Bracket every entry-point call with a pair of HIP events on the launch stream.

    Yields the dict the pairs are appended to (``{name: [(start, end), ...]}``); read
    ``start.elapsed_time(end)`` after a device synchronise.  Used by the benchmark to time the
    kernels of a whole step where they run, between the other launches of that step.
    """
    global _timing
    import torch
    rec = {}
    _timing = (rec, torch.cuda.Event)
    try:
        yield rec
    finally:
        _timing = None


def call(name, *args):
    """Call an entry point; raise :class:`Ti8Error` with the library's message on failure."""
    l = lib()
    t = _timing
    if t is None:
        rc = getattr(l, name)(*args)
    else:
        rec, Event = t
        a, b = Event(enable_timing=True), Event(enable_timing=True)
        a.record()
        rc = getattr(l, name)(*args)
        b.record()
        rec.setdefault(name, []).append((a, b))
    if rc != 0:
        raise Ti8Error(name, rc, l.ti8_last_error().decode())


def init():
    """One-time set-up of the library on the current device (``ti8_init``): kernel attributes, device
    properties, the fixed scratch array.  Optional; a caller that times or captures its first call
    runs it beforehand.  Returns the library's note (empty, or that the persistent GEMM kernel is not
    available on this device)."""
    l = lib()
    rc = l.ti8_init()
    if rc != 0:
        raise Ti8Error("ti8_init", rc, l.ti8_last_error().decode())
    return l.ti8_last_error().decode()


_EPILOGUES = ("int32 out", "per-row scales, int32 over the whole K", "promotion per K tile", "literal arithmetic",
              "promotion per K tile, per-lane factors", "chained promotion per K tile")
_KINDS = {KERNEL_NONE: "none", KERNEL_ONE_TILE: "gemm_i8_kernel (one workgroup per tile)",
          KERNEL_ONE_TILE_MULTI: "gemm_i8_multi_kernel (one workgroup per tile, several GEMMs per launch)",
          KERNEL_PERSISTENT_CHAIN: "gemm_i8_chain_kernel (persistent workgroups)",
          KERNEL_FEW_ROWS: "gemm_i8_wavering_kernel (few rows)"}


def describe_gemm_kernel(kernel_id=None):
    """Text for a value of ``ti8_last_gemm_kernel`` (default: the current one): kernel, tile, epilogue."""
    if kernel_id is None:
        kernel_id = lib().ti8_last_gemm_kernel()
    kind, epi, bm, bn = kernel_id & 0xff, (kernel_id >> 8) & 0xff, ((kernel_id >> 16) & 0xf) * 64, ((kernel_id >> 20) & 0xf) * 64
    name = _KINDS.get(kind, f"kernel kind {kind}")
    if kind in (KERNEL_NONE, KERNEL_FEW_ROWS):
        return name
    return f"{name}, {bm}x{bn} tiles, {_EPILOGUES[epi] if epi < len(_EPILOGUES) else epi}"


def last_gemm_kernel():
    """Kind of the GEMM kernel that the last GEMM entry point called from this thread launched
    (``KERNEL_*``): kernels of one family give the same bits, so this is how a caller tells which ran."""
    return lib().ti8_last_gemm_kernel() & 0xff
