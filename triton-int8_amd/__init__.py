"""MI355X-native INT8 quantized linear layer (forward + backward).

Drop-in replacements of the jiaoch/Triton-INT8 scripts, one module per script with
the same function names (``fwd_32``, ``bwd_33``, ``int8_gemm_pipeline``,
``triton_per_block_quant`` ...), running on hand-written gfx950 HIP kernels loaded
from ``libti8.so`` through its C ABI.  There is no fallback path: without the built
library every operator raises.

The directory name carries a hyphen, so import it as ``triton_int8_amd`` (the
top-level shim of that name loads this package).
"""
from . import _lib  # noqa: F401
from . import (block_channel_bwd33, block_channel_fwd32, decoder, double_channel_bwd33, double_channel_fwd32,
               double_channel_triton_bwd, double_channel_triton_fwd, fused_bwd33, fused_fwd32, graph, latency, linear, ops,
               tilelang_block_channel_bwd, tilelang_block_channel_fwd)
from ._common import calc_diff
from ._lib import init, last_gemm_kernel
from .decoder import DecoderLayer
from .graph import GraphedStep
from .linear import Int8Linear, Int8LinearFunction, linear_fwd_bwd

__version__ = "0.1.0"
