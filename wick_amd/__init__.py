"""wick_amd: MI355X (gfx950) backend for wick's block-quantized matmul hot path.

Scope: Q8_0 activation quantization, the decode GEMV and the batched prefill GEMM
over raw GGUF Q4_0 / Q8_0 weight blocks.  The product is the C-ABI library built
from ``wick_amd/csrc`` (``include/wick_rocm.h``); ``wick_amd.rocm`` is the host-side
mirror of the reference's call sites used by the tests and the benchmark.
"""
from . import build as build  # noqa: F401
from .rocm import (  # noqa: F401
    GEMM_MIN_N,
    GEMM_MIN_N_LARGE,
    LAYOUT_ROW_MAJOR,
    LAYOUT_TOKEN_MAJOR,
    Q4_0,
    Q6_K,
    Q8_0,
    DeviceBuffer,
    RocmContext,
    RocmError,
    RocmWeight,
    device_count,
    load_library,
)
