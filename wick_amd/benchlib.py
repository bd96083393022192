"""ctypes mirror of libwick_rocm_bench.so: bench.py's measurement aids (wick_amd/csrc/bench).  Not part of the backend:
nothing in wick_amd.rocm or the C ABI of include/wick_rocm.h refers to it."""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

from .rocm import RocmContext, RocmError, RocmWeight, _ptr

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libwick_rocm_bench.so")
_P = C.c_void_p
_SIGNATURES = {
    "wick_bench_probe_rate": (C.c_int, [_P, C.c_int, C.c_uint32, C.c_int, C.POINTER(C.c_double)]),
    "wick_bench_copy": (C.c_int, [_P, _P, _P, C.c_size_t]),
    "wick_bench_gemv_q8_span": (C.c_int, [_P, C.c_int, _P, C.c_uint32, C.c_uint32, _P, _P, _P, C.c_int, _P, C.c_uint32, C.POINTER(C.c_uint32)]),
}
_lib = None


def load_library() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: build it first (make -C wick_amd/csrc)")
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


def _check(rc: int, what: str) -> None:
    if rc != 0:
        raise RocmError(rc, f"{what} failed")


def probe_rate(ctx: RocmContext, shape: int, iters: int) -> float:
    """Enqueues a register-only instruction-rate probe on the context's stream; returns the operations it performs."""
    ops = C.c_double()
    _check(load_library().wick_bench_probe_rate(ctx.stream, shape, iters, ctx.compute_units, C.byref(ops)), "probe_rate")
    return ops.value


def copy(ctx: RocmContext, dst, src, nbytes: int) -> None:
    _check(load_library().wick_bench_copy(ctx.stream, _ptr(dst), _ptr(src), nbytes), "copy")


def gemv_q8_span(ctx: RocmContext, w: RocmWeight, d_scales, d_quants, d_y, d_span, span_capacity_waves: int) -> int:
    """The decode GEMV through its product kernel with the timing hook; returns the number of wave records written to d_span."""
    waves = C.c_uint32()
    _check(load_library().wick_bench_gemv_q8_span(ctx.stream, w.dtype, w.device_ptr, w.m, w.k, _ptr(d_quants), _ptr(d_scales), _ptr(d_y),
                                                  ctx.compute_units, _ptr(d_span), span_capacity_waves, C.byref(waves)), "gemv_q8_span")
    return waves.value


def span_us(records: np.ndarray) -> float:
    """First wave start -> last wave end of one launch's [waves][2] wall-clock records (100 MHz), in microseconds."""
    r = records.reshape(-1, 2)
    return float(int(r[:, 1].max()) - int(r[:, 0].min())) / 100.0
