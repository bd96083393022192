"""ctypes loader for the CPU oracle (TEST INFRASTRUCTURE, not product code).

Only tests, ``__graft_entry__.smoke()`` and ``bench.py``'s cpu-baseline leg may
import this module.  The shipped path (``wick_amd``) never does.

The functions mirror ``oracle/wick_oracle.c`` one to one and take / return numpy
arrays.  Layouts are the reference's: weights are raw GGUF block bytes (row-major
``m`` rows of ``k/32`` blocks), batched Q8_0 activations are ``scales[j*nb + b]``
and ``quants[j*k + ...]`` (wick/src/backend/simd.rs:683-685), GEMM output is
row-major ``out[i*n + j]`` (simd.rs:685).
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

Q4_0 = 2  # ggml type ids, wick/src/gguf.rs:36-51
Q8_0 = 8
BLOCK_BYTES = {Q4_0: 18, Q8_0: 34}

_HERE = os.path.dirname(os.path.abspath(__file__))
_BUILD = os.path.join(_HERE, "_build")


def build(force: bool = False) -> None:
    """Compile the oracle with gcc (seconds)."""
    args = ["make", "-C", _HERE]
    if force:
        args.append("-B")
    subprocess.run(args, check=True, stdout=subprocess.DEVNULL)


def _load(name: str) -> C.CDLL:
    path = os.path.join(_BUILD, name)
    if not os.path.exists(path):
        build()
    return C.CDLL(path)


_lib = None
_x86 = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        L = _load("libwick_oracle.so")
        L.orc_f16_bits_to_f32.restype = C.c_float
        L.orc_f16_bits_to_f32.argtypes = [C.c_uint16]
        L.orc_f32_to_f16_bits.restype = C.c_uint16
        L.orc_f32_to_f16_bits.argtypes = [C.c_float]
        L.orc_quantize_q8_0.restype = C.c_int64
        for f in ("orc_q6k_group_dots_i32", "orc_gemv_q6k_q8", "orc_gemv_q6k_q8_f64"):
            getattr(L, f).restype = C.c_int
        for f in ("orc_block_dots_i32", "orc_gemv_q8", "orc_gemv_q8_f64", "orc_gemm_q8", "orc_gemm_q8_f64"):
            getattr(L, f).restype = C.c_int
        _lib = L
    return _lib


def x86() -> C.CDLL:
    global _x86
    if _x86 is None:
        L = _load("libwick_x86_baseline.so")
        L.orc_x86_gemv_q8_0_f32.restype = C.c_int
        L.orc_x86_prefill_f32.restype = C.c_int
        _x86 = L
    return _x86


def _p(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


def _c(a, dtype) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=dtype)


def f16_bits_to_f32(h: int) -> float:
    return float(lib().orc_f16_bits_to_f32(int(h)))


def f32_to_f16_bits(f: float) -> int:
    return int(lib().orc_f32_to_f16_bits(C.c_float(float(f))))


def dequant_row(ggml_type: int, row_bytes: np.ndarray) -> np.ndarray:
    src = _c(row_bytes, np.uint8)
    nb = src.size // BLOCK_BYTES[ggml_type]
    dst = np.empty(nb * 32, np.float32)
    fn = lib().orc_dequant_q4_0_row if ggml_type == Q4_0 else lib().orc_dequant_q8_0_row
    fn(_p(src), C.c_int64(nb), _p(dst))
    return dst


def dequant_matrix(ggml_type: int, a: np.ndarray, m: int, k: int) -> np.ndarray:
    return dequant_row(ggml_type, a).reshape(m, k)


def quantize_q8_0(x: np.ndarray):
    """One vector -> (scales f32 [k/32], quants i8 [k])."""
    x = _c(x, np.float32).ravel()
    k = x.size
    assert k % 32 == 0
    scales = np.empty(k // 32, np.float32)
    quants = np.empty(k, np.int8)
    lib().orc_quantize_q8_0(_p(x), C.c_int64(k), _p(scales), _p(quants))
    return scales, quants


def quantize_q8_0_batch(x: np.ndarray, n: int, k: int, x_stride: int | None = None):
    """Token-major x[j*x_stride + i] -> (scales [n, k/32], quants [n, k])."""
    x = _c(x, np.float32).ravel()
    x_stride = k if x_stride is None else x_stride
    assert x.size >= (n - 1) * x_stride + k if n else True
    scales = np.empty((n, k // 32), np.float32)
    quants = np.empty((n, k), np.int8)
    lib().orc_quantize_q8_0_batch(_p(x), C.c_int64(n), C.c_int64(k), C.c_int64(x_stride), _p(scales), _p(quants))
    return scales, quants


def block_dots_i32(ggml_type: int, a: np.ndarray, quants: np.ndarray, m: int, n: int, k: int) -> np.ndarray:
    """Exact per-block i32 dots, shape [n, m, k/32]."""
    a = _c(a, np.uint8)
    q = _c(quants, np.int8)
    out = np.empty((n, m, k // 32), np.int32)
    rc = lib().orc_block_dots_i32(ggml_type, _p(a), _p(q), C.c_int64(m), C.c_int64(n), C.c_int64(k), _p(out))
    assert rc == 0
    return out


def gemv_q8(ggml_type: int, a, scales, quants, m: int, k: int, f64: bool = False) -> np.ndarray:
    a = _c(a, np.uint8)
    s = _c(scales, np.float32)
    q = _c(quants, np.int8)
    y = np.empty(m, np.float64 if f64 else np.float32)
    fn = lib().orc_gemv_q8_f64 if f64 else lib().orc_gemv_q8
    rc = fn(ggml_type, _p(a), _p(s), _p(q), _p(y), C.c_int64(m), C.c_int64(k))
    assert rc == 0
    return y


def gemm_q8(ggml_type: int, a, scales, quants, m: int, n: int, k: int, f64: bool = False) -> np.ndarray:
    """Row-major [m, n] output, as gemm_*_q8_0_neon writes it."""
    a = _c(a, np.uint8)
    s = _c(scales, np.float32)
    q = _c(quants, np.int8)
    out = np.empty((m, n), np.float64 if f64 else np.float32)
    fn = lib().orc_gemm_q8_f64 if f64 else lib().orc_gemm_q8
    rc = fn(ggml_type, _p(a), _p(s), _p(q), _p(out), C.c_int64(m), C.c_int64(n), C.c_int64(k))
    assert rc == 0
    return out


def build_matrix(ggml_type: int, values: np.ndarray, m: int, k: int) -> np.ndarray:
    """f32 [m, k] -> raw block bytes with the reference tests' weight quantizers."""
    v = _c(values, np.float32).ravel()
    assert v.size == m * k and k % 32 == 0
    out = np.empty(m * (k // 32) * BLOCK_BYTES[ggml_type], np.uint8)
    fn = lib().orc_build_q4_0_matrix if ggml_type == Q4_0 else lib().orc_build_q8_0_matrix
    fn(_p(v), C.c_int64(m), C.c_int64(k), _p(out))
    return out


# ---- Q6_K (the LM head of shipped LFM2 Q4_0 files) ---------------------------

Q6_K = 14
Q6K_BLOCK_BYTES = 210


def dequant_q6_k(a: np.ndarray, m: int, k: int) -> np.ndarray:
    src = _c(a, np.uint8)
    assert k % 256 == 0 and src.size == m * (k // 256) * Q6K_BLOCK_BYTES
    dst = np.empty(m * k, np.float32)
    lib().orc_dequant_q6_k_row(_p(src), C.c_int64(m * (k // 256)), _p(dst))
    return dst.reshape(m, k)


def q6k_group_dots_i32(a, quants, m: int, k: int) -> np.ndarray:
    """Exact i32 dots of every 16-weight group with its activation quants, shape [m, k/16]."""
    a = _c(a, np.uint8)
    q = _c(quants, np.int8)
    out = np.empty((m, k // 16), np.int32)
    assert lib().orc_q6k_group_dots_i32(_p(a), _p(q), C.c_int64(m), C.c_int64(k), _p(out)) == 0
    return out


def gemv_q6k_q8(a, scales, quants, m: int, k: int, f64: bool = False) -> np.ndarray:
    a = _c(a, np.uint8)
    s = _c(scales, np.float32)
    q = _c(quants, np.int8)
    y = np.empty(m, np.float64 if f64 else np.float32)
    fn = lib().orc_gemv_q6k_q8_f64 if f64 else lib().orc_gemv_q6k_q8
    assert fn(_p(a), _p(s), _p(q), _p(y), C.c_int64(m), C.c_int64(k)) == 0
    return y


def build_q6_k(values: np.ndarray, m: int, k: int) -> np.ndarray:
    v = _c(values, np.float32).ravel()
    assert v.size == m * k and k % 256 == 0
    out = np.empty(m * (k // 256) * Q6K_BLOCK_BYTES, np.uint8)
    lib().orc_build_q6_k_matrix(_p(v), C.c_int64(m), C.c_int64(k), _p(out))
    return out


def fill_normal(seed: int, sigma: float, n: int) -> np.ndarray:
    out = np.empty(n, np.float32)
    lib().orc_fill_normal(C.c_uint64(seed), C.c_float(sigma), C.c_int64(n), _p(out))
    return out


def synth_weight(ggml_type: int, m: int, k: int, seed: int, sigma: float = 0.02) -> np.ndarray:
    """Seeded N(0, sigma^2) weights quantized to raw GGUF blocks."""
    if ggml_type == Q6_K:
        return build_q6_k(fill_normal(seed, sigma, m * k), m, k)
    return build_matrix(ggml_type, fill_normal(seed, sigma, m * k), m, k)


# ---- x86 f32 timing baseline (what the reference runs on an x86 host) -------

def x86_gemv_f32(ggml_type: int, a, x, m: int, k: int, threads: int = 1):
    a = _c(a, np.uint8)
    x = _c(x, np.float32)
    y = np.empty(m, np.float32)
    if ggml_type == Q4_0:
        x86().orc_x86_gemv_q4_0_f32(_p(a), _p(x), _p(y), C.c_int64(m), C.c_int64(k))
        used = 1
    else:
        used = x86().orc_x86_gemv_q8_0_f32(_p(a), _p(x), _p(y), C.c_int64(m), C.c_int64(k), C.c_int(threads))
    return y, used


def x86_prefill_f32(ggml_type: int, a, x, m: int, n: int, k: int, threads: int = 1):
    a = _c(a, np.uint8)
    x = _c(x, np.float32)
    y = np.empty((n, m), np.float32)
    used = x86().orc_x86_prefill_f32(ggml_type, _p(a), _p(x), _p(y), C.c_int64(m), C.c_int64(n), C.c_int64(k),
                                     C.c_int(threads))
    return y, used
