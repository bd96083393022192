"""Host-side mirror of wick's GPU-backend matmul call sites over the gfx950 C ABI.

Everything here goes through ``libwick_rocm.so`` (``include/wick_rocm.h``); there is
no CPU fallback and no alternative backend: if the library has not been built, or
there is no gfx950 device, construction raises.

The method names follow the reference's call sites so that tests read like the
reference's own:

* ``RocmContext.encode_gemv`` / ``encode_gemm``  -- ``encode_gemv_impl`` /
  ``encode_gemm`` of wick/src/model/metal_lfm2.rs:881-992, 1231-1335
  (f32 activations in, ``X[col*x_stride + i]``; ``Y[col*y_stride + row]`` out).
* ``quantize_q8_0`` / ``gemv_with_preq`` / ``gemm_preq`` -- the CPU call sites
  ``quantize_to_scratch`` / ``quantize_columns`` (wick/src/model/lfm2.rs:571-612),
  ``gemv_with_preq`` (wick/src/backend/cpu.rs:334-354) and ``gemm_preq``
  (wick/src/model/lfm2.rs:539-565) on pre-quantized activations.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Optional, Sequence

import numpy as np

Q4_0 = 2  # ggml type ids, wick/src/gguf.rs:36-51
Q8_0 = 8
Q6_K = 14  # decode GEMV only; 210-byte blocks of 256 weights (wick/src/quant.rs:54-70)
BLOCK_BYTES = {Q4_0: 18, Q8_0: 34}
LAYOUT_TOKEN_MAJOR = 0
LAYOUT_ROW_MAJOR = 1
GEMM_MIN_N = 9  # default hand-off from the multi-token GEMV to the MFMA GEMM ...
GEMM_MIN_N_LARGE = 5  # ... and for weights of 16 MB and more (the reference's GEMM_MIN_N for its Metal path is 16)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libwick_rocm.so")

STATUS_NAMES = {
    0: "OK",
    -1: "INVALID_ARG",
    -2: "UNSUPPORTED_DTYPE",
    -3: "BAD_SHAPE",
    -4: "HIP",
    -5: "NO_DEVICE",
    -6: "STATE",
}


class RocmError(RuntimeError):
    """A C-ABI call returned a negative status (the Rust side would map this to
    WickError::Backend, cf. wick/src/engine.rs:1085-1100)."""

    def __init__(self, status: int, message: str):
        self.status = status
        super().__init__(f"wick_rocm status {status} ({STATUS_NAMES.get(status, '?')}): {message}")


_lib: Optional[C.CDLL] = None

# name -> (restype, argtypes); also the list the symbol-export test walks.
_P = C.c_void_p
_SIGNATURES = {
    "wick_rocm_version": (C.c_char_p, []),
    "wick_rocm_device_count": (C.c_int, [C.POINTER(C.c_int)]),
    "wick_rocm_ctx_create": (C.c_int, [C.c_int, C.POINTER(_P)]),
    "wick_rocm_ctx_destroy": (None, [_P]),
    "wick_rocm_last_error": (C.c_int, [_P, C.c_char_p, C.c_size_t]),
    "wick_rocm_device_info": (C.c_int, [_P, C.c_char_p, C.c_size_t, C.POINTER(C.c_int), C.POINTER(C.c_size_t)]),
    "wick_rocm_ctx_stream": (_P, [_P]),
    "wick_rocm_buffer_alloc": (C.c_int, [_P, C.c_size_t, C.POINTER(_P)]),
    "wick_rocm_buffer_free": (C.c_int, [_P, _P]),
    "wick_rocm_upload": (C.c_int, [_P, _P, _P, C.c_size_t]),
    "wick_rocm_download": (C.c_int, [_P, _P, _P, C.c_size_t]),
    "wick_rocm_sync": (C.c_int, [_P]),
    "wick_rocm_set_gemm_min_n": (C.c_int, [_P, C.c_uint32]),
    "wick_rocm_set_gemm_mfma_shape": (C.c_int, [_P, C.c_int]),
    "wick_rocm_set_gemm_packing": (C.c_int, [_P, C.c_int]),
    "wick_rocm_weight_device_bytes": (C.c_size_t, [_P]),
    "wick_rocm_set_gemm_max_k_splits": (C.c_int, [_P, C.c_uint32]),
    "wick_rocm_set_gemv_policy": (C.c_int, [_P, C.c_int64]),
    "wick_rocm_weight_upload": (C.c_int, [_P, _P, C.c_size_t, C.c_int, C.c_uint32, C.c_uint32, C.POINTER(_P)]),
    "wick_rocm_weight_from_gguf": (C.c_int, [_P, _P, C.c_char_p, C.POINTER(_P)]),
    "wick_rocm_weight_free": (C.c_int, [_P, _P]),
    "wick_rocm_weight_info": (C.c_int, [_P, C.POINTER(C.c_int), C.POINTER(C.c_uint32), C.POINTER(C.c_uint32), C.POINTER(C.c_size_t)]),
    "wick_rocm_weight_device_ptr": (_P, [_P]),
    "wick_rocm_quantize_q8_0": (C.c_int, [_P, _P, C.c_uint32, C.c_uint32, C.c_uint32, _P, _P]),
    "wick_rocm_gemv_q8": (C.c_int, [_P, _P, _P, _P, _P, C.c_int]),
    "wick_rocm_gemv_q8_multi": (C.c_int, [_P, C.POINTER(_P), C.POINTER(_P), C.c_uint32, _P, _P, C.c_int]),
    "wick_rocm_gemm_q8": (C.c_int, [_P, _P, _P, _P, C.c_uint32, _P, C.c_uint32, C.c_int, C.c_int]),
    "wick_rocm_gemm_q8_multi": (C.c_int, [_P, _P, _P, C.c_uint32, _P, _P, C.c_uint32, C.c_uint32, C.c_int, C.c_int]),
    "wick_rocm_gemm_q8_residual_rmsnorm_quantize": (C.c_int, [_P, _P, _P, _P, C.c_uint32, _P, C.c_uint32, _P, C.c_float, _P, _P]),
    "wick_rocm_matmul_f32": (C.c_int, [_P, _P, _P, C.c_size_t, C.c_uint32, C.c_uint32, _P, C.c_size_t, C.c_uint32, C.c_int]),
    "wick_rocm_matmul_f32_noalloc": (C.c_int, [_P, _P, _P, C.c_size_t, C.c_uint32, C.c_uint32, _P, C.c_size_t, C.c_uint32, C.c_int]),
    "wick_rocm_gemv_f32_multi": (C.c_int, [_P, C.POINTER(_P), C.POINTER(_P), C.c_uint32, _P, C.c_size_t, C.c_int]),
    "wick_rocm_gemv_rmsnorm_f32_multi": (C.c_int, [_P, C.POINTER(_P), C.POINTER(_P), C.c_uint32, _P, _P, C.c_float, C.c_int]),
    "wick_rocm_gemv_silu_mul_f32": (C.c_int, [_P, _P, _P, _P, _P, C.c_int]),
    "wick_rocm_ffn_gate_up_f32": (C.c_int, [_P, _P, _P, _P, _P, C.c_float, _P]),
    "wick_rocm_reserve_scratch": (C.c_int, [_P, C.c_uint32, C.c_uint32]),
    "wick_rocm_block_dots_i32": (C.c_int, [_P, _P, _P, C.c_uint32, _P]),
    "wick_rocm_block_dots_f32_i32": (C.c_int, [_P, _P, _P, _P]),
    "wick_rocm_graph_begin": (C.c_int, [_P]),
    "wick_rocm_graph_end": (C.c_int, [_P, C.POINTER(_P)]),
    "wick_rocm_graph_launch": (C.c_int, [_P, _P]),
    "wick_rocm_graph_destroy": (C.c_int, [_P, _P]),
    "wick_rocm_event_create": (C.c_int, [_P, C.POINTER(_P)]),
    "wick_rocm_event_record": (C.c_int, [_P, _P]),
    "wick_rocm_event_elapsed_ms": (C.c_int, [_P, _P, _P, C.POINTER(C.c_float)]),
    "wick_rocm_event_destroy": (C.c_int, [_P, _P]),
    "wick_rocm_kernel_timing_begin": (C.c_int, [_P]),
    "wick_rocm_kernel_timing_end": (C.c_int, [_P, C.POINTER(C.c_double), C.POINTER(C.c_uint64), C.c_int]),
}


def load_library() -> C.CDLL:
    """Loads the built C-ABI library.  Raises if it has not been built: the product
    path never falls back to anything else."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it first (python -c 'import __graft_entry__ as g; g.build()' "
                "or make -C wick_amd/csrc). There is no CPU fallback."
            )
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def device_count() -> int:
    c = C.c_int(0)
    load_library().wick_rocm_device_count(C.byref(c))
    return c.value


class DeviceBuffer:
    """A caller-owned HBM buffer (the counterpart of a Metal `Buffer`)."""

    def __init__(self, ctx: "RocmContext", nbytes: int):
        self.ctx = ctx
        self.nbytes = int(nbytes)
        p = _P()
        ctx._check(ctx._lib.wick_rocm_buffer_alloc(ctx._h, self.nbytes, C.byref(p)))
        self.ptr = p.value

    def upload(self, arr: np.ndarray, offset_bytes: int = 0) -> "DeviceBuffer":
        a = np.ascontiguousarray(arr)
        assert offset_bytes + a.nbytes <= self.nbytes
        self.ctx._check(self.ctx._lib.wick_rocm_upload(self.ctx._h, self.ptr + offset_bytes, a.ctypes.data, a.nbytes))
        return self

    def download(self, dtype, count: int, offset_bytes: int = 0) -> np.ndarray:
        out = np.empty(count, dtype=dtype)
        assert offset_bytes + out.nbytes <= self.nbytes
        self.ctx._check(self.ctx._lib.wick_rocm_download(self.ctx._h, out.ctypes.data, self.ptr + offset_bytes, out.nbytes))
        return out

    def free(self) -> None:
        if self.ptr:
            self.ctx._check(self.ctx._lib.wick_rocm_buffer_free(self.ctx._h, self.ptr))
            self.ptr = None


class RocmWeight:
    """Device-resident weight, GGUF block bytes kept verbatim
    (cf. MetalWeight, wick/src/model/metal_lfm2.rs:28-36)."""

    def __init__(self, ctx: "RocmContext", handle: int, dtype: int, m: int, k: int, nbytes: int):
        self.ctx, self.handle, self.dtype, self.m, self.k, self.nbytes = ctx, handle, dtype, m, k, nbytes

    @property
    def device_bytes(self) -> int:
        """Bytes this weight holds on the device: the raw blocks plus, where it was made, the prefill GEMM's own copy."""
        return int(self.ctx._lib.wick_rocm_weight_device_bytes(self.handle))

    @property
    def device_ptr(self) -> int:
        """Device address of the raw blocks (what the decode GEMVs stream)."""
        return int(self.ctx._lib.wick_rocm_weight_device_ptr(self.handle))

    def free(self) -> None:
        if self.handle:
            self.ctx._check(self.ctx._lib.wick_rocm_weight_free(self.ctx._h, self.handle))
            self.handle = None


def _ptr(b) -> Optional[int]:
    if b is None:
        return None
    if isinstance(b, DeviceBuffer):
        return b.ptr
    return int(b)


class RocmContext:
    def __init__(self, device: int = 0):
        self._lib = load_library()
        h = _P()
        rc = self._lib.wick_rocm_ctx_create(device, C.byref(h))
        if rc != 0:
            raise RocmError(rc, f"cannot create a context on device {device} (need a gfx950 GPU)")
        self._h = h.value
        name = C.create_string_buffer(256)
        cus = C.c_int(0)
        hbm = C.c_size_t(0)
        self._check(self._lib.wick_rocm_device_info(self._h, name, 256, C.byref(cus), C.byref(hbm)))
        self.device_name = name.value.decode()
        self.compute_units = cus.value
        self.hbm_bytes = hbm.value

    # -- plumbing -----------------------------------------------------------
    def _check(self, rc: int) -> None:
        if rc != 0:
            buf = C.create_string_buffer(512)
            self._lib.wick_rocm_last_error(self._h, buf, 512)
            raise RocmError(rc, buf.value.decode(errors="replace"))

    def close(self) -> None:
        if self._h:
            self._lib.wick_rocm_ctx_destroy(self._h)
            self._h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    @property
    def stream(self) -> int:
        return self._lib.wick_rocm_ctx_stream(self._h)

    def sync(self) -> None:
        self._check(self._lib.wick_rocm_sync(self._h))

    def set_gemv_policy(self, direct_max_bytes: int = -1) -> None:
        """Weight-fetch threshold of the n = 1 GEMV (negative = default); results do not depend on it."""
        self._check(self._lib.wick_rocm_set_gemv_policy(self._h, direct_max_bytes))

    def set_gemm_packing(self, enabled: bool) -> None:
        """Whether upload_weight also makes the prefill GEMM's own copy of a Q4_0 / Q8_0 weight (default: yes)."""
        self._check(self._lib.wick_rocm_set_gemm_packing(self._h, 1 if enabled else 0))

    def set_gemm_mfma_shape(self, shape: int = 0) -> None:
        """Block loop of the wide-tile GEMM: 32 (default, also 0) or 16 (the small MFMA shape)."""
        self._check(self._lib.wick_rocm_set_gemm_mfma_shape(self._h, shape))

    def set_gemm_min_n(self, min_n: int) -> None:
        self._check(self._lib.wick_rocm_set_gemm_min_n(self._h, min_n))

    def set_gemm_max_k_splits(self, max_splits: int) -> None:
        """Most K shares of a GEMM launch with few tiles and long K (1: never split, 0: the default)."""
        self._check(self._lib.wick_rocm_set_gemm_max_k_splits(self._h, max_splits))

    def alloc(self, nbytes: int) -> DeviceBuffer:
        return DeviceBuffer(self, nbytes)

    def to_device(self, arr: np.ndarray) -> DeviceBuffer:
        a = np.ascontiguousarray(arr)
        return DeviceBuffer(self, max(a.nbytes, 4)).upload(a)

    # -- weights ------------------------------------------------------------
    def upload_weight(self, blocks: np.ndarray, dtype: int, m: int, k: int) -> RocmWeight:
        a = np.ascontiguousarray(blocks, dtype=np.uint8)
        h = _P()
        self._check(self._lib.wick_rocm_weight_upload(self._h, a.ctypes.data, a.nbytes, dtype, m, k, C.byref(h)))
        return RocmWeight(self, h.value, dtype, m, k, a.nbytes)

    def weight_from_gguf(self, gguf, tensor_name: str) -> RocmWeight:
        """resolve_weight + upload (wick/src/model/lfm2.rs:310-338): `gguf` is a wick_amd.gguf.GgufFile."""
        h = _P()
        self._check(self._lib.wick_rocm_weight_from_gguf(self._h, gguf.handle, tensor_name.encode(), C.byref(h)))
        t, m, k, nb = C.c_int(), C.c_uint32(), C.c_uint32(), C.c_size_t()
        self._check(self._lib.wick_rocm_weight_info(h.value, C.byref(t), C.byref(m), C.byref(k), C.byref(nb)))
        return RocmWeight(self, h.value, t.value, m.value, k.value, nb.value)

    # -- hot path on pre-quantized activations ------------------------------
    def quantize_q8_0(self, x, n: int, k: int, x_stride: int, quants, scales) -> None:
        self._check(self._lib.wick_rocm_quantize_q8_0(self._h, _ptr(x), n, k, x_stride, _ptr(quants), _ptr(scales)))

    def gemv_with_preq(self, w: RocmWeight, scales, quants, y, accumulate: bool = False) -> None:
        self._check(self._lib.wick_rocm_gemv_q8(self._h, w.handle, _ptr(quants), _ptr(scales), _ptr(y), int(accumulate)))

    def gemv_with_preq_multi(self, ws: Sequence[RocmWeight], scales, quants, ys, accumulate: bool = False) -> None:
        n = len(ws)
        wa = (_P * n)(*[w.handle for w in ws])
        ya = (_P * n)(*[_ptr(y) for y in ys])
        self._check(self._lib.wick_rocm_gemv_q8_multi(self._h, wa, ya, n, _ptr(quants), _ptr(scales), int(accumulate)))

    def gemm_preq(self, w: RocmWeight, scales, quants, n: int, y, y_stride: Optional[int] = None,
                  layout: int = LAYOUT_ROW_MAJOR, accumulate: bool = False) -> None:
        if y_stride is None:
            y_stride = n if layout == LAYOUT_ROW_MAJOR else w.m
        self._check(self._lib.wick_rocm_gemm_q8(self._h, w.handle, _ptr(quants), _ptr(scales), n, _ptr(y), y_stride,
                                                layout, int(accumulate)))

    def gemm_preq_multi(self, ws: Sequence[RocmWeight], scales, quants, n: int, ys, y_stride: int, layout: int = LAYOUT_TOKEN_MAJOR,
                        accumulate: bool = False) -> None:
        """1..3 weights over the same quantized activations in one launch (Q / K / V, gate / up of a prompt pass)."""
        c = len(ws)
        wa = (_P * c)(*[w.handle for w in ws])
        ya = (_P * c)(*[_ptr(y) for y in ys])
        self._check(self._lib.wick_rocm_gemm_q8_multi(self._h, wa, ya, c, _ptr(quants), _ptr(scales), n, y_stride, layout, int(accumulate)))

    def gemm_preq_residual_rmsnorm_quantize(self, w: RocmWeight, scales, quants, n: int, x, x_stride: int, norm_weight, eps: float,
                                            out_quants, out_scales) -> None:
        """x[j] += W (activation j), then (out_quants, out_scales) = Q8_0(rmsnorm(x[j]) * norm_weight): a prompt pass's residual
        projection with the norm and quantizer behind it."""
        self._check(self._lib.wick_rocm_gemm_q8_residual_rmsnorm_quantize(self._h, w.handle, _ptr(quants), _ptr(scales), n, _ptr(x), x_stride,
                                                                          _ptr(norm_weight), eps, _ptr(out_quants), _ptr(out_scales)))

    def block_dots_i32(self, w: RocmWeight, quants, n: int, out) -> None:
        self._check(self._lib.wick_rocm_block_dots_i32(self._h, w.handle, _ptr(quants), n, _ptr(out)))

    def block_dots_f32_i32(self, w: RocmWeight, x, out) -> None:
        """The block dots of the fused decode GEMV (f32 activation vector quantized inside the kernel)."""
        self._check(self._lib.wick_rocm_block_dots_f32_i32(self._h, w.handle, _ptr(x), _ptr(out)))

    # -- the reference's GPU call-site shape (f32 in, f32 out) -----------------
    def encode_gemv(self, w: RocmWeight, x, x_off_bytes: int, y, y_off_bytes: int, accumulate: bool = False) -> None:
        self._check(self._lib.wick_rocm_matmul_f32(self._h, w.handle, _ptr(x), x_off_bytes, 1, w.k, _ptr(y), y_off_bytes,
                                                   w.m, int(accumulate)))

    def encode_gemm(self, w: RocmWeight, x, x_off_bytes: int, y, y_off_bytes: int, n: int, x_stride: int, y_stride: int,
                    accumulate: bool = False) -> None:
        self._check(self._lib.wick_rocm_matmul_f32(self._h, w.handle, _ptr(x), x_off_bytes, n, x_stride, _ptr(y),
                                                   y_off_bytes, y_stride, int(accumulate)))

    def encode_gemm_noalloc(self, w: RocmWeight, x, x_off_bytes: int, y, y_off_bytes: int, n: int, x_stride: int, y_stride: int,
                            accumulate: bool = False) -> None:
        """encode_gemm for callers that cannot allocate: quantized activations in the library's static device array."""
        self._check(self._lib.wick_rocm_matmul_f32_noalloc(self._h, w.handle, _ptr(x), x_off_bytes, n, x_stride, _ptr(y),
                                                           y_off_bytes, y_stride, int(accumulate)))

    def encode_gemv_fused(self, ws: Sequence[RocmWeight], x, x_off_bytes: int, ys, accumulate: bool = False) -> None:
        """encode_gemv_qkv / encode_gemv_gate_up: several weights, one f32 activation, one launch."""
        n = len(ws)
        wa = (_P * n)(*[w.handle for w in ws])
        ya = (_P * n)(*[_ptr(y) for y in ys])
        self._check(self._lib.wick_rocm_gemv_f32_multi(self._h, wa, ya, n, _ptr(x), x_off_bytes, int(accumulate)))

    def encode_gemv_rmsnorm_fused(self, ws: Sequence[RocmWeight], x, norm_weight, eps: float, ys, accumulate: bool = False) -> None:
        """encode_gemv_rmsnorm_gate_up (wick/src/model/metal_lfm2.rs:1157-1186) for any 1..4 weights."""
        n = len(ws)
        wa = (_P * n)(*[w.handle for w in ws])
        ya = (_P * n)(*[_ptr(y) for y in ys])
        self._check(self._lib.wick_rocm_gemv_rmsnorm_f32_multi(self._h, wa, ya, n, _ptr(x), _ptr(norm_weight), eps, int(accumulate)))

    def encode_gemv_silu_mul(self, w: RocmWeight, gate, up, y, accumulate: bool = False) -> None:
        """Down projection of silu(gate) * up in one launch."""
        self._check(self._lib.wick_rocm_gemv_silu_mul_f32(self._h, w.handle, _ptr(gate), _ptr(up), _ptr(y), int(accumulate)))

    def encode_ffn_gate_up(self, w_gate: RocmWeight, w_up: RocmWeight, x, norm_weight, eps: float, act) -> None:
        """act = silu(W_gate n(x)) * (W_up n(x)) in one launch (norm_weight may be None: no norm)."""
        self._check(self._lib.wick_rocm_ffn_gate_up_f32(self._h, w_gate.handle, w_up.handle, _ptr(x), _ptr(norm_weight), eps, _ptr(act)))

    def reserve_scratch(self, max_n: int, max_k: int) -> None:
        self._check(self._lib.wick_rocm_reserve_scratch(self._h, max_n, max_k))

    # -- one submission per token ---------------------------------------------
    def graph_begin(self) -> None:
        self._check(self._lib.wick_rocm_graph_begin(self._h))

    def graph_end(self) -> int:
        g = _P()
        self._check(self._lib.wick_rocm_graph_end(self._h, C.byref(g)))
        return g.value

    def graph_launch(self, g: int) -> None:
        self._check(self._lib.wick_rocm_graph_launch(self._h, g))

    def graph_destroy(self, g: int) -> None:
        self._check(self._lib.wick_rocm_graph_destroy(self._h, g))

    # -- GPU timestamps -----------------------------------------------------
    def event(self) -> int:
        e = _P()
        self._check(self._lib.wick_rocm_event_create(self._h, C.byref(e)))
        return e.value

    def record(self, e: int) -> None:
        self._check(self._lib.wick_rocm_event_record(self._h, e))

    def elapsed_ms(self, start: int, stop: int) -> float:
        ms = C.c_float(0)
        self._check(self._lib.wick_rocm_event_elapsed_ms(self._h, start, stop, C.byref(ms)))
        return ms.value

    FAMILIES = ("quantize", "gemv", "gemm", "other")

    def kernel_timing_begin(self) -> None:
        self._check(self._lib.wick_rocm_kernel_timing_begin(self._h))

    def kernel_timing_end(self) -> dict:
        """{family: (total_ms, launches)} of the kernels launched since kernel_timing_begin."""
        ms = (C.c_double * 4)()
        cnt = (C.c_uint64 * 4)()
        self._check(self._lib.wick_rocm_kernel_timing_end(self._h, ms, cnt, 4))
        return {f: (ms[i], int(cnt[i])) for i, f in enumerate(self.FAMILIES)}

    def event_destroy(self, e: int) -> None:
        self._check(self._lib.wick_rocm_event_destroy(self._h, e))
