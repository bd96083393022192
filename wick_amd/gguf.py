"""Host mirror of the GGUF reader in ``libwick_rocm.so`` (``include/wick_gguf.h``).

Mirrors the reference's ``GgufFile`` accessors (wick/src/gguf.rs:331-693): ``open`` /
``from_bytes``, typed metadata getters that match only the exact stored type, tensor
infos with absolute offsets, and ``tensor_meta`` (rows = ne1, cols = ne0).
"""
from __future__ import annotations

import ctypes as C
from typing import List, Optional, Tuple

import numpy as np

from . import rocm

_P = C.c_void_p
_CP = C.POINTER(C.c_char)  # strings in a GGUF file are not NUL-terminated

_SIGNATURES = {
    "wick_gguf_last_error": (C.c_char_p, []),
    "wick_gguf_open": (C.c_int, [C.c_char_p, C.POINTER(_P)]),
    "wick_gguf_from_bytes": (C.c_int, [_P, C.c_size_t, C.POINTER(_P)]),
    "wick_gguf_close": (None, [_P]),
    "wick_gguf_data": (_P, [_P, C.POINTER(C.c_size_t)]),
    "wick_gguf_data_offset": (C.c_size_t, [_P]),
    "wick_gguf_alignment": (C.c_uint32, [_P]),
    "wick_gguf_metadata_count": (C.c_uint64, [_P]),
    "wick_gguf_metadata_key": (C.c_int, [_P, C.c_uint64, C.POINTER(_CP), C.POINTER(C.c_size_t)]),
    "wick_gguf_value_type": (C.c_int, [_P, C.c_char_p, C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_uint64)]),
    "wick_gguf_get_u32": (C.c_int, [_P, C.c_char_p, C.POINTER(C.c_uint32)]),
    "wick_gguf_get_f32": (C.c_int, [_P, C.c_char_p, C.POINTER(C.c_float)]),
    "wick_gguf_get_bool": (C.c_int, [_P, C.c_char_p, C.POINTER(C.c_int)]),
    "wick_gguf_get_str": (C.c_int, [_P, C.c_char_p, C.POINTER(_CP), C.POINTER(C.c_size_t)]),
    "wick_gguf_get_int": (C.c_int, [_P, C.c_char_p, C.POINTER(C.c_int64)]),
    "wick_gguf_get_array": (C.c_int, [_P, C.c_char_p, C.c_int, C.POINTER(_P), C.POINTER(C.c_uint64)]),
    "wick_gguf_get_array_str": (C.c_int, [_P, C.c_char_p, C.c_uint64, C.POINTER(_CP), C.POINTER(C.c_size_t)]),
    "wick_gguf_tensor_count": (C.c_uint64, [_P]),
    "wick_gguf_tensor_name": (C.c_int, [_P, C.c_uint64, C.POINTER(_CP), C.POINTER(C.c_size_t)]),
    "wick_gguf_tensor_info": (C.c_int, [_P, C.c_char_p, C.POINTER(C.c_int), C.POINTER(C.c_uint32), C.POINTER(C.c_uint64),
                                        C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]),
    "wick_gguf_tensor_data": (C.c_int, [_P, C.c_char_p, C.POINTER(_P), C.POINTER(C.c_size_t)]),
    "wick_gguf_tensor_meta": (C.c_int, [_P, C.c_char_p, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64), C.POINTER(C.c_uint64),
                                        C.POINTER(C.c_int)]),
    "wick_gguf_tensor_data_size": (C.c_int, [C.c_int, C.c_uint64, C.POINTER(C.c_uint64)]),
    "wick_gguf_type_name": (C.c_char_p, [C.c_int]),
}

# metadata value type ids (wick/src/gguf.rs:20-33) -> numpy dtype of fixed-size scalars
T_U8, T_I8, T_U16, T_I16, T_U32, T_I32, T_F32, T_BOOL, T_STRING, T_ARRAY, T_U64, T_I64, T_F64 = range(13)
_NP = {T_U8: "<u1", T_I8: "<i1", T_U16: "<u2", T_I16: "<i2", T_U32: "<u4", T_I32: "<i4", T_F32: "<f4", T_BOOL: "<u1",
       T_U64: "<u8", T_I64: "<i8", T_F64: "<f8"}

STATUS_NAMES = {0: "OK", -1: "INVALID_ARG", -2: "IO", -3: "FORMAT", -4: "NOT_FOUND", -5: "UNSUPPORTED"}

_bound = False


class GgufError(RuntimeError):
    """A wick_gguf_* call failed (the reference returns anyhow errors from the same places)."""

    def __init__(self, status: int, message: str):
        self.status = status
        super().__init__(f"wick_gguf status {status} ({STATUS_NAMES.get(status, '?')}): {message}")


def _lib() -> C.CDLL:
    global _bound
    lib = rocm.load_library()
    if not _bound:
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _bound = True
    return lib


def _check(rc: int) -> None:
    if rc != 0:
        raise GgufError(rc, _lib().wick_gguf_last_error().decode("utf-8", "replace"))


def tensor_data_size(ggml_type: int, numel: int) -> int:
    """tensor_data_size, wick/src/gguf.rs:297-320."""
    out = C.c_uint64()
    _check(_lib().wick_gguf_tensor_data_size(ggml_type, numel, C.byref(out)))
    return out.value


def type_name(ggml_type: int) -> str:
    return _lib().wick_gguf_type_name(ggml_type).decode()


class GgufFile:
    """An open GGUF v3 file.  Tensor bytes are views into the handle's memory: keep the
    object alive while they are in use."""

    def __init__(self, handle: int):
        self._h = handle

    @classmethod
    def open(cls, path: str) -> "GgufFile":
        h = _P()
        _check(_lib().wick_gguf_open(str(path).encode(), C.byref(h)))
        return cls(h.value)

    @classmethod
    def from_bytes(cls, data: bytes) -> "GgufFile":
        h = _P()
        buf = (C.c_char * len(data)).from_buffer_copy(data) if len(data) else None
        _check(_lib().wick_gguf_from_bytes(buf, len(data), C.byref(h)))
        return cls(h.value)

    def close(self) -> None:
        if self._h:
            _lib().wick_gguf_close(self._h)
            self._h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    @property
    def handle(self) -> int:
        return self._h

    # -- whole file -------------------------------------------------------------
    @property
    def size(self) -> int:
        n = C.c_size_t()
        _lib().wick_gguf_data(self._h, C.byref(n))
        return n.value

    @property
    def data_offset(self) -> int:
        return _lib().wick_gguf_data_offset(self._h)

    @property
    def alignment(self) -> int:
        return _lib().wick_gguf_alignment(self._h)

    # -- metadata ---------------------------------------------------------------
    def keys(self) -> List[str]:
        out = []
        for i in range(_lib().wick_gguf_metadata_count(self._h)):
            p, n = _CP(), C.c_size_t()
            _check(_lib().wick_gguf_metadata_key(self._h, i, C.byref(p), C.byref(n)))
            out.append(C.string_at(p, n.value).decode())
        return out

    def value_type(self, key: str) -> Tuple[int, int, int]:
        t, e, n = C.c_int(), C.c_int(), C.c_uint64()
        _check(_lib().wick_gguf_value_type(self._h, key.encode(), C.byref(t), C.byref(e), C.byref(n)))
        return t.value, e.value, n.value

    def _opt(self, fn, key, out):
        rc = fn(self._h, key.encode(), C.byref(out))
        if rc == -4:  # NOT_FOUND: the reference's getters return None
            return None
        _check(rc)
        return out.value

    def get_u32(self, key: str) -> Optional[int]:
        return self._opt(_lib().wick_gguf_get_u32, key, C.c_uint32())

    def get_f32(self, key: str) -> Optional[float]:
        return self._opt(_lib().wick_gguf_get_f32, key, C.c_float())

    def get_bool(self, key: str) -> Optional[bool]:
        v = self._opt(_lib().wick_gguf_get_bool, key, C.c_int())
        return None if v is None else bool(v)

    def get_int(self, key: str) -> Optional[int]:
        return self._opt(_lib().wick_gguf_get_int, key, C.c_int64())

    def get_str(self, key: str) -> Optional[str]:
        p, n = _CP(), C.c_size_t()
        rc = _lib().wick_gguf_get_str(self._h, key.encode(), C.byref(p), C.byref(n))
        if rc == -4:
            return None
        _check(rc)
        return C.string_at(p, n.value).decode("utf-8", "replace")

    def architecture(self) -> Optional[str]:
        return self.get_str("general.architecture")

    def get_array(self, key: str, elem_type: int) -> Optional[np.ndarray]:
        """get_f32_array / get_i32_array (wick/src/gguf.rs:589-629): None unless the stored element type matches."""
        p, n = _P(), C.c_uint64()
        rc = _lib().wick_gguf_get_array(self._h, key.encode(), elem_type, C.byref(p), C.byref(n))
        if rc == -4:
            return None
        _check(rc)
        dt = np.dtype(_NP[elem_type])
        return np.frombuffer(C.string_at(p.value, n.value * dt.itemsize), dtype=dt).copy()

    def get_string_array(self, key: str) -> Optional[List[str]]:
        try:
            t, e, n = self.value_type(key)
        except GgufError:
            return None
        if t != T_ARRAY or e != T_STRING:
            return None
        out = []
        for i in range(n):
            p, ln = _CP(), C.c_size_t()
            _check(_lib().wick_gguf_get_array_str(self._h, key.encode(), i, C.byref(p), C.byref(ln)))
            out.append(C.string_at(p, ln.value).decode("utf-8", "replace"))
        return out

    # -- tensors ----------------------------------------------------------------
    def tensor_names(self) -> List[str]:
        out = []
        for i in range(_lib().wick_gguf_tensor_count(self._h)):
            p, n = _CP(), C.c_size_t()
            _check(_lib().wick_gguf_tensor_name(self._h, i, C.byref(p), C.byref(n)))
            out.append(C.string_at(p, n.value).decode())
        return out

    def tensor_info(self, name: str) -> dict:
        t, nd, dims, off, size = C.c_int(), C.c_uint32(), (C.c_uint64 * 8)(), C.c_uint64(), C.c_uint64()
        _check(_lib().wick_gguf_tensor_info(self._h, name.encode(), C.byref(t), C.byref(nd), dims, C.byref(off), C.byref(size)))
        return {"name": name, "ggml_type": t.value, "shape": list(dims[: nd.value]), "offset": off.value, "size_bytes": size.value}

    def tensor_data(self, name: str) -> np.ndarray:
        p, n = _P(), C.c_size_t()
        _check(_lib().wick_gguf_tensor_data(self._h, name.encode(), C.byref(p), C.byref(n)))
        return np.ctypeslib.as_array(C.cast(p, C.POINTER(C.c_uint8)), shape=(n.value,))

    def tensor_meta(self, name: str) -> Tuple[int, int, int, int]:
        """(absolute byte offset, rows, cols, ggml type), wick/src/gguf.rs:678-693."""
        off, rows, cols, t = C.c_uint64(), C.c_uint64(), C.c_uint64(), C.c_int()
        _check(_lib().wick_gguf_tensor_meta(self._h, name.encode(), C.byref(off), C.byref(rows), C.byref(cols), C.byref(t)))
        return off.value, rows.value, cols.value, t.value


# ---- writing (synthetic models for benchmarks; the reference only reads GGUF) ----------------------------

def _gstr(s) -> bytes:
    b = s if isinstance(s, bytes) else str(s).encode()
    return len(b).to_bytes(8, "little") + b


def _gvalue(type_id: int, v) -> bytes:
    if type_id in _NP:
        return np.array(v, dtype=_NP[type_id]).tobytes()
    if type_id == T_STRING:
        return _gstr(v)
    if type_id == T_ARRAY:
        elem_type, items = v
        return int(elem_type).to_bytes(4, "little") + len(items).to_bytes(8, "little") + b"".join(_gvalue(elem_type, x) for x in items)
    raise ValueError(f"unknown GGUF value type {type_id}")


def build_image(metadata, tensors, alignment: int = 32) -> bytes:
    """A GGUF v3 image from ``[(key, value_type, value)]`` and ``[(name, dims, ggml_type, bytes-like)]``
    (dims in GGUF order: ne0 first).  Tensor data is laid out in the given order, each padded to `alignment`."""
    head = bytearray(b"GGUF" + (3).to_bytes(4, "little") + len(tensors).to_bytes(8, "little") + len(metadata).to_bytes(8, "little"))
    for key, t, v in metadata:
        head += _gstr(key) + int(t).to_bytes(4, "little") + _gvalue(t, v)
    blobs = [np.ascontiguousarray(d).view(np.uint8).ravel() if isinstance(d, np.ndarray) else np.frombuffer(bytes(d), np.uint8) for *_, d in tensors]
    rel = 0
    for (name, dims, gt, _), blob in zip(tensors, blobs):
        head += _gstr(name) + len(dims).to_bytes(4, "little") + b"".join(int(d).to_bytes(8, "little") for d in dims)
        head += int(gt).to_bytes(4, "little") + rel.to_bytes(8, "little")
        rel += -(-blob.size // alignment) * alignment
    data_offset = -(-len(head) // alignment) * alignment
    out = np.zeros(data_offset + rel, np.uint8)
    out[: len(head)] = np.frombuffer(bytes(head), np.uint8)
    at = data_offset
    for blob in blobs:
        out[at: at + blob.size] = blob
        at += -(-blob.size // alignment) * alignment
    return out.tobytes()
