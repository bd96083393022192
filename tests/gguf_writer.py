"""Builds GGUF v3 byte images for the reader tests (not collected by pytest).

Layout per the container the reference parses (wick/src/gguf.rs:404-545): magic, version,
tensor count, kv count, key/value records, tensor infos, padding to the alignment, data."""
import struct

import numpy as np

T_U8, T_I8, T_U16, T_I16, T_U32, T_I32, T_F32, T_BOOL, T_STRING, T_ARRAY, T_U64, T_I64, T_F64 = range(13)
_FMT = {T_U8: "<B", T_I8: "<b", T_U16: "<H", T_I16: "<h", T_U32: "<I", T_I32: "<i", T_F32: "<f", T_BOOL: "<B", T_U64: "<Q",
        T_I64: "<q", T_F64: "<d"}


def gstr(s) -> bytes:
    b = s if isinstance(s, bytes) else s.encode()
    return struct.pack("<Q", len(b)) + b


def value(type_id, v) -> bytes:
    """Encoded value WITHOUT its leading type id.  Arrays are (elem_type, [items])."""
    if type_id in _FMT:
        return struct.pack(_FMT[type_id], v)
    if type_id == T_STRING:
        return gstr(v)
    if type_id == T_ARRAY:
        et, items = v
        return struct.pack("<IQ", et, len(items)) + b"".join(value(et, x) for x in items)
    raise ValueError(type_id)


def build(metadata=(), tensors=(), version=3, magic=b"GGUF", alignment=None, pad_tail=0):
    """metadata: [(key, type_id, value)], tensors: [(name, dims, ggml_type, bytes-like)].
    Returns (image bytes, {name: absolute offset})."""
    metadata = list(metadata)
    if alignment is not None:
        metadata.append(("general.alignment", T_U32, alignment))
    align = alignment or 32
    head = magic + struct.pack("<IQQ", version, len(tensors), len(metadata))
    for k, t, v in metadata:
        head += gstr(k) + struct.pack("<I", t) + value(t, v)
    rel, offsets = 0, []
    for _, _, _, data in tensors:
        offsets.append(rel)
        rel += -(-len(bytes(data)) // align) * align
    for (name, dims, gt, _), off in zip(tensors, offsets):
        head += gstr(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims) + struct.pack("<IQ", gt, off)
    data_offset = -(-len(head) // align) * align
    img = bytearray(head) + bytes(data_offset - len(head))
    absolute = {}
    for (name, _, _, data), off in zip(tensors, offsets):
        b = bytes(data)
        absolute[name] = data_offset + off
        img += b + bytes(-(-len(b) // align) * align - len(b))
    img += bytes(pad_tail)
    return bytes(img), absolute


def as_bytes(a: np.ndarray) -> bytes:
    return np.ascontiguousarray(a).tobytes()
