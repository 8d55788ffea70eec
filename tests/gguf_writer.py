"""Writes small GGUF v3 files for the loader tests (layout: crates/strix-models/src/gguf.rs:119-176)."""
import struct

import numpy as np

T_U8, T_I8, T_U16, T_I16, T_U32, T_I32, T_F32, T_BOOL, T_STR, T_ARR, T_U64, T_I64, T_F64 = range(13)
_FMT = {T_U8: "<B", T_I8: "<b", T_U16: "<H", T_I16: "<h", T_U32: "<I", T_I32: "<i", T_F32: "<f", T_BOOL: "<B",
        T_U64: "<Q", T_I64: "<q", T_F64: "<d"}


def _s(s):
    b = s.encode()
    return struct.pack("<Q", len(b)) + b


def _value(ty, v):
    if ty == T_STR:
        return _s(v)
    if ty == T_ARR:
        ety, items = v
        return struct.pack("<IQ", ety, len(items)) + b"".join(_value(ety, x) for x in items)
    return struct.pack(_FMT[ty], v)


def write_gguf(path, meta, tensors, version=3, alignment=None, magic=0x46554747):
    """meta: [(key, type, value)]; tensors: [(name, ggml_type, dims, raw uint8 array)]."""
    meta = list(meta)
    if alignment is not None:
        meta.append(("general.alignment", T_U32, alignment))
    align = alignment or 32
    out = struct.pack("<IIQQ", magic, version, len(tensors), len(meta))
    for k, ty, v in meta:
        out += _s(k) + struct.pack("<I", ty) + _value(ty, v)
    off, offs = 0, []
    for _, _, _, raw in tensors:
        offs.append(off)
        off += -(-len(raw) // align) * align
    for (name, ty, dims, _), o in zip(tensors, offs):
        out += _s(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        out += struct.pack("<IQ", ty, o)
    out += b"\0" * (-len(out) % align)
    for (_, _, _, raw), o in zip(tensors, offs):
        raw = np.ascontiguousarray(raw, np.uint8).tobytes()
        out += raw + b"\0" * (-len(raw) % align)
    with open(path, "wb") as f:
        f.write(out)
    return path
