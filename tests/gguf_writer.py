"""A minimal GGUF v3 writer for the tests: metadata of every scalar type, strings, arrays; tensors at aligned offsets."""
import struct

import numpy as np

T_U8, T_I8, T_U16, T_I16, T_U32, T_I32, T_F32, T_BOOL, T_STR, T_ARR, T_U64, T_I64, T_F64 = range(13)
_FMT = {T_U8: "<B", T_I8: "<b", T_U16: "<H", T_I16: "<h", T_U32: "<I", T_I32: "<i", T_F32: "<f", T_BOOL: "<B",
        T_U64: "<Q", T_I64: "<q", T_F64: "<d"}


def _s(b):
    b = b.encode() if isinstance(b, str) else b
    return struct.pack("<Q", len(b)) + b


def _value(t, v):
    if t == T_STR:
        return _s(v)
    if t == T_ARR:
        et, items = v
        return struct.pack("<IQ", et, len(items)) + b"".join(_value(et, x) for x in items)
    return struct.pack(_FMT[t], v)


def write_gguf(path, kv, tensors, alignment=32, version=3, pad_header=True):
    """kv: list of (key, type, value); tensors: list of (name, ggml_type, dims (dims[0] innermost), bytes)."""
    kv = list(kv)
    if alignment != 32:
        kv.append(("general.alignment", T_U32, alignment))
    head = struct.pack("<IIQQ", 0x46554747, version, len(tensors), len(kv))
    for key, t, v in kv:
        head += _s(key) + struct.pack("<I", t) + _value(t, v)
    offs, off = [], 0
    for name, typ, dims, data in tensors:
        offs.append(off)
        off += (len(data) + alignment - 1) // alignment * alignment
    for (name, typ, dims, data), o in zip(tensors, offs):
        head += _s(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        head += struct.pack("<IQ", typ, o)
    with open(path, "wb") as f:
        f.write(head)
        if pad_header:
            f.write(b"\0" * (-len(head) % alignment))
        for name, typ, dims, data in tensors:
            data = np.ascontiguousarray(data, dtype=np.uint8).tobytes()
            f.write(data + b"\0" * (-len(data) % alignment))
    return len(head)
