"""Minimal GGUF v3 writer for synthetic models (the container mesh-client/src/models/gguf.rs reads)."""
import struct

import numpy as np

T_U8, T_I8, T_U16, T_I16, T_U32, T_I32, T_F32, T_BOOL, T_STR, T_ARR, T_U64, T_I64, T_F64 = range(13)


def _s(x):
    b = x.encode()
    return struct.pack("<Q", len(b)) + b


def kv_bytes(key, vtype, value):
    out = _s(key) + struct.pack("<I", vtype)
    if vtype == T_U32:
        out += struct.pack("<I", value)
    elif vtype == T_I32:
        out += struct.pack("<i", value)
    elif vtype == T_F32:
        out += struct.pack("<f", value)
    elif vtype == T_U64:
        out += struct.pack("<Q", value)
    elif vtype == T_STR:
        out += _s(value)
    elif vtype == T_BOOL:
        out += struct.pack("<B", 1 if value else 0)
    elif vtype == T_ARR:
        et, items = value
        out += struct.pack("<IQ", et, len(items))
        for it in items:
            out += _s(it) if et == T_STR else struct.pack({T_U32: "<I", T_I32: "<i", T_F32: "<f", T_U8: "<B"}[et], it)
    else:
        raise ValueError(vtype)
    return out


def write_gguf(path, kvs, tensors, alignment=32, version=3):
    """kvs: list of (key, vtype, value).  tensors: list of (name, ggml_type, dims(ne0, ne1, ...), uint8 ndarray)."""
    head = b"GGUF" + struct.pack("<IqQ", version, len(tensors), len(kvs))
    body = b"".join(kv_bytes(*kv) for kv in kvs)
    infos = b""
    off = 0
    offsets = []
    for name, ttype, dims, data in tensors:
        infos += _s(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        infos += struct.pack("<IQ", ttype, off)
        offsets.append(off)
        off += (data.nbytes + alignment - 1) // alignment * alignment
    pre = head + body + infos
    pad = (-len(pre)) % alignment
    with open(path, "wb") as f:
        f.write(pre + b"\0" * pad)
        for (name, ttype, dims, data), o in zip(tensors, offsets):
            b = np.ascontiguousarray(data).view(np.uint8).reshape(-1)
            f.write(memoryview(b))
            f.write(b"\0" * ((-b.nbytes) % alignment))
    return len(pre) + pad
