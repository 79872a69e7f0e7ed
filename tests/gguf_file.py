"""A minimal GGUF writer for the tests (version 3, little-endian): key-values of a few scalar types, strings and
arrays, and tensors laid out at the file's alignment, as the format's specification orders them. It writes what the
reader under test must accept; the refusal tests damage its output."""
import struct

import numpy as np

U8, I8, U16, I16, U32, I32, F32, BOOL, STR, ARR, U64, I64, F64 = range(13)
_FMT = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<B", U64: "<Q", I64: "<q", F64: "<d"}


def _string(s):
    b = s.encode()
    return struct.pack("<Q", len(b)) + b


def _value(vtype, v):
    if vtype == STR:
        return _string(v)
    if vtype == ARR:
        etype, items = v
        return struct.pack("<IQ", etype, len(items)) + b"".join(_value(etype, x) for x in items)
    return struct.pack(_FMT[vtype], v)


def write(path, kvs, tensors, alignment=32, version=3):
    """kvs: [(key, type, value)], tensors: [(name, dims (ne0 first), ggml type id, bytes)]. Returns each tensor's
    offset from the data section."""
    head = struct.pack("<IIQQ", 0x46554747, version, len(tensors), len(kvs))
    for key, vtype, v in kvs:
        head += _string(key) + struct.pack("<I", vtype) + _value(vtype, v)
    offsets, at = [], 0
    for _, _, _, data in tensors:
        offsets.append(at)
        at += (len(data) + alignment - 1) // alignment * alignment
    for (name, dims, ttype, _), off in zip(tensors, offsets):
        head += _string(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        head += struct.pack("<IQ", ttype, off)
    pad = (-len(head)) % alignment
    with open(path, "wb") as f:
        f.write(head + b"\0" * pad)
        for (_, _, _, data), off in zip(tensors, offsets):
            b = np.ascontiguousarray(data, np.uint8).tobytes()
            f.write(b + b"\0" * ((-len(b)) % alignment))
    return offsets
