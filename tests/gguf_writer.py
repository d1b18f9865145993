"""A minimal GGUF writer for the tests (the public container format, versions 2 / 3): header, typed key-value pairs
(scalars, strings, arrays, nested arrays), tensor table, aligned data section. Test infrastructure only."""
import struct

import numpy as np

U8, I8, U16, I16, U32, I32, F32, BOOL, STR, ARR, U64, I64, F64 = range(13)
_FMT = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<B", U64: "<Q", I64: "<q", F64: "<d"}


def _s(x):
    b = x.encode()
    return struct.pack("<Q", len(b)) + b


def _val(t, v):
    if t == STR:
        return _s(v)
    if t == ARR:
        et, items = v
        return struct.pack("<IQ", et, len(items)) + b"".join(_val(et, i) for i in items)
    return struct.pack(_FMT[t], v)


def write_gguf(path, kvs, tensors, alignment=32, version=3, write_alignment_key=None):
    """kvs: list of (key, type, value) -- an array value is (element type, items); tensors: list of
    (name, ggml type, ne (ggml order), bytes as numpy uint8). Returns {name: absolute data offset}."""
    kvs = list(kvs)
    if write_alignment_key if write_alignment_key is not None else alignment != 32:
        kvs.append(("general.alignment", U32, alignment))
    head = struct.pack("<IIQQ", 0x46554747, version, len(tensors), len(kvs))
    for k, t, v in kvs:
        head += _s(k) + struct.pack("<I", t) + _val(t, v)
    offs, rel = {}, 0
    table = b""
    for name, gt, ne, data in tensors:
        rel = (rel + alignment - 1) // alignment * alignment
        table += _s(name) + struct.pack("<I", len(ne)) + b"".join(struct.pack("<Q", d) for d in ne) + struct.pack("<IQ", gt, rel)
        offs[name] = rel
        rel += len(data)
    data_off = (len(head) + len(table) + alignment - 1) // alignment * alignment
    with open(path, "wb") as f:
        f.write(head + table)
        f.write(b"\0" * (data_off - len(head) - len(table)))
        pos = 0
        for name, gt, ne, data in tensors:
            f.write(b"\0" * (offs[name] - pos))
            f.write(np.ascontiguousarray(data, dtype=np.uint8).tobytes())
            pos = offs[name] + len(data)
    return {n: o + data_off for n, o in offs.items()}, data_off
