"""A minimal GGUF v3 writer for the tests (test infrastructure): metadata
key/values of every value type and raw tensor payloads at aligned offsets."""
import struct

import numpy as np

U8, I8, U16, I16, U32, I32, F32, BOOL, STRING, ARRAY, U64, I64, F64 = range(13)
_FMT = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<B",
        U64: "<Q", I64: "<q", F64: "<d"}


def _string(s):
    b = s if isinstance(s, bytes) else s.encode()
    return struct.pack("<Q", len(b)) + b


def _value(vtype, v):
    if vtype == STRING:
        return _string(v)
    if vtype == ARRAY:
        etype, items = v
        return struct.pack("<IQ", etype, len(items)) + b"".join(_value(etype, i) for i in items)
    return struct.pack(_FMT[vtype], v)


def build(metadata, tensors, version=3, alignment=None, pad_to=None):
    """metadata: [(key, value type, value)]; tensors: [(name, dims innermost
    first, on-disk type id, payload bytes)].  Returns the file's bytes."""
    if alignment is not None:
        metadata = list(metadata) + [("general.alignment", U32, alignment)]
    align = alignment or 32
    head = struct.pack("<IIQQ", 0x46554747, version, len(tensors), len(metadata))
    for key, vtype, v in metadata:
        head += _string(key) + struct.pack("<I", vtype) + _value(vtype, v)
    offsets, off = [], 0
    for _, _, _, payload in tensors:
        offsets.append(off)
        off += (len(payload) + align - 1) // align * align
    for (name, dims, type_id, _), o in zip(tensors, offsets):
        head += _string(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        head += struct.pack("<IQ", type_id, o)
    head += b"\0" * (-len(head) % align)
    body = b""
    for (_, _, _, payload), o in zip(tensors, offsets):
        body += b"\0" * (o - len(body)) + bytes(payload)
    out = head + body
    if pad_to:
        out += b"\0" * max(0, pad_to - len(out))
    return out


def as_bytes(a):
    return np.ascontiguousarray(a).tobytes()
