"""Writes GGUF files for the container tests, straight from the published layout:
header (magic, version, tensor count, kv count), typed key-value pairs, tensor
table, padding to the alignment, tensor data each aligned the same way.  The
contents of a written file are therefore known by construction."""
import struct

import numpy as np

U8, I8, U16, I16, U32, I32, F32, BOOL, STRING, ARRAY, U64, I64, F64 = range(13)
_FMT = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<B", U64: "<Q", I64: "<q",
        F64: "<d"}


def _s(b) -> bytes:
    b = b.encode() if isinstance(b, str) else b
    return struct.pack("<Q", len(b)) + b


def _value(t, v) -> bytes:
    if t == STRING:
        return _s(v)
    if t == ARRAY:
        et, items = v
        out = struct.pack("<IQ", et, len(items))
        return out + b"".join(_value(et, x) for x in items)
    return struct.pack(_FMT[t], v)


def write(path, metadata, tensors, version=3, alignment=32, declare_alignment=False, tail=b""):
    """metadata: list of (key, type, value); an ARRAY value is (elem_type, items).
    tensors: list of (name, dims tuple in GGUF order, type code, data bytes).
    Returns {name: offset into the data section} and the data section's offset."""
    md = list(metadata)
    if declare_alignment:
        md.append(("general.alignment", U32, alignment))
    head = struct.pack("<IIQQ", 0x46554747, version, len(tensors), len(md))
    for k, t, v in md:
        head += _s(k) + struct.pack("<I", t) + _value(t, v)
    offsets, pos = {}, 0
    body = b""
    for name, dims, type_, data in tensors:
        data = bytes(np.asarray(data, dtype=np.uint8).tobytes()) if not isinstance(data, bytes) else data
        pad = (-pos) % alignment
        body += b"\0" * pad
        pos += pad
        offsets[name] = pos
        body += data
        pos += len(data)
    for name, dims, type_, data in tensors:
        head += _s(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        head += struct.pack("<IQ", type_, offsets[name])
    data_offset = (len(head) + alignment - 1) // alignment * alignment
    blob = head + b"\0" * (data_offset - len(head)) + body + tail
    with open(path, "wb") as f:
        f.write(blob)
    return offsets, data_offset
