"""CPU restatement of the reference's GGUF container parser.

TEST INFRASTRUCTURE ONLY: imported by tests/ (and nothing on the product path).
Follows GGUFFile::open and its accessors, runtime/gguf_loader.cpp:20-182, field
by field, including which array kinds are kept (string, int32/uint32, float32,
bool) and which are walked and dropped.

Pinned by tests/test_gguf.py against (a) files whose contents are known by
construction (written to the published GGUF layout by an independent writer)
and (b) the reference's own parser compiled into oracle/_ref, where it builds.
"""
from __future__ import annotations

import struct

# metadata value type codes (GGUFMetaType, runtime/gguf_loader.cpp:8-13)
U8, I8, U16, I16, U32, I32, F32, BOOL, STRING, ARRAY, U64, I64, F64 = range(13)
_SCALAR = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", U64: "<Q", I64: "<q",
           F64: "<d"}


class Parsed:
    def __init__(self):
        self.version = 0
        self.n_tensors = 0
        self.data_offset = 0
        self.metadata = {}    # key -> (kind, value); kind in {"u8".."f64","bool","str","strs","i32s","f32s","bools","skipped"}
        self.tensors = []     # (name, shape tuple, type, offset)
        self.tensor_index = {}


_KIND = {U8: "u8", I8: "i8", U16: "u16", I16: "i16", U32: "u32", I32: "i32", F32: "f32", U64: "u64", I64: "i64",
         F64: "f64"}


class _Reader:
    def __init__(self, b: bytes):
        self.b, self.p = b, 0

    def take(self, fmt):
        n = struct.calcsize(fmt)
        v = struct.unpack_from(fmt, self.b, self.p)[0]
        self.p += n
        return v

    def string(self):   # read_string, gguf_loader.cpp:20-25
        n = self.take("<Q")
        s = self.b[self.p:self.p + n]
        self.p += n
        return s

    def value(self, t):   # read_meta_value, gguf_loader.cpp:28-87
        if t in _SCALAR:
            return _KIND[t], self.take(_SCALAR[t])
        if t == BOOL:
            return "bool", self.take("<B") != 0
        if t == STRING:
            return "str", self.string()
        if t == ARRAY:
            et = self.take("<I")
            n = self.take("<Q")
            if et == STRING:
                return "strs", [self.string() for _ in range(n)]
            if et in (I32, U32):
                return "i32s", [self.take("<i") for _ in range(n)]
            if et == F32:
                return "f32s", [self.take("<f") for _ in range(n)]
            if et == BOOL:
                return "bools", [self.take("<B") != 0 for _ in range(n)]
            for _ in range(n):
                self.value(et)
            return "skipped", b""
        raise ValueError(f"unknown metadata type {t}")


def parse(data: bytes) -> Parsed:
    """GGUFFile::open, gguf_loader.cpp:90-128."""
    r = _Reader(data)
    if r.take("<I") != 0x46554747:
        raise ValueError("bad magic")
    g = Parsed()
    g.version = r.take("<I")
    g.n_tensors = r.take("<Q")
    n_kv = r.take("<Q")
    for _ in range(n_kv):
        key = r.string()
        t = r.take("<I")
        g.metadata[key] = r.value(t)
    for i in range(g.n_tensors):
        name = r.string()
        nd = r.take("<I")
        shape = tuple(r.take("<Q") for _ in range(nd))
        type_ = r.take("<I")
        off = r.take("<Q")
        g.tensors.append((name, shape, type_, off))
        g.tensor_index[name] = i
    g.data_offset = (r.p + 31) & ~31
    return g


def get_u32(g: Parsed, key: bytes, default: int = 0) -> int:
    """GGUFFile::getU32, gguf_loader.cpp:141-162 (any integer width; the largest element of an int array)."""
    if key not in g.metadata:
        return default
    kind, v = g.metadata[key]
    if kind in ("u8", "i8", "u16", "i16", "u32", "i32", "u64", "i64"):
        return v & 0xFFFFFFFF
    if kind == "i32s":
        return (max(v) & 0xFFFFFFFF) if v else default
    return default


def get_float(g: Parsed, key: bytes, default: float = 0.0) -> float:
    """GGUFFile::getFloat, gguf_loader.cpp:164-170."""
    kind, v = g.metadata.get(key, (None, None))
    if kind == "f32":
        return v
    if kind == "f64":
        return struct.unpack("<f", struct.pack("<f", v))[0]
    return default


def get_bool(g: Parsed, key: bytes, default: bool = False) -> bool:
    """GGUFFile::getBool, gguf_loader.cpp:172-177."""
    kind, v = g.metadata.get(key, (None, None))
    return v if kind == "bool" else default


def get_string(g: Parsed, key: bytes, default: bytes = b"") -> bytes:
    """GGUFFile::getString, gguf_loader.cpp:132-139.  An array the parser dropped reads as the empty
    string there (its placeholder); callers of this restatement see the same."""
    kind, v = g.metadata.get(key, (None, None))
    return v if kind in ("str", "skipped") else default
