"""GGUF container reader over the C ABI (bpk_gguf_*), torch-free.

Mirrors the reference's GGUFFile (runtime/gguf_loader.h:49-86): `version`,
`n_tensors`, `data_offset`, `tensors`, `tensor_index` lookups and the typed
metadata getters with defaults.  Tensor data is exposed as numpy views into the
library's read-only mapping; they are valid until `close()`.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass

import numpy as np

from . import capi

_ELEM_DTYPES = {0: np.uint8, 1: np.int8, 2: np.uint16, 3: np.int16, 4: np.uint32, 5: np.int32, 6: np.float32,
                7: np.uint8, 10: np.uint64, 11: np.int64, 12: np.float64}


@dataclass
class TensorInfo:
    name: str
    type: int
    shape: tuple      # GGUF order: shape[0] is the row length K
    offset: int       # from the start of the data section
    nbytes: int
    address: int      # host address inside the mapping


class GGUFFile:
    def __init__(self, path: str):
        self._h = C.c_void_p()
        capi.check(capi.lib().bpk_gguf_open(str(path).encode(), C.byref(self._h)))
        v, nt, nkv, off = C.c_uint32(), C.c_uint64(), C.c_uint64(), C.c_uint64()
        capi.check(capi.lib().bpk_gguf_info(self._h, C.byref(v), C.byref(nt), C.byref(nkv), C.byref(off)))
        self.version, self.n_tensors, self.n_kv, self.data_offset = v.value, nt.value, nkv.value, off.value

    # -- lifetime ---------------------------------------------------------
    def close(self) -> None:
        if self._h:
            capi.lib().bpk_gguf_close(self._h)
            self._h = C.c_void_p()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def handle(self) -> C.c_void_p:
        if not self._h:
            raise ValueError("GGUF file is closed")
        return self._h

    # -- tensors ----------------------------------------------------------
    @staticmethod
    def _info(t: capi.GgufTensor) -> TensorInfo:
        return TensorInfo(t.name.decode(), t.type, tuple(t.dims[d] for d in range(t.n_dims)), t.offset, t.bytes,
                          t.data or 0)

    def tensor_at(self, i: int) -> TensorInfo:
        t = capi.GgufTensor()
        capi.check(capi.lib().bpk_gguf_tensor_at(self.handle, i, C.byref(t)))
        return self._info(t)

    @property
    def tensors(self) -> list[TensorInfo]:
        return [self.tensor_at(i) for i in range(self.n_tensors)]

    def tensor(self, name: str) -> TensorInfo:
        t = capi.GgufTensor()
        capi.check(capi.lib().bpk_gguf_find_tensor(self.handle, name.encode(), C.byref(t)))
        return self._info(t)

    def tensor_bytes(self, name: str) -> np.ndarray:
        """uint8 view of the tensor's data inside the mapping (no copy)."""
        t = self.tensor(name)
        if t.nbytes == 0:
            return np.empty(0, dtype=np.uint8)
        return np.ctypeslib.as_array((C.c_uint8 * t.nbytes).from_address(t.address))

    # -- metadata ---------------------------------------------------------
    def has_key(self, key: str) -> bool:
        return bool(capi.lib().bpk_gguf_has_key(self.handle, key.encode()))

    def get_u32(self, key: str, default: int = 0) -> int:
        v = C.c_uint32()
        capi.check(capi.lib().bpk_gguf_get_u32(self.handle, key.encode(), default, C.byref(v)))
        return v.value

    def get_float(self, key: str, default: float = 0.0) -> float:
        v = C.c_float()
        capi.check(capi.lib().bpk_gguf_get_f32(self.handle, key.encode(), default, C.byref(v)))
        return v.value

    def get_bool(self, key: str, default: bool = False) -> bool:
        v = C.c_int()
        capi.check(capi.lib().bpk_gguf_get_bool(self.handle, key.encode(), int(default), C.byref(v)))
        return bool(v.value)

    def key_type(self, key: str) -> int:
        """GGUF metadata type code of the key, -1 when absent."""
        return capi.lib().bpk_gguf_key_type(self.handle, key.encode())

    def get_string(self, key: str, default: str = "") -> str:
        if self.key_type(key) != 8:
            return default
        n = C.c_size_t()
        capi.check(capi.lib().bpk_gguf_get_string(self.handle, key.encode(), None, 0, C.byref(n)))
        buf = C.create_string_buffer(n.value + 1)
        capi.check(capi.lib().bpk_gguf_get_string(self.handle, key.encode(), buf, n.value + 1, None))
        return buf.raw[: n.value].decode("utf-8", errors="replace")

    def array_len(self, key: str) -> tuple[int, int]:
        n, et = C.c_uint64(), C.c_uint32()
        capi.check(capi.lib().bpk_gguf_array_len(self.handle, key.encode(), C.byref(n), C.byref(et)))
        return n.value, et.value

    def get_string_array(self, key: str) -> list[str]:
        n, et = self.array_len(key)
        if et != 8:
            return []
        out = []
        L = capi.lib()
        for i in range(n):
            ln = C.c_size_t()
            capi.check(L.bpk_gguf_array_string(self.handle, key.encode(), i, None, 0, C.byref(ln)))
            buf = C.create_string_buffer(ln.value + 1)
            capi.check(L.bpk_gguf_array_string(self.handle, key.encode(), i, buf, ln.value + 1, None))
            out.append(buf.raw[: ln.value].decode("utf-8", errors="replace"))
        return out

    def model_config(self) -> dict:
        """The model's hyper-parameters (extractModelConfig, runtime/gguf_loader.cpp:184-317) as a dict;
        'layer_attn_types' lists 0 (global) / 1 (sliding window) per layer, empty without a sliding window."""
        c = capi.ModelConfig()
        L = capi.lib()
        capi.check(L.bpk_gguf_model_config(self.handle, C.byref(c), None, 0))
        types = (C.c_uint8 * max(1, c.n_layer_attn_types))()
        if c.n_layer_attn_types:
            capi.check(L.bpk_gguf_model_config(self.handle, C.byref(c), types, c.n_layer_attn_types))
        out = {}
        for name, _ in capi.ModelConfig._fields_:
            v = getattr(c, name)
            out[name] = v.decode() if name == "arch" else list(v) if name == "rope_sections" else v
        out["layer_attn_types"] = list(types)[: c.n_layer_attn_types]
        return out

    def get_array(self, key: str) -> np.ndarray:
        """Fixed-size-element array as a numpy copy (empty when absent or an array of strings)."""
        p, n, et = C.c_void_p(), C.c_uint64(), C.c_uint32()
        capi.check(capi.lib().bpk_gguf_array_data(self.handle, key.encode(), C.byref(p), C.byref(n), C.byref(et)))
        if not p.value or n.value == 0:
            return np.empty(0, dtype=_ELEM_DTYPES.get(et.value, np.uint8))
        dt = np.dtype(_ELEM_DTYPES[et.value])
        raw = np.ctypeslib.as_array((C.c_uint8 * (n.value * dt.itemsize)).from_address(p.value))
        return raw.copy().view(dt)
