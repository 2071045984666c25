"""ctypes binding of the CPU oracle (oracle/kq_oracle.c) and, when built, of the
compiled reference (oracle/_ref/libbp_ref.so).

TEST INFRASTRUCTURE ONLY.  Imported by tests/, by the smoke check and by the
benchmark's cpu_baseline leg; never by the shipped package.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libkq_oracle.so")
REF_PATH = os.path.join(HERE, "_ref", "libbp_ref.so")

Q4_K = 12
Q6_K = 14
BLOCK_BYTES = {Q4_K: 144, Q6_K: 210}

_u32p = C.POINTER(C.c_uint32)
_i32p = C.POINTER(C.c_int32)
_f32p = C.POINTER(C.c_float)
_f64p = C.POINTER(C.c_double)
_u16p = C.POINTER(C.c_uint16)
_u8p = C.POINTER(C.c_uint8)


def build(ref: bool = True) -> None:
    """Compile the oracle (and the reference object where its sources exist)."""
    target = ["all"] if ref else ["libkq_oracle.so"]
    subprocess.run(["make", "-C", HERE, "-s"] + target, check=True)


def _load() -> C.CDLL:
    if not os.path.exists(LIB_PATH):
        build(ref=False)
    lib = C.CDLL(LIB_PATH)
    lib.kqo_fp16_to_f32.restype = C.c_float
    lib.kqo_fp16_to_f32.argtypes = [C.c_uint16]
    lib.kqo_fp16_to_f32_bits.restype = C.c_uint32
    lib.kqo_fp16_to_f32_bits.argtypes = [C.c_uint16]
    lib.kqo_q4k_scale_min.restype = None
    lib.kqo_q4k_scale_min.argtypes = [_u8p, C.c_int, _u32p, _u32p]
    lib.kqo_row_stride_words.restype = C.c_uint32
    lib.kqo_row_stride_words.argtypes = [C.c_int, C.c_uint32]
    lib.kqo_n_blocks.restype = C.c_uint32
    lib.kqo_n_blocks.argtypes = [C.c_uint32]
    lib.kqo_pack.argtypes = [C.c_int, C.c_void_p, C.c_uint32, C.c_uint32, _u32p]
    lib.kqo_dequant.argtypes = [C.c_int, C.c_void_p, _f32p, C.c_uint32, C.c_uint32]
    lib.kqo_dequant_rows.argtypes = [C.c_int, _u32p, C.c_uint32, _i32p, C.c_uint32,
                                     C.c_uint32, _f32p]
    lib.kqo_matmul.argtypes = [C.c_int, _f32p, _u32p, _f32p, _f32p, C.c_uint32,
                               C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32]
    lib.kqo_prologue.argtypes = [C.c_int, _f32p, _f32p, C.c_float, C.c_uint32, C.c_uint32, _f32p]
    lib.kqo_matmul_f64.argtypes = [C.c_int, _f32p, _u32p, _f32p, _f64p, C.c_uint32,
                                   C.c_uint32, C.c_uint32, C.c_uint32]
    lib.kqo_matmul_bf16.argtypes = [C.c_int, _u16p, _u32p, _f32p, _f32p, C.c_uint32,
                                    C.c_uint32, C.c_uint32, C.c_uint32]
    lib.kqo_matmul_timed.argtypes = [C.c_int, _f32p, C.c_void_p, _f32p, _f32p,
                                     C.c_uint32, C.c_uint32, C.c_uint32, _f64p, _f64p]
    lib.kqo_moe_topk_softmax.restype = None
    lib.kqo_moe_topk_softmax.argtypes = [_f32p, C.c_uint32, C.c_uint32, C.c_int, _u32p, _f32p]
    lib.kqo_moe_offsets.restype = None
    lib.kqo_moe_offsets.argtypes = [_u32p, C.c_uint32, C.c_uint32, _u32p]
    lib.kqo_moe_matmul.argtypes = [C.c_int, _f32p, _u32p, _u32p, _f32p, C.c_uint32,
                                   C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, C.c_int]
    lib.kqo_moe_ffn.argtypes = [C.c_int, C.c_int, _f32p, _u32p, _u32p, _u32p, _u32p,
                                _f32p, _f32p, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32]
    lib.kqo_rng_seed.restype = None
    lib.kqo_rng_seed.argtypes = [C.c_void_p, C.c_uint32]
    lib.kqo_rng_next.restype = C.c_uint32
    lib.kqo_rng_next.argtypes = [C.c_void_p]
    lib.kqo_rng_randn_vec.restype = None
    lib.kqo_rng_randn_vec.argtypes = [C.c_void_p, _f32p, C.c_int]
    lib.kqo_f32_to_f16_trunc.restype = C.c_uint16
    lib.kqo_f32_to_f16_trunc.argtypes = [C.c_float]
    lib.kqo_assert_close.argtypes = [_f32p, _f32p, C.c_int, C.c_float, C.c_float, _f32p]
    return lib


_lib = None
_ref = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        _lib = _load()
    return _lib


def ref():
    """The compiled reference, or None where it was not built."""
    global _ref
    if _ref is None and os.path.exists(REF_PATH):
        r = C.CDLL(REF_PATH)
        r.bpref_pack.argtypes = [C.c_int, C.c_void_p, C.c_uint32, C.c_uint32, _u32p, _u32p, _u32p]
        r.bpref_dequant.argtypes = [C.c_int, C.c_void_p, _f32p, C.c_uint32, C.c_uint32]
        r.bpref_matmul_timed.argtypes = [C.c_int, _f32p, C.c_void_p, _f32p, _f32p, C.c_uint32,
                                         C.c_uint32, C.c_uint32, _f64p, _f64p]
        _ref = r
    return _ref


def _p(a: np.ndarray, t):
    return a.ctypes.data_as(t)


def _c(a, dtype) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=dtype)


# --------------------------------------------------------------------------- #
def fp16_to_f32(h: int) -> float:
    return lib().kqo_fp16_to_f32(int(h) & 0xFFFF)


def fp16_to_f32_bits(h: int) -> int:
    """Bit pattern of the result (keeps signalling-NaN payloads intact)."""
    return lib().kqo_fp16_to_f32_bits(int(h) & 0xFFFF)


def q4k_scale_min(s12, sb: int):
    s = _c(s12, np.uint8)
    sc, mn = C.c_uint32(), C.c_uint32()
    lib().kqo_q4k_scale_min(_p(s, _u8p), sb, C.byref(sc), C.byref(mn))
    return sc.value, mn.value


def row_stride_words(type_: int, K: int) -> int:
    return lib().kqo_row_stride_words(type_, K)


def n_blocks(K: int) -> int:
    return lib().kqo_n_blocks(K)


def pack(type_: int, raw, N: int, K: int) -> np.ndarray:
    raw = _c(raw, np.uint8)
    rs = row_stride_words(type_, K)
    out = np.empty(N * rs, dtype=np.uint32)
    rc = lib().kqo_pack(type_, raw.ctypes.data, N, K, _p(out, _u32p))
    assert rc == 0
    return out


def dequant(type_: int, raw, N: int, K: int) -> np.ndarray:
    raw = _c(raw, np.uint8)
    out = np.empty((N, K), dtype=np.float32)
    rc = lib().kqo_dequant(type_, raw.ctypes.data, _p(out, _f32p), N, K)
    assert rc == 0
    return out


def dequant_rows(type_: int, packed, rows, K: int) -> np.ndarray:
    packed = _c(packed, np.uint32)
    rows = _c(rows, np.int32)
    out = np.empty((len(rows), K), dtype=np.float32)
    rc = lib().kqo_dequant_rows(type_, _p(packed, _u32p), row_stride_words(type_, K),
                                _p(rows, _i32p), len(rows), K, _p(out, _f32p))
    assert rc == 0
    return out


def matmul(type_: int, X, packed, N: int, K: int, bias=None, y_offset: int = 0,
           ldy: int = 0, Y=None) -> np.ndarray:
    X = _c(X, np.float32).reshape(-1, K)
    M = X.shape[0]
    packed = _c(packed, np.uint32)
    b = None if bias is None else _c(bias, np.float32)
    if Y is None:
        Y = np.zeros((M, ldy or N), dtype=np.float32)
    rc = lib().kqo_matmul(type_, _p(X, _f32p), _p(packed, _u32p),
                          None if b is None else _p(b, _f32p), _p(Y, _f32p), M, N, K,
                          row_stride_words(type_, K), y_offset, ldy)
    assert rc == 0
    return Y


def prologue(pro: int, X, K: int, norm_w=None, eps: float = 0.0) -> np.ndarray:
    """RMSNorm (1) / silu(gate)*up (2) / gelu_tanh(gate)*up (3) of the rows of X; gate | up rows are 2K wide."""
    X = _c(X, np.float32)
    M = X.size // (K if pro == 1 else 2 * K)
    out = np.empty((M, K), dtype=np.float32)
    w = _c(norm_w, np.float32) if norm_w is not None else np.zeros(1, np.float32)
    rc = lib().kqo_prologue(pro, _p(X, _f32p), _p(w, _f32p), eps, M, K, _p(out, _f32p))
    assert rc == 0
    return out


def matmul_f64(type_: int, X, packed, N: int, K: int, bias=None) -> np.ndarray:
    X = _c(X, np.float32).reshape(-1, K)
    M = X.shape[0]
    packed = _c(packed, np.uint32)
    b = None if bias is None else _c(bias, np.float32)
    Y = np.zeros((M, N), dtype=np.float64)
    rc = lib().kqo_matmul_f64(type_, _p(X, _f32p), _p(packed, _u32p),
                              None if b is None else _p(b, _f32p), _p(Y, _f64p), M, N, K,
                              row_stride_words(type_, K))
    assert rc == 0
    return Y


def matmul_bf16(type_: int, Xbits, packed, N: int, K: int, bias=None) -> np.ndarray:
    Xb = _c(Xbits, np.uint16).reshape(-1, K)
    M = Xb.shape[0]
    packed = _c(packed, np.uint32)
    b = None if bias is None else _c(bias, np.float32)
    Y = np.zeros((M, N), dtype=np.float32)
    rc = lib().kqo_matmul_bf16(type_, _p(Xb, _u16p), _p(packed, _u32p),
                               None if b is None else _p(b, _f32p), _p(Y, _f32p), M, N, K,
                               row_stride_words(type_, K))
    assert rc == 0
    return Y


def matmul_timed(type_: int, X, raw, N: int, K: int, use_ref: bool = False):
    """(Y, seconds_dequant, seconds_dot) of the dequantise-then-dot CPU path."""
    X = _c(X, np.float32).reshape(-1, K)
    M = X.shape[0]
    raw = _c(raw, np.uint8)
    deq = np.empty((N, K), dtype=np.float32)
    Y = np.empty((M, N), dtype=np.float32)
    td, tm = C.c_double(), C.c_double()
    fn = ref().bpref_matmul_timed if use_ref else lib().kqo_matmul_timed
    rc = fn(type_, _p(X, _f32p), raw.ctypes.data, _p(deq, _f32p), _p(Y, _f32p), M, N, K,
            C.byref(td), C.byref(tm))
    assert rc == 0
    return Y, td.value, tm.value


def moe_topk_softmax(logits, k: int, normalize: bool = True):
    lg = _c(logits, np.float32)
    idx = np.empty(k, dtype=np.uint32)
    wt = np.empty(k, dtype=np.float32)
    lib().kqo_moe_topk_softmax(_p(lg, _f32p), len(lg), k, int(normalize), _p(idx, _u32p),
                               _p(wt, _f32p))
    return idx, wt


def argmax_rows(logits) -> np.ndarray:
    """Greedy pick per row as the reference's argmax + argmax_reduce kernels compute it on a sequential
    scan (`v > best` from best = -1e30, index 0; argmax.wgsl, wired in runtime/model_runner.cpp:2441-2453):
    the first index holding the maximum, 0 when nothing exceeds -1e30.  Pinned by a python loop on small
    rows in tests/test_oracle_pins.py."""
    lg = np.asarray(logits, dtype=np.float32)
    masked = np.where(lg > np.float32(-1e30), lg, -np.inf)      # NaN compares false: never picked
    idx = np.argmax(masked, axis=1)
    none = ~np.any(lg > np.float32(-1e30), axis=1)
    return np.where(none, 0, idx).astype(np.int32)


def moe_offsets(idx, rows_per_expert: int) -> np.ndarray:
    idx = _c(idx, np.uint32)
    out = np.empty_like(idx)
    lib().kqo_moe_offsets(_p(idx, _u32p), len(idx), rows_per_expert, _p(out, _u32p))
    return out


def moe_matmul(type_: int, X, packed, expert_idx, N: int, K: int,
               x_per_slot: bool = False) -> np.ndarray:
    eidx = _c(expert_idx, np.uint32)
    T, k = eidx.shape
    X = _c(X, np.float32)
    packed = _c(packed, np.uint32)
    Y = np.zeros((T, k, N), dtype=np.float32)
    rc = lib().kqo_moe_matmul(type_, _p(X, _f32p), _p(packed, _u32p), _p(eidx, _u32p),
                              _p(Y, _f32p), T, k, N, K, row_stride_words(type_, K),
                              int(x_per_slot))
    assert rc == 0
    return Y


def moe_ffn(type_gu: int, type_dn: int, X, gate, up, down, expert_idx, expert_wt,
            hidden: int, inter: int) -> np.ndarray:
    eidx = _c(expert_idx, np.uint32)
    ew = _c(expert_wt, np.float32)
    T, k = eidx.shape
    X = _c(X, np.float32)
    gate, up, down = (_c(a, np.uint32) for a in (gate, up, down))
    out = np.zeros((T, hidden), dtype=np.float32)
    rc = lib().kqo_moe_ffn(type_gu, type_dn, _p(X, _f32p), _p(gate, _u32p), _p(up, _u32p),
                           _p(down, _u32p), _p(eidx, _u32p), _p(ew, _f32p), _p(out, _f32p),
                           T, k, hidden, inter)
    assert rc == 0
    return out


class Rng:
    """The reference kernel-test generator (kernel_test.cpp:62-99)."""

    def __init__(self, seed: int):
        self._s = (C.c_uint32 * 4)()
        lib().kqo_rng_seed(C.byref(self._s), seed)

    def next(self) -> int:
        return lib().kqo_rng_next(C.byref(self._s))

    def randn_vec(self, n: int) -> np.ndarray:
        out = np.empty(n, dtype=np.float32)
        lib().kqo_rng_randn_vec(C.byref(self._s), _p(out, _f32p), n)
        return out


def f32_to_f16_trunc(f: float) -> int:
    return lib().kqo_f32_to_f16_trunc(float(np.float32(f)))


def assert_close(actual, expected, atol: float, rtol: float):
    a = _c(actual, np.float32).ravel()
    e = _c(expected, np.float32).ravel()
    assert a.shape == e.shape
    worst = C.c_float()
    bad = lib().kqo_assert_close(_p(a, _f32p), _p(e, _f32p), a.size, atol, rtol, C.byref(worst))
    return bad, worst.value


# --------------------------------------------------------------------------- #
def ref_pack(type_: int, raw, N: int, K: int):
    r = ref()
    raw = _c(raw, np.uint8)
    nb, rs = C.c_uint32(), C.c_uint32()
    assert r.bpref_pack(type_, raw.ctypes.data, N, K, None, C.byref(nb), C.byref(rs)) == 0
    out = np.empty(N * rs.value, dtype=np.uint32)
    assert r.bpref_pack(type_, raw.ctypes.data, N, K, _p(out, _u32p), None, None) == 0
    return out, nb.value, rs.value


def ref_dequant(type_: int, raw, N: int, K: int) -> np.ndarray:
    raw = _c(raw, np.uint8)
    out = np.empty((N, K), dtype=np.float32)
    assert ref().bpref_dequant(type_, raw.ctypes.data, _p(out, _f32p), N, K) == 0
    return out
