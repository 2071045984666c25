"""The reference's eleven Q4_K / Q5_K / Q6_K known-answer recipes, regenerated from
their closed forms (runtime/tests/kernel_test.cpp:1669-1748).  Inputs only: expected
values come from the oracle or from the golden fixture, never from here."""
from __future__ import annotations

import numpy as np

Q4_K, Q5_K, Q6_K = 12, 13, 14


def _h(kqo, f):
    # the test-suite's truncating fp32->fp16; the argument is evaluated in fp32
    return kqo.f32_to_f16_trunc(np.float32(f))


def _f(*terms):
    """Left-to-right fp32 sum of fp32 products, as the C expressions evaluate."""
    acc = np.float32(terms[0])
    for t in terms[1:]:
        acc = np.float32(acc + np.float32(t))
    return acc


def _mul(a, b):
    return np.float32(np.float32(a) * np.float32(b))


def _q4k(kqo, N, NB, dfun, dmfun, bfun):
    raw = np.zeros((N, NB, 144), dtype=np.uint8)
    for n in range(N):
        for b in range(NB):
            raw[n, b, 0:2] = np.frombuffer(np.uint16(_h(kqo, dfun(n, b))).tobytes(), np.uint8)
            raw[n, b, 2:4] = np.frombuffer(np.uint16(_h(kqo, dmfun(n, b))).tobytes(), np.uint8)
            i = np.arange(4, 144)
            raw[n, b, 4:] = (bfun(n, b, i) & 255).astype(np.uint8)
    return raw.reshape(N, -1)


def _q5k(kqo, N, NB, dfun, dmfun, bfun):
    raw = np.zeros((N, NB, 176), dtype=np.uint8)
    for n in range(N):
        for b in range(NB):
            raw[n, b, 0:2] = np.frombuffer(np.uint16(_h(kqo, dfun(n, b))).tobytes(), np.uint8)
            raw[n, b, 2:4] = np.frombuffer(np.uint16(_h(kqo, dmfun(n, b))).tobytes(), np.uint8)
            i = np.arange(4, 176)
            raw[n, b, 4:] = (bfun(n, b, i) & 255).astype(np.uint8)
    return raw.reshape(N, -1)


def _q6k(kqo, N, NB, dfun, bfun):
    raw = np.zeros((N, NB, 210), dtype=np.uint8)
    for n in range(N):
        for b in range(NB):
            i = np.arange(0, 208)
            raw[n, b, :208] = (bfun(n, b, i) & 255).astype(np.uint8)
            raw[n, b, 208:210] = np.frombuffer(np.uint16(_h(kqo, dfun(n, b))).tobytes(), np.uint8)
    return raw.reshape(N, -1)


def _bias(N, on):
    if not on:
        return np.zeros(N, dtype=np.float32)
    return np.array([_mul(0.01, n) for n in range(N)], dtype=np.float32)


def build(kqo):
    """name -> dict(type, M, N, K, raw, x | rows, bias, bias_first, atol, rtol, ref)."""
    R = {}

    def d1(n, b): return _f(0.02, _mul(0.001, n))
    def d2(n, b): return _f(0.02, _mul(0.001, n))

    # q4k_matmul_reference :1678
    R["q4k_matmul"] = dict(
        type=Q4_K, M=1, N=8, K=256, seed=4343, bias_on=False,
        raw=_q4k(kqo, 8, 1, d1, lambda n, b: _f(0.01, _mul(0.0005, n)),
                 lambda n, b, i: n * 31 + i * 17 + 3), ref="kernel_test.cpp:1678")
    # q4k_matmul_128_reference :1687
    q4b = lambda n, b, i: n * 31 + b * 13 + i * 17
    dm2 = lambda n, b: _f(0.01, _mul(0.0002, b))
    R["q4k_matmul_128"] = dict(type=Q4_K, M=1, N=7, K=512, seed=5555, bias_on=True,
                               raw=_q4k(kqo, 7, 2, d2, dm2, q4b), ref="kernel_test.cpp:1687")
    # q6k_matmul_reference :1691
    R["q6k_matmul"] = dict(
        type=Q6_K, M=1, N=8, K=768, seed=4646, bias_on=False,
        raw=_q6k(kqo, 8, 3, lambda n, q: _f(0.02, _mul(0.001, n), _mul(0.0003, q)),
                 lambda n, q, i: n * 29 + q * 23 + i * 19 + 5), ref="kernel_test.cpp:1691")
    # q6k_gather_reference :1700
    R["q6k_gather"] = dict(
        type=Q6_K, M=1, N=3, K=768, rows=[2],
        raw=_q6k(kqo, 3, 3, lambda n, b: _f(0.015, _mul(0.001, n), _mul(0.0002, b)),
                 lambda n, b, i: n * 41 + b * 23 + i * 11 + 9), ref="kernel_test.cpp:1700")
    # q6k_matmul_wide_reference :1709
    dw = lambda n, b: _f(0.018, _mul(0.0007, n), _mul(0.0002, b))
    R["q6k_matmul_wide"] = dict(
        type=Q6_K, M=1, N=19, K=768, seed=4747, bias_on=True,
        raw=_q6k(kqo, 19, 3, dw, lambda n, b, i: n * 37 + b * 17 + i * 13 + 11),
        ref="kernel_test.cpp:1709")
    # q6k_gather_batched_reference :1718
    R["q6k_gather_batched"] = dict(
        type=Q6_K, M=3, N=4, K=768, rows=[3, 0, 2],
        raw=_q6k(kqo, 4, 3, lambda n, b: _f(0.014, _mul(0.001, n)),
                 lambda n, b, i: n * 43 + b * 19 + i * 7 + 3), ref="kernel_test.cpp:1718")
    # q4k_matmul_batched4_reference :1726
    R["q4k_matmul_batched4"] = dict(type=Q4_K, M=5, N=9, K=512, seed=4848, bias_on=True,
                                    raw=_q4k(kqo, 9, 2, d2, dm2, q4b), ref="kernel_test.cpp:1726")
    # q6k_matmul_batched4_reference :1738
    R["q6k_matmul_batched4"] = dict(
        type=Q6_K, M=5, N=9, K=768, seed=5050, bias_on=True,
        raw=_q6k(kqo, 9, 3, dw, lambda n, b, i: n * 23 + b * 17 + i * 13),
        ref="kernel_test.cpp:1738")
    # q4k_matmul_batched8_reference :1744
    R["q4k_matmul_batched8"] = dict(type=Q4_K, M=9, N=9, K=512, seed=5151, bias_on=True,
                                    raw=_q4k(kqo, 9, 2, d2, dm2, q4b), ref="kernel_test.cpp:1744")

    # q5k_matmul_reference :1669
    R["q5k_matmul"] = dict(
        type=Q5_K, M=1, N=8, K=256, seed=4242, bias_on=False,
        raw=_q5k(kqo, 8, 1, d1, lambda n, b: _f(0.01, _mul(0.0005, n)),
                 lambda n, b, i: n * 37 + i * 13 + 7), ref="kernel_test.cpp:1669")
    # q5k_matmul_batched4_reference :1732
    R["q5k_matmul_batched4"] = dict(
        type=Q5_K, M=5, N=9, K=512, seed=4949, bias_on=True,
        raw=_q5k(kqo, 9, 2, d2, dm2, lambda n, b, i: n * 29 + b * 11 + i * 19), ref="kernel_test.cpp:1732")

    for name, r in R.items():
        if "seed" in r:
            r["x"] = kqo.Rng(r["seed"]).randn_vec(r["M"] * r["K"]).reshape(r["M"], r["K"])
            r["bias"] = _bias(r["N"], r["bias_on"])
            r["atol"], r["rtol"] = 2e-4, 2e-4
        else:
            r["atol"], r["rtol"] = 1e-6, 1e-6
    return R
