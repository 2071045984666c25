"""CPU-side checks of the C ABI: the shared library loads, exports every symbol
the public header declares, and its host-only entry points (layout, packer,
argument validation) agree with the oracle.  No kernel is launched."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from backpack_amd import capi, synth

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
Q4_K, Q6_K = 12, 14


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "bpk_kquant.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"BPK_API[^;(]*?\b(bpk_\w+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound():
    names = declared_symbols()
    assert len(names) >= 15
    lib = C.CDLL(capi.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), f"{n} declared in the header but not exported"
    assert set(names) == set(capi.exported_names()), "ctypes binding out of step with the header"


@pytest.mark.parametrize("type_", [Q4_K, Q6_K])
@pytest.mark.parametrize("K", [256, 768, 2048, 4096, 14336])
def test_layout_matches_oracle(kqo, type_, K):
    assert capi.layout(type_, K) == (kqo.n_blocks(K), kqo.row_stride_words(type_, K))


def test_layout_rejects_unknown_type():
    with pytest.raises(capi.BpkError) as e:
        capi.layout(11, 256)   # Q3_K is outside this library
    assert e.value.code == -1
    assert capi.layout(13, 512) == (2, 88)   # Q5_K: 44 words per block


@pytest.mark.parametrize("type_,N,K", [(Q4_K, 5, 512), (Q6_K, 7, 768), (Q6_K, 3, 256), (13, 4, 768)])
def test_pack_host_matches_oracle(kqo, type_, N, K):
    from backpack_amd import kquant  # imports torch; no GPU needed for the packer
    raw = synth.make_raw(type_, N, K, seed=3)
    assert np.array_equal(kquant.pack_host(type_, raw, N, K), kqo.pack(type_, raw, N, K))


def test_matmul_argument_validation_needs_no_gpu():
    L = capi.lib()
    one = C.c_void_p(16)
    # K not a multiple of 256
    assert L.bpk_kq_matmul(Q4_K, one, one, None, one, 1, 8, 100, 1, 36, 0, None) == -2
    assert b"256" in L.bpk_last_error()
    # unknown type
    assert L.bpk_kq_matmul(2, one, one, None, one, 1, 8, 256, 1, 36, 0, None) == -1
    # null X
    assert L.bpk_kq_matmul(Q4_K, None, one, None, one, 1, 8, 256, 1, 36, 0, None) == -3
    # row stride smaller than a row
    assert L.bpk_kq_matmul(Q6_K, one, one, None, one, 1, 8, 768, 3, 100, 0, None) == -2
    # misaligned W
    assert L.bpk_kq_matmul(Q4_K, one, C.c_void_p(18), None, one, 1, 8, 256, 1, 36, 0, None) == -4
    # n_blocks inconsistent with K
    assert L.bpk_kq_matmul(Q4_K, one, one, None, one, 1, 8, 512, 1, 72, 0, None) == -2


# ---- which form of the bf16 dequant-GEMM serves a shape: host arithmetic, pinned on the shapes it was priced on ----
SMALL, WHOLE, SHARES, HALF, ROUNDS_THEN_HALF, N192 = range(6)


@pytest.mark.parametrize("name,type_,N,K,M,want", [
    # the Llama-3-8B matrices at 2048 tokens on 256 CUs
    ("gate_up", Q4_K, 28672, 4096, 2048, ROUNDS_THEN_HALF),   # 896 tiles = 3.5 rounds: 3 rounds, then 4096 rows as 256 x 128 tiles
    ("qkv", Q4_K, 6144, 4096, 2048, N192),                     # 256 tiles of 256 x 192: one per CU
    ("qkv", Q4_K, 6144, 4096, 1024, HALF),                     # 128 such tiles would leave half the CUs idle
    ("o", Q4_K, 4096, 4096, 2048, HALF),                       # 256 tiles of 256 x 128: one per CU
    ("down", Q6_K, 4096, 14336, 2048, SHARES),                 # 128 tiles of long K: every tile cut in two
    ("lm_head", Q6_K, 128256, 4096, 2048, WHOLE),              # 4008 tiles; the last round is more than half full
    # ... and at 512 tokens
    ("gate_up", Q4_K, 28672, 4096, 512, WHOLE),
    ("down", Q6_K, 4096, 14336, 512, SHARES),
    ("o", Q4_K, 4096, 4096, 512, SHARES),
    # one small tile's worth of work
    ("tiny", Q4_K, 128, 256, 128, SMALL),
])
def test_gemm_plan_on_the_shapes_it_was_priced_on(name, type_, N, K, M, want):
    form, share, first = capi.gemm_plan(type_, M, N, K, 256)
    assert form == want, (name, form, share, first)
    nk = K // 64
    if form == ROUNDS_THEN_HALF:
        # the first launch is whole rounds of whole tiles, the second at most one round of half tiles
        m_tiles = -(-M // 256)
        assert share == nk and first % 256 == 0 and 0 < first < N
        assert (m_tiles * (first // 256)) % 256 == 0
        assert m_tiles * -(-(N - first) // 128) <= 256
    if form == WHOLE:
        assert share == nk
    if form == SHARES:
        assert share % 4 == 0 and share != nk


def test_gemm_plan_follows_the_options_and_refuses_bad_arguments():
    try:
        capi.set_option("gemm_tile", 128)
        assert capi.gemm_plan(Q4_K, 2048, 28672, 4096)[0] == SMALL
        capi.set_option("gemm_tile", 129)
        assert capi.gemm_plan(Q4_K, 2048, 28672, 4096)[0] == HALF
        capi.set_option("gemm_tile", 192)
        assert capi.gemm_plan(Q6_K, 2048, 4096, 14336)[0] == N192
        capi.set_option("gemm_tile", 256)
        capi.set_option("gemm_split", 1)
        assert capi.gemm_plan(Q6_K, 2048, 4096, 14336)[:2] == (WHOLE, 14336 // 64)
        capi.set_option("gemm_split", 2)
        form, share, _ = capi.gemm_plan(Q4_K, 2048, 28672, 4096)
        assert form == SHARES and share == 224    # 896 tiles x 64 steps over 256 CUs
    finally:
        capi.set_option("gemm_tile", 0)
        capi.set_option("gemm_split", 0)
    with pytest.raises(capi.BpkError):
        capi.gemm_plan(Q4_K, 2048, 4096, 100)     # K not a multiple of 256
    with pytest.raises(capi.BpkError):
        capi.gemm_plan(11, 2048, 4096, 4096)      # unknown type
    # a part with fewer CUs: o no longer fits one round of half tiles and the answer changes with the count
    assert capi.gemm_plan(Q4_K, 2048, 4096, 4096, 128)[0] in (WHOLE, SHARES, HALF, SMALL)


def test_options_take_their_values_and_refuse_others():
    """bpk_set_option is host state: it can be checked without a device."""
    for name, good, bad in [("moe_tile_iters", (0, 1, 2, 4, 8), (3, 16, -1)), ("gemm_tile", (0, 128, 129, 192, 256), (64, 130)),
                            ("gemm_split", (0, 1, 2), (3,))]:
        try:
            for v in good:
                capi.set_option(name, v)
            for v in bad:
                with pytest.raises(capi.BpkError):
                    capi.set_option(name, v)
        finally:
            capi.set_option(name, 0)
    with pytest.raises(capi.BpkError):
        capi.set_option("no_such_option", 1)
