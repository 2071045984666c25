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
