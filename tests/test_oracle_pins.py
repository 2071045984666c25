"""Pins for the CPU oracle: each check is independent of the oracle's own code
(closed forms in float64, bit-level definitions, brute force, the compiled
reference, the committed golden fixtures)."""
import os

import numpy as np
import pytest

from backpack_amd import synth

GOLD = os.path.join(os.path.dirname(__file__), "golden")
Q4_K, Q5_K, Q6_K = 12, 13, 14


# ---- fp16 -> fp32 ----------------------------------------------------------
def test_fp16_exhaustive_closed_form(kqo):
    for h in range(65536):
        s = -1.0 if h & 0x8000 else 1.0
        e = (h >> 10) & 31
        m = h & 1023
        got = np.float32(kqo.fp16_to_f32(h))
        if e == 31:
            bits = ((h & 0x8000) << 16) | 0x7F800000 | (m << 13)
            assert kqo.fp16_to_f32_bits(h) == bits
        elif e == 0:
            want = np.float32(s * m * 2.0 ** -24)
            assert got == want and np.signbit(got) == (s < 0)
        else:
            assert got == np.float32(s * 2.0 ** (e - 25) * (1024 + m))


def test_fp16_matches_numpy_half(kqo):
    h = np.arange(65536, dtype=np.uint16)
    want = h.view(np.float16).astype(np.float32)
    got = np.array([kqo.fp16_to_f32(int(v)) for v in h], dtype=np.float32)
    finite = np.isfinite(want)
    assert np.array_equal(got[finite].view(np.uint32), want[finite].view(np.uint32))
    assert np.array_equal(np.isnan(got), np.isnan(want))


# ---- 6-bit scale / min -----------------------------------------------------
def test_q4k_scale_min_bit_definition(kqo):
    """ggml's get_scale_min_k4 written out bit by bit, over every value of the
    three bytes that feed one (scale, min) pair."""
    rng = np.random.default_rng(1)
    for sb in range(8):
        for _ in range(4000):
            s = rng.integers(0, 256, size=12, dtype=np.uint8)
            sc, mn = kqo.q4k_scale_min(s, sb)
            bits = [(int(s[i]) >> b) & 1 for i in range(12) for b in range(8)]
            bit = lambda byte, b: bits[byte * 8 + b]
            if sb < 4:
                wsc = sum(bit(sb, b) << b for b in range(6))
                wmn = sum(bit(sb + 4, b) << b for b in range(6))
            else:
                j = sb - 4
                wsc = sum(bit(8 + j, b) << b for b in range(4)) | (bit(j, 6) << 4) | (bit(j, 7) << 5)
                wmn = sum(bit(8 + j, 4 + b) << b for b in range(4)) | (bit(4 + j, 6) << 4) | (bit(4 + j, 7) << 5)
            assert (sc, mn) == (wsc, wmn)


def test_q4k_scale_min_roundtrips_encoder(kqo):
    rng = np.random.default_rng(2)
    d, dmin, sc, mn, q = synth.q4k_fields(rng, 64, 3)
    blk = synth.q4k_encode(d, dmin, sc, mn, q)
    for n in range(0, 64, 7):
        for b in range(3):
            for sb in range(8):
                assert kqo.q4k_scale_min(blk[n, b, 4:16], sb) == (sc[n, b, sb], mn[n, b, sb])


# ---- dequant ----------------------------------------------------------------
def test_q4k_dequant_is_single_rounding_of_exact_value(kqo):
    rng = np.random.default_rng(3)
    f = synth.q4k_fields(rng, 48, 4)
    raw = synth.q4k_encode(*f).reshape(48, -1)
    got = kqo.dequant(Q4_K, raw, 48, 1024)
    exact = synth.q4k_decode_f64(*f)            # every term exact in float64
    assert np.array_equal(got, exact.astype(np.float32))


def test_q5k_dequant_is_single_rounding_of_exact_value(kqo):
    """d*sc*q has at most 11 + 6 + 5 = 22 significant bits, so as for Q4_K the only rounding is the
    subtraction of dmin*mn."""
    rng = np.random.default_rng(13)
    f = synth.q5k_fields(rng, 48, 4)
    raw = synth.q5k_encode(*f).reshape(48, -1)
    got = kqo.dequant(Q5_K, raw, 48, 1024)
    exact = synth.q4k_decode_f64(*f)            # same formula, q now five bits
    assert np.array_equal(got, exact.astype(np.float32))


def test_q5k_element_order_and_fifth_bit_bruteforce(kqo):
    """One element set to 17 (nibble 1, fifth bit 1), then to 16 (fifth bit alone): it must land in
    out[e] with that value, and nowhere else."""
    for e in range(256):
        for v in (17, 16, 15):
            d = np.array([[1.0]], dtype=np.float16)
            z = np.array([[0.0]], dtype=np.float16)
            sc = np.ones((1, 1, 8), dtype=np.uint8)
            mn = np.zeros((1, 1, 8), dtype=np.uint8)
            q = np.zeros((1, 1, 256), dtype=np.uint8)
            q[0, 0, e] = v
            blk = synth.q5k_encode(d, z, sc, mn, q)
            # the layout itself, independent of the encoder: fifth bits at 16 + i, bit sb; nibbles at 48 + 32*(sb/2) + i
            sb, i = e // 32, e % 32
            assert blk[0, 0, 16 + i] == ((v >> 4) << sb)
            assert blk[0, 0, 48 + 32 * (sb // 2) + i] == ((v & 15) << (4 * (sb & 1)))
            out = kqo.dequant(Q5_K, blk.reshape(1, -1), 1, 256)[0]
            want = np.zeros(256, dtype=np.float32)
            want[e] = float(v)
            assert np.array_equal(out, want)


def test_q6k_dequant_is_exact(kqo):
    rng = np.random.default_rng(4)
    f = synth.q6k_fields(rng, 48, 4)
    raw = synth.q6k_encode(*f).reshape(48, -1)
    got = kqo.dequant(Q6_K, raw, 48, 1024)
    exact = synth.q6k_decode_f64(*f)
    assert np.array_equal(got.astype(np.float64), exact)


def test_q6k_element_order_bruteforce(kqo):
    """One-hot stored quants: element e must land in out[e]."""
    for e in range(256):
        d = np.array([[1.0]], dtype=np.float16)
        sc = np.ones((1, 1, 16), dtype=np.int8)
        q = np.full((1, 1, 256), 32, dtype=np.uint8)
        q[0, 0, e] = 33
        out = kqo.dequant(Q6_K, synth.q6k_encode(d, sc, q).reshape(1, -1), 1, 256)[0]
        want = np.zeros(256, dtype=np.float32)
        want[e] = 1.0
        assert np.array_equal(out, want)


def test_q6k_scale_group_bruteforce(kqo):
    """Scale j must govern exactly elements 16j .. 16j+15."""
    for j in range(16):
        d = np.array([[0.5]], dtype=np.float16)
        sc = np.zeros((1, 1, 16), dtype=np.int8)
        sc[0, 0, j] = -3
        q = np.full((1, 1, 256), 34, dtype=np.uint8)
        out = kqo.dequant(Q6_K, synth.q6k_encode(d, sc, q).reshape(1, -1), 1, 256)[0]
        want = np.zeros(256, dtype=np.float32)
        want[16 * j:16 * j + 16] = 0.5 * -3 * 2
        assert np.array_equal(out, want)


def test_q4k_element_order_bruteforce(kqo):
    for e in range(256):
        d = np.array([[1.0]], dtype=np.float16)
        z = np.array([[0.0]], dtype=np.float16)
        sc = np.ones((1, 1, 8), dtype=np.uint8)
        mn = np.zeros((1, 1, 8), dtype=np.uint8)
        q = np.zeros((1, 1, 256), dtype=np.uint8)
        q[0, 0, e] = 9
        out = kqo.dequant(Q4_K, synth.q4k_encode(d, z, sc, mn, q).reshape(1, -1), 1, 256)[0]
        want = np.zeros(256, dtype=np.float32)
        want[e] = 9.0
        assert np.array_equal(out, want)


def test_golden_random_blocks(kqo):
    g = np.load(os.path.join(GOLD, "random_blocks.npz"))
    for name in ("q4k", "q6k"):
        type_, N, K, nb, rs = (int(v) for v in g[f"{name}/desc"])
        assert kqo.n_blocks(K) == nb and kqo.row_stride_words(type_, K) == rs
        assert np.array_equal(kqo.pack(type_, g[f"{name}/raw"], N, K), g[f"{name}/packed"])
        got = kqo.dequant(type_, g[f"{name}/raw"], N, K)
        assert np.array_equal(got.view(np.uint32), g[f"{name}/deq_bits"])
        rows = np.arange(N, dtype=np.int32)[::-1]
        got2 = kqo.dequant_rows(type_, g[f"{name}/packed"], rows, K)
        assert np.array_equal(got2.view(np.uint32), g[f"{name}/deq_bits"][rows])


def test_differential_vs_compiled_reference(kqref):
    kqo = kqref
    for type_, (N, K) in ((Q4_K, (33, 1280)), (Q5_K, (33, 1280)), (Q6_K, (33, 1280))):
        raw = synth.make_raw(type_, N, K, seed=11)
        assert np.array_equal(kqo.dequant(type_, raw, N, K).view(np.uint32),
                              kqo.ref_dequant(type_, raw, N, K).view(np.uint32))
        pk, nb, rs = kqo.ref_pack(type_, raw, N, K)
        assert np.array_equal(kqo.pack(type_, raw, N, K), pk)
        assert (nb, rs) == (kqo.n_blocks(K), kqo.row_stride_words(type_, K))


# ---- layout ------------------------------------------------------------------
@pytest.mark.parametrize("K,q4,q6", [(4096, 576, 840), (14336, 2016, 2940), (768, 108, 158),
                                     (2048, 288, 420), (256, 36, 53)])
def test_row_stride_rule(kqo, K, q4, q6):
    assert kqo.row_stride_words(Q5_K, K) == 44 * (K // 256) == synth.row_stride_words(Q5_K, K)
    assert kqo.row_stride_words(Q4_K, K) == q4 == synth.row_stride_words(Q4_K, K)
    assert kqo.row_stride_words(Q6_K, K) == q6 == synth.row_stride_words(Q6_K, K)


def test_pack_pads_q6k_rows_with_zeros(kqo):
    raw = np.full((3, 3 * 210), 0xAB, dtype=np.uint8)
    pk = kqo.pack(Q6_K, raw, 3, 768).view(np.uint8).reshape(3, 632)
    assert np.all(pk[:, :630] == 0xAB) and np.all(pk[:, 630:] == 0)
    assert np.array_equal(kqo.pack(Q6_K, raw, 3, 768), synth.pack_rows(Q6_K, raw, 3, 768))


# ---- matmul ------------------------------------------------------------------
@pytest.mark.parametrize("type_", [Q4_K, Q6_K])
def test_matmul_unit_vectors_return_columns(kqo, type_):
    N, K = 5, 512
    raw = synth.make_raw(type_, N, K, seed=5)
    pk = kqo.pack(type_, raw, N, K)
    deq = kqo.dequant(type_, raw, N, K)
    X = np.eye(K, dtype=np.float32)[[0, 31, 32, 255, 256, 300, 511]]
    Y = kqo.matmul(type_, X, pk, N, K)
    assert np.array_equal(Y, deq[:, [0, 31, 32, 255, 256, 300, 511]].T)


@pytest.mark.parametrize("type_", [Q4_K, Q6_K])
def test_matmul_against_float64_and_sequential_numpy(kqo, type_):
    N, K, M = 9, 768, 3
    raw = synth.make_raw(type_, N, K, seed=6)
    pk = kqo.pack(type_, raw, N, K)
    deq = kqo.dequant(type_, raw, N, K)
    rng = np.random.default_rng(7)
    X = rng.standard_normal((M, K)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    Y = kqo.matmul(type_, X, pk, N, K, bias=bias)
    # independent sequential float32 evaluation, bias first
    for m in range(M):
        for n in range(N):
            a = np.float32(bias[n])
            for k in range(K):
                a = np.float32(a + np.float32(X[m, k] * deq[n, k]))
            assert Y[m, n] == a
    exact = bias.astype(np.float64) + X.astype(np.float64) @ deq.astype(np.float64).T
    y64 = kqo.matmul_f64(type_, X, pk, N, K, bias=bias)
    assert np.allclose(y64, exact, rtol=1e-13, atol=1e-12)
    scale = np.abs(X).astype(np.float64) @ np.abs(deq).astype(np.float64).T
    assert np.all(np.abs(Y - exact) <= K * 2.0 ** -24 * scale + 1e-6)


def test_matmul_y_offset_and_ld(kqo):
    N, K = 4, 256
    pk = synth.make_packed(Q4_K, N, K, seed=8)
    x = np.random.default_rng(9).standard_normal((2, K)).astype(np.float32)
    base = kqo.matmul(Q4_K, x, pk, N, K)
    Y = np.full((2, 10), -7.0, dtype=np.float32)
    kqo.matmul(Q4_K, x, pk, N, K, y_offset=3, ldy=10, Y=Y)
    assert np.array_equal(Y[:, 3:7], base)
    assert np.all(Y[:, :3] == -7) and np.all(Y[:, 7:] == -7)


def test_matmul_bf16_widens_exactly(kqo):
    N, K = 6, 512
    pk = synth.make_packed(Q6_K, N, K, seed=10)
    x = np.random.default_rng(11).standard_normal((3, K)).astype(np.float32)
    bits = (x.view(np.uint32) >> 16).astype(np.uint16)
    xw = (bits.astype(np.uint32) << 16).view(np.float32)
    assert np.array_equal(kqo.matmul_bf16(Q6_K, bits, pk, N, K), kqo.matmul(Q6_K, xw, pk, N, K))


# ---- the reference's eleven recipes -------------------------------------------
def test_reference_recipes_against_golden(kqo):
    import recipes
    g = np.load(os.path.join(GOLD, "recipes.npz"))
    R = recipes.build(kqo)
    assert len(R) == 11
    for name, r in R.items():
        type_, M, N, K, nb, rs = (int(v) for v in g[f"{name}/desc"])
        assert np.array_equal(r["raw"], g[f"{name}/raw"]), name      # closed-form bytes
        assert np.array_equal(kqo.pack(type_, r["raw"], N, K), g[f"{name}/packed"])
        assert np.array_equal(kqo.dequant(type_, r["raw"], N, K), g[f"{name}/deq"])
        if "rows" in r:
            got = kqo.dequant_rows(type_, g[f"{name}/packed"], g[f"{name}/rows"], K)
        else:
            # x is libm-dependent in the last place: regenerate, compare loosely,
            # then run the oracle on the stored x
            assert np.allclose(r["x"], g[f"{name}/x"], rtol=0, atol=1e-5)
            assert np.array_equal(r["bias"], g[f"{name}/bias"])
            got = kqo.matmul(type_, g[f"{name}/x"], g[f"{name}/packed"], N, K,
                             bias=g[f"{name}/bias"])
        assert np.array_equal(got, g[f"{name}/expected"]), name


# ---- MoE ---------------------------------------------------------------------
def test_topk_softmax_bruteforce(kqo):
    rng = np.random.default_rng(12)
    for _ in range(50):
        lg = rng.standard_normal(16).astype(np.float32)
        lg[rng.integers(0, 16)] = lg[rng.integers(0, 16)]   # ties now and then
        idx, wt = kqo.moe_topk_softmax(lg, 4)
        order = sorted(range(16), key=lambda e: (-lg[e], e))[:4]
        assert list(idx) == order
        ex = np.exp(lg[order].astype(np.float64) - lg[order].max())
        assert np.allclose(wt, ex / ex.sum(), rtol=1e-6)
        assert abs(wt.sum() - 1) < 1e-6


def test_moe_matmul_is_dense_matmul_on_row_slice(kqo):
    E, N, K, T, k = 5, 6, 512, 3, 2
    pk = synth.make_packed(Q4_K, E * N, K, seed=13)
    rs = kqo.row_stride_words(Q4_K, K)
    X = np.random.default_rng(14).standard_normal((T, K)).astype(np.float32)
    eidx = np.array([[4, 0], [2, 2], [1, 3]], dtype=np.uint32)
    Y = kqo.moe_matmul(Q4_K, X, pk, eidx, N, K)
    assert np.array_equal(kqo.moe_offsets(eidx[0], N), eidx[0] * N)
    for t in range(T):
        for s in range(k):
            e = int(eidx[t, s])
            want = kqo.matmul(Q4_K, X[t], pk[e * N * rs:(e + 1) * N * rs], N, K)[0]
            assert np.array_equal(Y[t, s], want)


def test_moe_ffn_composition(kqo):
    E, H, I, T, k = 4, 512, 256, 2, 2
    gate = synth.make_packed(Q4_K, E * I, H, seed=15)
    up = synth.make_packed(Q4_K, E * I, H, seed=16)
    down = synth.make_packed(Q6_K, E * H, I, seed=17)
    X = np.random.default_rng(18).standard_normal((T, H)).astype(np.float32) * 0.1
    eidx = np.array([[3, 1], [0, 3]], dtype=np.uint32)
    ew = np.array([[0.7, 0.3], [0.4, 0.6]], dtype=np.float32)
    out = kqo.moe_ffn(Q4_K, Q6_K, X, gate, up, down, eidx, ew, H, I)
    g = kqo.moe_matmul(Q4_K, X, gate, eidx, I, H).astype(np.float64)
    u = kqo.moe_matmul(Q4_K, X, up, eidx, I, H).astype(np.float64)
    act = (g / (1 + np.exp(-g)) * u).astype(np.float32)
    y = kqo.moe_matmul(Q6_K, act.reshape(T * k, I), down, eidx, H, I, x_per_slot=True)
    want = (ew[..., None].astype(np.float64) * y).sum(axis=1)
    assert np.allclose(out, want, rtol=2e-4, atol=2e-4 * np.abs(want).max())


# ---- prologues of the fused decode forms -----------------------------------------
def test_prologues_against_closed_forms_in_float64(kqo):
    """RMSNorm, silu*up and gelu_tanh*up against their definitions evaluated in float64 by numpy:
    a dropped eps, a mean over the wrong length, gate and up swapped, a wrong constant or sign in
    the gelu would each move the result by far more than the float32 rounding allowed here."""
    rng = np.random.default_rng(11)
    M, K = 3, 768
    x = (rng.standard_normal((M, K)) * 3).astype(np.float32)
    w = (1 + 0.2 * rng.standard_normal(K)).astype(np.float32)
    for eps in (1e-6, 0.5):
        got = kqo.prologue(1, x, K, norm_w=w, eps=eps)
        x64 = x.astype(np.float64)
        want = x64 / np.sqrt((x64 ** 2).mean(axis=1, keepdims=True) + eps) * w
        assert np.abs(got - want).max() <= 4e-7 * np.abs(want).max()
    # rows are independent and the norm is scale-free up to eps
    assert np.array_equal(kqo.prologue(1, x[1:2], K, norm_w=w, eps=1e-6), kqo.prologue(1, x, K, norm_w=w, eps=1e-6)[1:2])
    a = kqo.prologue(1, x, K, norm_w=w, eps=0.0)
    b = kqo.prologue(1, 4.0 * x, K, norm_w=w, eps=0.0)
    assert np.abs(a - b).max() <= 4e-7 * np.abs(a).max()
    gu = (rng.standard_normal((M, 2 * K)) * 4).astype(np.float32)
    g, u = gu[:, :K].astype(np.float64), gu[:, K:].astype(np.float64)
    silu = kqo.prologue(2, gu, K)
    assert np.abs(silu - g / (1 + np.exp(-g)) * u).max() <= 1e-6 * np.abs(u).max() * 4
    gelu = kqo.prologue(3, gu, K)
    want = 0.5 * g * (1 + np.tanh(np.sqrt(2 / np.pi) * (g + 0.044715 * g ** 3))) * u
    assert np.abs(gelu - want).max() <= 2e-6 * np.abs(u).max() * 4
    # special values: silu(0) = gelu(0) = 0; large positive gate passes up through, large negative kills it
    edge = np.array([[0.0, 30.0, -30.0, 1.0, 2.0, 3.0]], dtype=np.float32)
    assert kqo.prologue(2, edge, 3).tolist() == [[0.0, 60.0, -0.0]] or np.allclose(kqo.prologue(2, edge, 3), [[0, 60, 0]], atol=1e-10)
    assert np.allclose(kqo.prologue(3, edge, 3), [[0, 60, 0]], atol=1e-10)


def test_argmax_rows_is_the_sequential_scan(kqo):
    """The numpy form against the reference's scan written out as a loop, including ties, rows with
    nothing above the starting value, NaN and infinities."""
    rng = np.random.default_rng(2)
    rows = [rng.standard_normal(37).astype(np.float32) for _ in range(20)]
    rows += [np.zeros(37, np.float32), np.full(37, -2e30, np.float32), np.full(37, -np.inf, np.float32)]
    r = rng.standard_normal(37).astype(np.float32); r[[5, 20]] = r.max() + 1; rows.append(r)     # a tie
    r = rng.standard_normal(37).astype(np.float32); r[3] = np.nan; r[30] = np.inf; rows.append(r)
    r = np.full(37, np.nan, np.float32); rows.append(r)
    lg = np.stack(rows)
    want = []
    for row in lg:
        best, bi = np.float32(-1e30), 0
        for i, v in enumerate(row):
            if v > best:
                best, bi = v, i
        want.append(bi)
    assert kqo.argmax_rows(lg).tolist() == want
