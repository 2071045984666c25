"""GPU parity: the HIP path through the C ABI against the CPU oracle and the
committed golden fixtures.  Integer/bit work (dequantised weights) must match
bit for bit; matmuls are held to the tolerances written in gpu_util.check_matmul
and, for the reference's own nine cases, to the reference's tolerances."""
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

GOLD = os.path.join(os.path.dirname(__file__), "golden")
Q4_K, Q5_K, Q6_K = 12, 13, 14


@pytest.fixture(scope="module")
def gpu():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from backpack_amd import capi
    capi.check(capi.lib().bpk_init(0))
    import gpu_util
    return gpu_util


def _say(*a):
    print(*a, flush=True)


# ---- dequantised weights: bit-exact ---------------------------------------------
@pytest.mark.parametrize("type_", [Q4_K, Q5_K, Q6_K])
@pytest.mark.parametrize("N,K", [(1, 256), (33, 768), (64, 4096), (5, 14336)])
def test_dequant_bit_exact(gpu, kqo, type_, N, K):
    from backpack_amd import kquant
    _say("dequant", type_, N, K)
    raw, packed, w = gpu.make_weight(type_, N, K, seed=100 + N)
    got = kquant.dequant_rows(w).cpu().numpy()
    want = kqo.dequant(type_, raw, N, K)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("name", ["q4k", "q6k"])
def test_dequant_golden_random_blocks(gpu, name):
    from backpack_amd import kquant
    g = np.load(os.path.join(GOLD, "random_blocks.npz"))
    type_, N, K, nb, rs = (int(v) for v in g[f"{name}/desc"])
    w = kquant.upload(type_, g[f"{name}/packed"], N, K)
    assert (w.n_blocks, w.row_stride_words) == (nb, rs)
    rows = np.array([N - 1, 0, -3, 2], dtype=np.int32)          # negative ids clamp to row 0
    got = kquant.dequant_rows(w, gpu.dev(rows)).cpu().numpy()
    want = g[f"{name}/deq_bits"][np.maximum(rows, 0)]
    assert np.array_equal(got.view(np.uint32), want)


def test_dequant_full_size_row_checksum(gpu, kqo):
    """lm_head-sized Q6_K matrix: gather a scattered set of rows, bit-exact."""
    from backpack_amd import kquant
    N, K = 4096, 4096
    raw, packed, w = gpu.make_weight(Q6_K, N, K, seed=7)
    rows = np.array([0, 1, 63, 64, 1000, 4095], dtype=np.int32)
    got = kquant.dequant_rows(w, gpu.dev(rows)).cpu().numpy()
    want = kqo.dequant_rows(Q6_K, packed, rows, K)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


# ---- the reference's eleven known-answer cases --------------------------------------
RECIPES = ["q4k_matmul", "q4k_matmul_128", "q6k_matmul", "q6k_gather", "q6k_matmul_wide",
           "q6k_gather_batched", "q4k_matmul_batched4", "q6k_matmul_batched4", "q4k_matmul_batched8",
           "q5k_matmul", "q5k_matmul_batched4"]


@pytest.mark.parametrize("name", RECIPES)
@pytest.mark.parametrize("family", [0, 1])
def test_reference_recipe(gpu, kqo, name, family):
    from backpack_amd import capi, kquant
    g = np.load(os.path.join(GOLD, "recipes.npz"))
    type_, M, N, K, nb, rs = (int(v) for v in g[f"{name}/desc"])
    atol, rtol = (float(v) for v in g[f"{name}/tol"])
    w = kquant.upload(type_, g[f"{name}/packed"], N, K)
    _say("recipe", name, "family", family)
    if f"{name}/rows" in g:
        got = kquant.dequant_rows(w, gpu.dev(g[f"{name}/rows"])).cpu().numpy()
        assert np.array_equal(got, g[f"{name}/expected"])       # stricter than the 1e-6 asked
        return
    capi.force_kernel(family)
    try:
        got = kquant.matmul(gpu.dev(g[f"{name}/x"]), w, bias=gpu.dev(g[f"{name}/bias"])).cpu().numpy()
    finally:
        capi.force_kernel(0)
    bad, worst = kqo.assert_close(got, g[f"{name}/expected"], atol, rtol)
    assert bad == 0, f"{name}: {bad} elements outside atol={atol} rtol={rtol}, worst excess {worst}"


# ---- three and four tokens on the lanes-along-K kernel ---------------------------------
@pytest.mark.parametrize("type_,M,N,K", [
    (Q4_K, 3, 130, 2048), (Q4_K, 4, 300, 4096), (Q4_K, 3, 200, 8192), (Q4_K, 4, 100, 14336), (Q4_K, 4, 4096, 4096),
    (Q4_K, 3, 77, 6400),                       # 25 superblocks: the fourth K slice is partial
    (Q6_K, 4, 33, 768), (Q6_K, 3, 150, 4096), (Q6_K, 4, 120, 8192), (Q6_K, 3, 4096, 14336), (Q6_K, 4, 64, 2048),
    (Q5_K, 3, 90, 1024), (Q5_K, 4, 300, 4096), (Q5_K, 4, 60, 8192), (Q5_K, 3, 50, 14336), (Q5_K, 4, 4096, 4096),
])
def test_four_token_stream_kernels(gpu, kqo, type_, M, N, K):
    """Every K-slice count (1, 2, 4, 7 waves), three tokens run as four with the last masked: the rows of Y
    beyond M must stay untouched."""
    from backpack_amd import capi, kquant
    _say("four-token stream", type_, M, N, K)
    raw, packed, w = gpu.make_weight(type_, N, K, seed=M * 31 + N)
    X = np.random.default_rng(N + K).standard_normal((M, K)).astype(np.float32)
    bias = np.random.default_rng(2).standard_normal(N).astype(np.float32)
    out = gpu.dev(np.full((M + 1, N), 7.5, np.float32))
    kquant.matmul(gpu.dev(X), w, bias=gpu.dev(bias), out=out[:M])
    assert capi.last_kernel() == "gemv_stream"
    got = out.cpu().numpy()
    assert np.all(got[M] == 7.5)
    gpu.check_matmul(kqo, type_, got[:M], X, packed, N, K, bias=bias, label=f"four {type_} {M}x{N}x{K}")


# ---- Q5_K: the fp32 matmul's automatic choice (lanes-along-K kernel, tile kernel, generic) ---------
@pytest.mark.parametrize("M,N,K,kernel", [(1, 300, 4096, "gemv_stream"), (2, 64, 768, "gemv_stream"),
                                          (1, 4096, 4096, "gemv_stream"), (2, 6144, 4096, "gemv_stream"),
                                          (1, 77, 256, "gemv_stream"), (1, 500, 3072, "gemv_stream"),
                                          (5, 130, 2048, "mtile"), (17, 40, 512, "mtile"), (4, 64, 768, "gemv_stream"),
                                          (13, 700, 4096, "mtile"), (70, 40, 512, "mtile"), (300, 40, 512, "mtile"),
                                          (1, 1000, 14336, "gemv_stream"), (2, 300, 8192, "gemv_stream"),
                                          (1, 200, 28672, "gemv_stream"), (2, 200, 28672, "generic"),
                                          (1, 50, 32768, "generic")])
def test_q5k_matmul_vs_oracle(gpu, kqo, M, N, K, kernel):
    from backpack_amd import capi, kquant
    _say("q5k matmul", M, N, K)
    raw, packed, w = gpu.make_weight(Q5_K, N, K, seed=M + N)
    X = np.random.default_rng(K).standard_normal((M, K)).astype(np.float32)
    bias = np.random.default_rng(1).standard_normal(N).astype(np.float32)
    y = kquant.matmul(gpu.dev(X), w, bias=gpu.dev(bias)).cpu().numpy()
    assert capi.last_kernel() == kernel
    gpu.check_matmul(kqo, Q5_K, y, X, packed, N, K, bias=bias, label=f"q5k {M}x{N}x{K}", slack=2e-5 if kernel == "mtile" else 1e-6)
    if kernel != "generic":      # and the generic kernel on the same inputs
        capi.force_kernel(1)
        try:
            y1 = kquant.matmul(gpu.dev(X), w, bias=gpu.dev(bias)).cpu().numpy()
        finally:
            capi.force_kernel(0)
        gpu.check_matmul(kqo, Q5_K, y1, X, packed, N, K, bias=bias, label=f"q5k generic {M}x{N}x{K}")


# ---- matmul against the oracle ------------------------------------------------------
# Extra distance from the exact contraction allowed on top of twice the CPU path's own, in
# units of the output rms: VALU kernels accumulate like the CPU; the matrix-core kernels feed
# activations as fp16 hi + lo (22 bits relative to the largest element of the token's
# superblock) and the MFMA adds its products with about 2^-19 relative alignment loss.
SLACK = {"mrow": 1e-5, "mrow_grouped": 1e-5, "mtile": 2e-5, "mgemv": 2e-5}

SHAPES = [
    # type, M, N, K
    (Q4_K, 1, 4096, 4096),      # one decode projection (config 0)
    (Q4_K, 1, 1024, 4096),      # k / v projection
    (Q4_K, 1, 100, 256),        # ragged N, single block
    (Q4_K, 1, 333, 3072),       # 12 blocks: the second pass of the lanes-along-K kernel is partial
    (Q4_K, 1, 6144, 4096),      # fused q|k|v
    (Q4_K, 1, 64, 14336),       # long rows: K slices over 7 waves
    (Q4_K, 2, 500, 14336),
    (Q4_K, 1, 300, 8192),       # ... over 4 waves
    (Q4_K, 2, 100, 6400),       # ... 25 superblocks: the last slice is partial
    (Q4_K, 1, 90, 28672),       # ... 7 slices of two passes
    (Q4_K, 2, 90, 28672),
    (Q4_K, 1, 40, 32768),       # beyond the slices: row-per-lane kernel
    (Q4_K, 2, 200, 1024),
    (Q4_K, 3, 130, 2048),
    (Q4_K, 4, 65, 512),
    (Q4_K, 4, 70, 4096),        # two K slices x four walkers that share the activations; some walkers idle
    (Q4_K, 5, 9, 512),
    (Q4_K, 16, 96, 1024),
    (Q6_K, 1, 512, 4096),
    (Q6_K, 1, 100, 768),        # rows only 8-byte aligned
    (Q6_K, 1, 64, 14336),
    (Q6_K, 2, 70, 2048),
    (Q6_K, 4, 33, 768),
    (Q6_K, 8, 40, 1024),
    (Q6_K, 16, 130, 2048),
    (Q4_K, 7, 300, 4096),
    (Q4_K, 12, 64, 768),
    (Q6_K, 3, 2048, 768),       # the MoE down projection: odd block count, 632-byte rows
    (Q4_K, 16, 2000, 4096),     # tile kernel, one tile per workgroup, ragged last tile
    (Q4_K, 9, 2300, 1280),      # ... with a partial last chunk of superblocks (5 blocks)
    (Q6_K, 8, 2000, 4096),
    (Q6_K, 13, 1800, 1536),     # Q6_K beyond 8 tokens: two groups; 6 blocks
    (Q4_K, 37, 300, 1024),      # fp32 X beyond 16 tokens: groups of 16 (Q4_K) / 8 (Q6_K) on the tile kernel
    (Q6_K, 21, 200, 1024),
    (Q4_K, 64, 1024, 4096),     # ... a prefill-sized chunk through the fp32 entry point: four groups
    (Q4_K, 128, 512, 4096),
    (Q6_K, 300, 96, 1024),      # ... beyond 255 tokens (the tile kernel, not the generic one)
    (Q4_K, 16, 22500, 512),     # tile kernel, a wave per tile (7 or 8 tiles per workgroup), ragged last tile
    (Q6_K, 5, 23001, 768),
    (Q4_K, 16, 6144, 4096),     # tile kernel with K cut over workgroups (4 runs of one chunk), partials folded by the last
    (Q4_K, 6, 4100, 5376),      # ... 21 superblocks: runs of unequal length, the last with a partial chunk
    (Q6_K, 5, 4096, 14336),     # ... 7 runs of two chunks
    (Q6_K, 12, 1000, 7168),     # ... two token groups through the same scratch
    # Q5_K: the lanes-along-K kernel (one pass, two, K slices) and every mode of the tile kernel
    (Q5_K, 1, 4096, 4096),
    (Q5_K, 1, 100, 256),
    (Q5_K, 2, 500, 14336),
    (Q5_K, 1, 90, 28672),
    (Q5_K, 3, 130, 2048),
    (Q5_K, 3, 70, 4096),
    (Q5_K, 5, 9, 512),
    (Q5_K, 7, 300, 4096),
    (Q5_K, 16, 2000, 4096),     # one tile per workgroup, ragged last tile
    (Q5_K, 9, 2300, 1280),      # ... partial last chunk of superblocks
    (Q5_K, 37, 300, 1024),      # groups of 16 tokens
    (Q5_K, 16, 22500, 512),     # a wave per tile
    (Q5_K, 16, 6144, 4096),     # K cut over workgroups
    (Q5_K, 6, 4100, 5376),      # ... runs of unequal length
]


@pytest.mark.parametrize("type_,M,N,K", SHAPES)
@pytest.mark.parametrize("family", [0, 1, 2, 3, 5, 6, 7])
def test_matmul_vs_oracle(gpu, kqo, type_, M, N, K, family):
    from backpack_amd import capi, kquant
    raw, packed, w = gpu.make_weight(type_, N, K, seed=N + K)
    rng = np.random.default_rng(M * 7 + N)
    X = rng.standard_normal((M, K)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    capi.force_kernel(family)
    try:
        _say("matmul", type_, M, N, K, "family", family)
        try:
            got = kquant.matmul(gpu.dev(X), w, bias=gpu.dev(bias)).cpu().numpy()
        except capi.BpkError as e:
            assert family >= 2 and e.code == -2, e     # a forced family may decline a shape
            pytest.skip(f"family {family} declines this shape")
        kern = capi.last_kernel()
    finally:
        capi.force_kernel(0)
    r = gpu.check_matmul(kqo, type_, got, X, packed, N, K, bias=bias, label=f"{kern} {type_} {M}x{N}x{K}",
                         slack=SLACK.get(kern, 1e-6))
    _say("   kernel", kern, r)


@pytest.mark.parametrize("type_", [Q4_K, Q6_K])
@pytest.mark.parametrize("family,kernel", [(2, "gemv_rows"), (3, "mrow")])
@pytest.mark.parametrize("waves", [2, 4, 8])
@pytest.mark.parametrize("splits", [1, 2, 3, 16])
def test_gemv_split_k_and_counter_reset(gpu, kqo, type_, family, kernel, waves, splits):
    from backpack_amd import capi, kquant
    N, K, M = 200, 4096, 2
    raw, packed, w = gpu.make_weight(type_, N, K, seed=5)
    X = np.random.default_rng(splits).standard_normal((M, K)).astype(np.float32)
    capi.set_option("gemv_splits", splits)
    capi.set_option("gemv_waves", waves)
    capi.force_kernel(family)
    try:
        _say("split", type_, kernel, waves, splits)
        xd = gpu.dev(X)
        a = kquant.matmul(xd, w).cpu().numpy()
        assert capi.last_kernel() == kernel
        b = kquant.matmul(xd, w).cpu().numpy()          # counters must have been re-armed
    finally:
        capi.force_kernel(0)
        capi.set_option("gemv_splits", 0)
        capi.set_option("gemv_waves", 0)
    assert np.array_equal(a, b), "split-K result depends on the launch"
    gpu.check_matmul(kqo, type_, a, X, packed, N, K, label=f"waves={waves} splits={splits}",
                     slack=1e-5 if kernel == "mrow" else 1e-6)


STREAM_SHAPES = [
    (Q4_K, 9, 256), (Q4_K, 70, 1280), (Q4_K, 257, 2048), (Q4_K, 1000, 4096),
    # Q6_K: one pass, two passes, 4 K-slices (one partial), 7 slices, 7 slices x 2 passes
    (Q6_K, 9, 256), (Q6_K, 70, 768), (Q6_K, 300, 4096), (Q6_K, 130, 6400), (Q6_K, 200, 14336), (Q6_K, 40, 28672),
]


@pytest.mark.parametrize("type_,N,K", STREAM_SHAPES)
@pytest.mark.parametrize("depth", [1, 2, 4])
@pytest.mark.parametrize("rows_per_wave", [1, 3, 100])
@pytest.mark.parametrize("M", [1, 2])
def test_gemv_stream_shapes(gpu, kqo, type_, N, K, depth, rows_per_wave, M):
    """The lanes-along-K kernel over its tuning space: rows in flight per wave,
    rows per wave (1 = every wave a single row, 100 = more than the 64 rows a
    wave folds at a time), every pass / K-slice configuration, ragged last
    pass, one and two tokens, with a y offset and bias."""
    import torch
    from backpack_amd import capi, kquant
    raw, packed, w = gpu.make_weight(type_, N, K, seed=N)
    rng = np.random.default_rng(depth * 100 + rows_per_wave)
    X = rng.standard_normal((M, K)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    out = torch.full((M, N), 123.0, device="cuda")
    if M == 1:
        out = torch.full((1, N + 7), 123.0, device="cuda")   # room for a y offset
    capi.set_option("gemv_depth", depth)
    capi.set_option("gemv_splits", rows_per_wave)
    capi.force_kernel(5)
    try:
        _say("stream", type_, N, K, depth, rows_per_wave)
        xd, bd = gpu.dev(X), gpu.dev(bias)      # named: the buffers must outlive the call
        capi.check(capi.lib().bpk_kq_matmul(type_, xd.data_ptr(), w.data.data_ptr(), bd.data_ptr(),
                                            out.data_ptr(), M, N, K, w.n_blocks, w.row_stride_words, 7 if M == 1 else 0, None))
        assert capi.last_kernel() == "gemv_stream"
    finally:
        capi.force_kernel(0)
        capi.set_option("gemv_depth", 0)
        capi.set_option("gemv_splits", 0)
    got = out.cpu().numpy()
    if M == 1:
        assert np.all(got[:, :7] == 123.0), "wrote before y_offset"
        got = got[:, 7:]
    gpu.check_matmul(kqo, type_, got, X, packed, N, K, bias=bias,
                     label=f"stream {type_} {N}x{K} d{depth} r{rows_per_wave}")


@pytest.mark.parametrize("form", [0, 1])
@pytest.mark.parametrize("N,K", [(16, 256), (17, 512), (100, 4096), (1000, 2048), (333, 3840), (4099, 4096), (16400, 1792),
                                 (40000, 768)])
def test_matrix_core_gemv_shapes(gpu, kqo, N, K, form):
    """One token on the matrix cores (what Q4_K matrices of 16384 rows and more get by default), forced on small
    and ragged shapes: a last tile moved up to end at row N - 1, K slices that do not exist (fewer than 16
    superblocks, odd counts), more than eight tiles per workgroup (two rounds of the waves' meeting), both forms
    (eight waves of two superblocks, sixteen of one); with a y offset and bias, unit vectors, twice in a row."""
    import torch
    from backpack_amd import capi, kquant
    raw, packed, w = gpu.make_weight(Q4_K, N, K, seed=N + 2)
    rng = np.random.default_rng(N + form)
    bias = rng.standard_normal(N).astype(np.float32)
    out = torch.full((1, N + 3), 4.5, device="cuda")
    capi.set_option("gemv_splits", form)
    capi.force_kernel(7)
    try:
        for case in ("randn", "unit", "outlier"):
            X = rng.standard_normal((1, K)).astype(np.float32)
            if case == "unit":
                X[:] = 0.0
                X[0, int(rng.integers(K))] = 1.0
            elif case == "outlier":
                X[0, int(rng.integers(K))] = 3.0e4      # one huge activation: its superblock's other elements keep 22 bits of IT
            _say("mgemv", N, K, form, case)
            xd, bd = gpu.dev(X), gpu.dev(bias)
            got = []
            for _ in range(2):
                out.fill_(4.5)
                capi.check(capi.lib().bpk_kq_matmul(Q4_K, xd.data_ptr(), w.data.data_ptr(), bd.data_ptr(), out.data_ptr(), 1, N, K,
                                                    w.n_blocks, w.row_stride_words, 3, None))
                assert capi.last_kernel() == "mgemv"
                got.append(out.cpu().numpy())
            assert np.array_equal(got[0], got[1]), "two launches on the same inputs differ"
            assert np.all(got[0][:, :3] == 4.5)
            # (the outlier's products dominate the matrix instruction's running sums, whose additions lose alignment
            # bits at about 2^-19 of the LARGEST addend: every output carries a few 1e-5 of the outlier's product)
            gpu.check_matmul(kqo, Q4_K, got[0][:, 3:], X, packed, N, K, bias=bias, label=f"mgemv {N}x{K} form {form} {case}",
                             slack=1e-4 if case == "outlier" else 2e-5)
    finally:
        capi.force_kernel(0)
        capi.set_option("gemv_splits", 0)


def test_fp32_chunks_of_any_size_stay_off_the_generic_kernel(gpu, kqo):
    """fp32 X with more than 255 tokens: the tile kernel in groups of 16 tokens, as for 17 .. 255 (the generic
    kernel, one wave per output row, is the fallback for shapes no other kernel takes, not for token counts)."""
    from backpack_amd import capi, kquant
    M, N, K = 260, 128, 512
    raw, packed, w = gpu.make_weight(Q4_K, N, K, seed=9)
    X = np.random.default_rng(9).standard_normal((M, K)).astype(np.float32)
    got = kquant.matmul(gpu.dev(X), w).cpu().numpy()
    assert capi.last_kernel() == "mtile"
    gpu.check_matmul(kqo, Q4_K, got, X, packed, N, K, label="mtile 260 tokens", slack=2e-5)


def test_matrix_core_gemv_by_choice(gpu, kqo):
    """The library's own choice: Q4_K, one token, 49152 rows or more -> the matrix-core kernel; the option moves the
    threshold or switches it off."""
    from backpack_amd import capi, kquant
    N, K = 49152, 256
    raw, packed, w = gpu.make_weight(Q4_K, N, K, seed=5)
    X = np.random.default_rng(5).standard_normal((1, K)).astype(np.float32)
    got = kquant.matmul(gpu.dev(X), w).cpu().numpy()
    assert capi.last_kernel() == "mgemv"
    gpu.check_matmul(kqo, Q4_K, got, X, packed, N, K, label="mgemv by choice", slack=2e-5)
    capi.set_option("mgemv", 0)
    try:
        got2 = kquant.matmul(gpu.dev(X), w).cpu().numpy()
        assert capi.last_kernel() == "gemv_stream"
        capi.set_option("mgemv", 2)
        raw3, packed3, w3 = gpu.make_weight(Q4_K, 16384, 256, seed=6)
        got3 = kquant.matmul(gpu.dev(X), w3).cpu().numpy()
        assert capi.last_kernel() == "mgemv"
        gpu.check_matmul(kqo, Q4_K, got3, X, packed3, 16384, 256, label="mgemv from 16384 rows", slack=2e-5)
    finally:
        capi.set_option("mgemv", 1)
    gpu.check_matmul(kqo, Q4_K, got2, X, packed, N, K, label="stream with the option off")
    two = kquant.matmul(gpu.dev(np.repeat(X, 2, axis=0)), w)
    assert capi.last_kernel() != "mgemv"       # two tokens: not this kernel


@pytest.mark.parametrize("N,K", [(1000, 4096), (70, 3072), (16500, 2304), (9, 4096)])
def test_gemv_stream_eight_wave_form(gpu, kqo, N, K):
    """The lanes-along-K kernel as eight waves per workgroup, two rows in flight each (what matrices of
    12288 rows and more get by default), forced on small and ragged shapes; with a y offset and bias."""
    import torch
    from backpack_amd import capi, kquant
    raw, packed, w = gpu.make_weight(Q4_K, N, K, seed=N + 1)
    rng = np.random.default_rng(N)
    X = rng.standard_normal((1, K)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    out = torch.full((1, N + 5), 4.5, device="cuda")
    capi.set_option("gemv_waves", 8)
    capi.force_kernel(5)
    try:
        _say("stream eight waves", N, K)
        xd, bd = gpu.dev(X), gpu.dev(bias)
        capi.check(capi.lib().bpk_kq_matmul(Q4_K, xd.data_ptr(), w.data.data_ptr(), bd.data_ptr(), out.data_ptr(), 1, N, K,
                                            w.n_blocks, w.row_stride_words, 5, None))
        assert capi.last_kernel() == "gemv_stream"
    finally:
        capi.force_kernel(0)
        capi.set_option("gemv_waves", 0)
    got = out.cpu().numpy()
    assert np.all(got[:, :5] == 4.5)
    gpu.check_matmul(kqo, Q4_K, got[:, 5:], X, packed, N, K, bias=bias, label=f"stream 8 waves {N}x{K}")


@pytest.mark.parametrize("type_,M,N,K", [(Q6_K, 5, 4096, 14336), (Q4_K, 16, 6144, 4096)])
def test_tile_kernel_k_split_repeatable_and_counters_rearmed(gpu, type_, M, N, K):
    """Matrices of few rows: K is cut over workgroups and the last one to arrive adds the partial tiles in
    split order, so repeated calls give the same bits; the arrival counters are back at zero for the next."""
    import torch
    from backpack_amd import capi, kquant
    raw, packed, w = gpu.make_weight(type_, N, K, seed=5)
    x = torch.from_numpy(np.random.default_rng(3).standard_normal((M, K)).astype(np.float32)).cuda()
    _say("mtile repeat", type_, M, N, K)
    first = kquant.matmul(x, w).cpu().numpy()
    assert capi.last_kernel() == "mtile"
    for _ in range(3):
        again = kquant.matmul(x, w).cpu().numpy()
        assert np.array_equal(first.view(np.uint32), again.view(np.uint32))


def test_matmul_y_offset_no_bias(gpu, kqo):
    import torch
    from backpack_amd import kquant
    type_, N, K = Q4_K, 96, 512
    raw, packed, w = gpu.make_weight(type_, N, K, seed=9)
    X = np.random.default_rng(1).standard_normal((1, K)).astype(np.float32)
    # write into the middle of a wider, pre-filled output row (the fused q|k|v use)
    Y = torch.full((1, N), -5.0, device="cuda")
    half = kquant.KQuantPacked(w.data, type_, N // 2, K, w.row_stride_words, w.n_blocks)
    kquant.matmul(gpu.dev(X), half, out=Y, y_offset=10)
    got = Y.cpu().numpy()
    want = kqo.matmul(type_, X, packed, N // 2, K)
    assert np.all(got[0, :10] == -5) and np.all(got[0, 10 + N // 2:] == -5)
    assert np.allclose(got[0, 10:10 + N // 2], want[0], rtol=1e-4, atol=1e-3)


def test_matmul_unit_vector_returns_dequantised_column(gpu, kqo):
    from backpack_amd import kquant
    for type_ in (Q4_K, Q6_K):
        N, K = 128, 1024
        raw, packed, w = gpu.make_weight(type_, N, K, seed=21)
        deq = kqo.dequant(type_, raw, N, K)
        for k in (0, 31, 32, 255, 256, 777, 1023):
            X = np.zeros((1, K), dtype=np.float32)
            X[0, k] = 1.0
            got = kquant.matmul(gpu.dev(X), w).cpu().numpy()[0]
            assert np.allclose(got, deq[:, k], rtol=1e-6, atol=1e-7), (type_, k)


def test_matmul_linearity_full_size(gpu):
    """gate|up-sized matrix: W(ax + by) = a Wx + b Wy to fp32 accuracy."""
    import torch
    from backpack_amd import kquant
    N, K = 28672, 4096
    raw, packed, w = gpu.make_weight(Q4_K, N, K, seed=2)
    g = torch.Generator(device="cuda").manual_seed(0)
    x = torch.randn(1, K, device="cuda", generator=g)
    y = torch.randn(1, K, device="cuda", generator=g)
    lhs = kquant.matmul(1.5 * x - 0.25 * y, w)
    rhs = 1.5 * kquant.matmul(x, w) - 0.25 * kquant.matmul(y, w)
    scale = rhs.abs().max().item()
    assert (lhs - rhs).abs().max().item() <= 2e-5 * scale


# ---- MoE indirection ------------------------------------------------------------------
@pytest.mark.parametrize("type_,N,K,per_slot", [(Q4_K, 96, 512, False), (Q6_K, 64, 768, True), (Q5_K, 96, 512, False),
                                                 (Q5_K, 64, 768, True)])
def test_moe_matmul_vs_oracle(gpu, kqo, type_, N, K, per_slot):
    from backpack_amd import kquant
    E, T, k = 6, 5, 3
    raw, packed, w = gpu.make_weight(type_, E * N, K, seed=31)
    rng = np.random.default_rng(32)
    eidx = np.stack([rng.permutation(E)[:k] for _ in range(T)]).astype(np.uint32)
    X = rng.standard_normal((T * k if per_slot else T, K)).astype(np.float32)
    got = kquant.moe_matmul(gpu.dev(X), w, gpu.dev(eidx.view(np.int32)), E, x_per_slot=per_slot).cpu().numpy()
    want = kqo.moe_matmul(type_, X, packed, eidx, N, K, x_per_slot=per_slot)
    rms = np.sqrt(np.mean(want.astype(np.float64) ** 2))
    assert np.all(np.abs(got - want) <= 1e-3 * rms + 1e-3 * np.abs(want))


# ---- prefill GEMM on the matrix cores (bf16 X) -------------------------------------------
GEMM_SHAPES = [
    # type, M, N, K, tile
    (Q4_K, 128, 128, 256, 128),
    (Q4_K, 256, 256, 512, 256),
    (Q4_K, 200, 300, 1024, 128),     # ragged M and N
    (Q4_K, 300, 520, 768, 256),
    (Q4_K, 512, 1024, 4096, 0),
    (Q4_K, 33, 70, 2048, 0),
    (Q6_K, 128, 128, 256, 128),
    (Q6_K, 256, 256, 768, 256),      # odd block count: rows only 8-byte aligned
    (Q6_K, 190, 260, 1024, 128),
    (Q6_K, 512, 512, 4096, 0),
    # Q5_K: both tiles, the automatic choice, whole tiles and equal shares
    (Q5_K, 128, 128, 256, 128),
    (Q5_K, 200, 300, 1024, 0),
    (Q5_K, 512, 1024, 4096, 0),
    (Q5_K, 300, 520, 768, 256),
    (Q5_K, 256, 256, 512, 257),
    (Q5_K, 300, 520, 1024, 257),
    (Q5_K, 512, 1024, 4096, 258),
    (Q5_K, 190, 260, 2048, 258),
    # 256-tile with the walk cut into equal shares per CU (tiles summed with atomics)
    (Q4_K, 256, 256, 256, 258),
    (Q4_K, 300, 520, 768, 258),
    (Q4_K, 512, 1024, 4096, 258),
    (Q4_K, 2048, 1024, 1024, 258),   # 32 tiles x 16 steps on 256 CUs: two steps per workgroup
    (Q6_K, 256, 256, 768, 258),
    (Q6_K, 190, 260, 1024, 258),
    (Q6_K, 512, 512, 4096, 258),
    # 256-tile, one tile per workgroup
    (Q4_K, 512, 1024, 4096, 257),
    (Q6_K, 300, 520, 768, 257),
    # 256 tokens x 128 rows per workgroup (option value 129)
    (Q4_K, 300, 520, 768, 129),
    (Q4_K, 512, 1024, 4096, 129),
    (Q4_K, 33, 70, 2048, 129),
    (Q5_K, 300, 520, 1024, 129),
    (Q6_K, 190, 260, 1024, 129),
    (Q6_K, 256, 256, 768, 129),      # odd block count
    (Q6_K, 512, 512, 4096, 129),
    # 256 tokens x 192 rows per workgroup (option value 192)
    (Q4_K, 300, 520, 768, 192),
    (Q4_K, 768, 512, 4096, 192),
    (Q4_K, 33, 70, 2048, 192),
    (Q5_K, 300, 580, 1024, 192),
    (Q6_K, 190, 260, 1024, 192),
    (Q6_K, 384, 256, 768, 192),      # odd block count
    (Q6_K, 576, 512, 4096, 192),
]


def _bf16_bits(x32):
    """Round-to-nearest-even fp32 -> bf16 bit patterns (numpy)."""
    u = x32.view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


@pytest.mark.parametrize("type_,M,N,K,split", [
    (Q6_K, 1024, 2048, 8192, 0),    # 32 big tiles, long K: the automatic choice cuts every tile
    (Q4_K, 2048, 5120, 512, 0),     # 160 tiles
    (Q6_K, 256, 512, 8192, 2),      # 2 tiles x 128 k steps over all CUs: a tile is the sum of up to 128 runs
    (Q4_K, 512, 1536, 4096, 2),     # 12 tiles x 64 k steps: shares of 3, cut points wander through the tiles
])
def test_gemm_bf16_repeatable(gpu, type_, M, N, K, split):
    """Runs over part of a tile leave their sums in a workspace and a second kernel adds them in the order
    of the walk, so a call repeated on the same inputs gives the same bits however many runs a tile has."""
    import torch
    from backpack_amd import capi, kquant
    raw, packed, w = gpu.make_weight(type_, N, K, seed=7)
    rng = np.random.default_rng(11)
    bits = _bf16_bits(rng.standard_normal((M, K)).astype(np.float32))
    xd = torch.from_numpy(bits.view(np.int16)).cuda().view(torch.bfloat16)
    _say("gemm repeat", type_, M, N, K, split)
    if split:
        capi.set_option("gemm_tile", 256)
        capi.set_option("gemm_split", split)
    try:
        _gemm_repeat_body(capi, kquant, xd, w, split)
    finally:
        capi.set_option("gemm_tile", 0)
        capi.set_option("gemm_split", 0)


def _gemm_repeat_body(capi, kquant, xd, w, split):
    first = kquant.matmul(xd, w).cpu().numpy()
    assert capi.last_kernel() == "gemm_bf16"
    capi.set_option("gemm_split", 1)    # whole tiles, each walked by one workgroup
    try:
        whole = kquant.matmul(xd, w).cpu().numpy()
    finally:
        capi.set_option("gemm_split", split)
    assert np.allclose(first, whole, rtol=0, atol=1e-4 * float(np.abs(whole).max()))
    for _ in range(3):
        again = kquant.matmul(xd, w).cpu().numpy()
        assert np.array_equal(first.view(np.uint32), again.view(np.uint32))


@pytest.mark.parametrize("type_,M,N,K,tile", GEMM_SHAPES)
def test_gemm_bf16_vs_oracle(gpu, kqo, type_, M, N, K, tile):
    import torch
    from backpack_amd import capi, kquant
    raw, packed, w = gpu.make_weight(type_, N, K, seed=M + N)
    rng = np.random.default_rng(K + M)
    X = rng.standard_normal((M, K)).astype(np.float32)
    bits = _bf16_bits(X)
    bias = rng.standard_normal(N).astype(np.float32)
    xd = torch.from_numpy(bits.view(np.int16)).cuda().view(torch.bfloat16)
    capi.set_option("gemm_tile", min(tile, 256))
    capi.set_option("gemm_split", max(tile - 256, 0))   # 257 / 258: the 256-tile with split 1 / 2
    try:
        _say("gemm", type_, M, N, K, tile)
        got = kquant.matmul(xd, w, bias=gpu.dev(bias)).cpu().numpy()
        assert capi.last_kernel() == "gemm_bf16"
    finally:
        capi.set_option("gemm_tile", 0)
        capi.set_option("gemm_split", 0)
    Xw = (bits.astype(np.uint32) << 16).view(np.float32)
    cpu = kqo.matmul(type_, Xw, packed, N, K, bias=bias)        # the reference's fp32 CPU path
    err = np.abs(got.astype(np.float64) - cpu)
    peak, rms = float(np.abs(cpu).max()), float(np.sqrt(np.mean(cpu.astype(np.float64) ** 2)))
    # (1) the stated bar for the bf16 matrix-core path: 1e-2, relative to the
    #     largest output (bf16 weights carry a unit roundoff of 2^-8, so an
    #     output near zero can be off by more than 1e-2 of its own size)
    assert err.max() <= 1e-2 * peak, f"max error {err.max():.3g} vs 1e-2*peak {1e-2 * peak:.3g}"
    # (2) in aggregate the error is far smaller
    fro = float(np.sqrt((err ** 2).sum() / (cpu.astype(np.float64) ** 2).sum()))
    assert fro <= 4e-3, f"Frobenius relative error {fro:.3g}"
    # (3) and it is *only* that rounding: against the exact contraction of the
    #     bf16-rounded weights the kernel is accurate to fp32 accumulation
    deq = kqo.dequant(type_, raw, N, K)
    wbf = (_bf16_bits(deq).astype(np.uint32) << 16).view(np.float32)
    exact = Xw.astype(np.float64) @ wbf.astype(np.float64).T + bias.astype(np.float64)
    assert np.abs(got - exact).max() <= 2e-5 * peak + K * 2.0 ** -24 * rms
    _say(f"    max err/peak {err.max() / peak:.2e}  max err/rms {err.max() / rms:.2e}  frobenius {fro:.2e}")


# ---- MoE expert FFN ---------------------------------------------------------------------
def _routing(rng, T, E, k):
    eidx = np.stack([rng.permutation(E)[:k] for _ in range(T)]).astype(np.uint32)
    logits = rng.standard_normal((T, k)).astype(np.float32)
    ew = np.exp(logits - logits.max(axis=1, keepdims=True))
    ew = (ew / ew.sum(axis=1, keepdims=True)).astype(np.float32)
    return eidx, ew


@pytest.mark.parametrize("family", [0, 1, 3])
@pytest.mark.parametrize("tgu,tdn", [(Q4_K, Q6_K), (Q5_K, Q5_K), (Q5_K, Q6_K), (Q4_K, Q5_K)])
@pytest.mark.parametrize("T,E,k,H,I", [(1, 8, 2, 512, 512), (5, 6, 3, 512, 768), (40, 16, 4, 512, 512),
                                       (3, 4, 2, 512, 256), (70, 5, 4, 768, 512), (20, 64, 4, 512, 512)])
def test_moe_ffn_vs_oracle(gpu, kqo, family, tgu, tdn, T, E, k, H, I):
    from backpack_amd import capi, kquant
    _say("moe_ffn", tgu, tdn, T, E, k, H, I, "family", family)
    _, gp, gw = gpu.make_weight(tgu, E * I, H, seed=41)
    _, up, uw = gpu.make_weight(tgu, E * I, H, seed=42)
    _, dp, dw = gpu.make_weight(tdn, E * H, I, seed=43)
    rng = np.random.default_rng(T + E)
    eidx, ew = _routing(rng, T, E, k)
    X = (rng.standard_normal((T, H)) * 0.1).astype(np.float32)
    capi.force_kernel(family)
    try:
        got = kquant.moe_ffn(gpu.dev(X), gw, uw, dw, gpu.dev(eidx.view(np.int32)), gpu.dev(ew), E).cpu().numpy()
        kern = capi.last_kernel()
    finally:
        capi.force_kernel(0)
    # 1.25 or more pairs per expert on average go to the 16x16 tile kernel (family 3 keeps them on the
    # row kernel); a single-block Q6_K down projection (inter = 256) is outside the row kernel's reach
    # Q5_K has no row kernel: its thinly spread pairs beyond the lanes-along-K kernel's 256 take the tile kernel
    q5 = Q5_K in (tgu, tdn)
    if family == 1:
        expect = "moe_ffn_generic"
    elif family == 0 and 4 * T * k >= 5 * E:
        expect = "moe_ffn_mtile"
    elif family == 0 and T * k <= 256:
        expect = "moe_ffn_stream"     # thinly spread pairs: one lanes-along-K matvec each
    elif family == 0:
        expect = "moe_ffn_mtile" if q5 else "moe_ffn_mrow"
    else:
        expect = "moe_ffn_generic" if I == 256 or q5 else "moe_ffn_mrow"
    assert kern == expect, (kern, expect)
    want = kqo.moe_ffn(tgu, tdn, X, gp, up, dp, eidx, ew, H, I)
    rms = float(np.sqrt(np.mean(want.astype(np.float64) ** 2)))
    err = np.abs(got - want)
    # three chained fp32 matvecs and an exp(): 1e-3 relative, floor 1e-3 of the output rms
    assert np.all(err <= 1e-3 * rms + 1e-3 * np.abs(want)), f"max err {err.max():.3g} rms {rms:.3g}"


@pytest.mark.parametrize("tgu,tdn", [(Q4_K, Q6_K), (Q5_K, Q5_K)])
def test_moe_ffn_qwen3_shapes_decode_and_prefill(gpu, kqo, tgu, tdn):
    """Qwen3-30B-A3B-shaped experts (128 x [768x2048 Q4_K gate/up, 2048x768 Q6_K down]),
    top-8 routing: T=1 against the oracle, T=256 grouped path against the ungrouped
    one on the GPU plus an oracle spot check of four tokens."""
    import torch
    from backpack_amd import capi, kquant, synth
    E, k, H, I = 128, 8, 2048, 768
    mk = lambda t, N, K, seed: kquant.KQuantPacked(synth.make_packed_device(t, N, K, seed=seed), t, N, K,
                                                   synth.row_stride_words(t, K), synth.n_blocks(K))
    gw, uw, dw = mk(tgu, E * I, H, 51), mk(tgu, E * I, H, 52), mk(tdn, E * H, I, 53)
    host = lambda w: w.data[: w.N * w.row_stride_bytes].cpu().numpy().view(np.uint32)
    gp, up, dp = host(gw), host(uw), host(dw)
    rng = np.random.default_rng(5)
    for T in (1, 256):
        _say("moe qwen3 T", T)
        eidx, ew = _routing(rng, T, E, k)
        X = (rng.standard_normal((T, H)) * 0.1).astype(np.float32)
        xd, ed, wd = gpu.dev(X), gpu.dev(eidx.view(np.int32)), gpu.dev(ew)
        got = kquant.moe_ffn(xd, gw, uw, dw, ed, wd, E).cpu().numpy()
        assert capi.last_kernel() == ("moe_ffn_stream" if T == 1 else "moe_ffn_mtile")
        sel = np.arange(T) if T == 1 else np.array([0, 100, 101, 255])
        want = kqo.moe_ffn(tgu, tdn, X[sel], gp, up, dp, eidx[sel], ew[sel], H, I)
        rms = float(np.sqrt(np.mean(want.astype(np.float64) ** 2)))
        assert np.all(np.abs(got[sel] - want) <= 1e-3 * rms + 1e-3 * np.abs(want))
        if T > 1:
            capi.force_kernel(1)
            try:
                ref = kquant.moe_ffn(xd, gw, uw, dw, ed, wd, E).cpu().numpy()
            finally:
                capi.force_kernel(0)
            assert np.all(np.abs(got - ref) <= 1e-3 * rms + 1e-3 * np.abs(ref))
            again = kquant.moe_ffn(xd, gw, uw, dw, ed, wd, E).cpu().numpy()
            assert np.array_equal(got, again), "grouped path must not depend on bucket fill order"
            capi.force_kernel(3)   # the row kernel's grouped mode on the same routing
            try:
                rowk = kquant.moe_ffn(xd, gw, uw, dw, ed, wd, E).cpu().numpy()
                assert capi.last_kernel() == ("moe_ffn_mrow" if tgu == Q4_K else "moe_ffn_generic")
            finally:
                capi.force_kernel(0)
            assert np.all(np.abs(rowk - ref) <= 1e-3 * rms + 1e-3 * np.abs(ref))


@pytest.mark.parametrize("T,E,k,H,I", [(1, 16, 8, 512, 768), (3, 8, 2, 512, 256), (5, 64, 7, 768, 2304), (2, 16, 9, 512, 512),
                                       # rows of exactly four superblocks (two rows per step, every lane busy); odd rows per workgroup
                                       (4, 32, 4, 768, 1024), (7, 64, 8, 1280, 768)])
def test_moe_ffn_slot_sum_inside_the_last_matvec(gpu, kqo, T, E, k, H, I):
    """A few pairs with a Q6_K down projection: the weighted sum over a token's slots rides in down's launch
    (up to 8 slots; option moe_fold 0 keeps it a launch of its own).  Both against the oracle and each other."""
    from backpack_amd import capi, kquant
    _say("moe slot sum", T, E, k, H, I)
    _, gp, gw = gpu.make_weight(Q4_K, E * I, H, seed=61)
    _, up, uw = gpu.make_weight(Q4_K, E * I, H, seed=62)
    _, dp, dw = gpu.make_weight(Q6_K, E * H, I, seed=63)
    rng = np.random.default_rng(T * 7 + k)
    eidx, ew = _routing(rng, T, E, k)
    X = (rng.standard_normal((T, H)) * 0.1).astype(np.float32)
    got = {}
    try:
        for fold in (1, 0):
            capi.set_option("moe_fold", fold)
            got[fold] = kquant.moe_ffn(gpu.dev(X), gw, uw, dw, gpu.dev(eidx.view(np.int32)), gpu.dev(ew), E).cpu().numpy()
            assert capi.last_kernel() == "moe_ffn_stream"
    finally:
        capi.set_option("moe_fold", 1)
    want = kqo.moe_ffn(Q4_K, Q6_K, X, gp, up, dp, eidx, ew, H, I)
    rms = float(np.sqrt(np.mean(want.astype(np.float64) ** 2)))
    for fold in (1, 0):
        assert np.all(np.abs(got[fold] - want) <= 1e-3 * rms + 1e-3 * np.abs(want)), fold
    # the same products summed in the same slot order: only the rounding of wt * y may differ
    assert np.abs(got[1] - got[0]).max() <= 1e-5 * rms


@pytest.mark.parametrize("tgu,T,E,k,H,I", [(Q4_K, 40, 8, 2, 2048, 512), (Q4_K, 33, 4, 3, 1280, 512), (Q5_K, 24, 4, 2, 1536, 256),
                                           (Q6_K, 40, 8, 2, 2048, 256), (Q6_K, 10, 8, 2, 1280, 256)])
def test_moe_ffn_gate_and_up_in_one_tile_launch(gpu, kqo, tgu, T, E, k, H, I):
    """Batches of pairs on the tile kernel, hidden of more than one chunk of four superblocks: gate and up are
    walked in one launch that stores silu(gate x) * (up x) (option moe_fold 0: two launches and the activation
    kernel).  The same products in the same order and the same activation formula: equal bits; and the oracle."""
    from backpack_amd import capi, kquant
    _say("moe dual", tgu, T, E, k, H, I)
    _, gp, gw = gpu.make_weight(tgu, E * I, H, seed=71)
    _, up, uw = gpu.make_weight(tgu, E * I, H, seed=72)
    _, dp, dw = gpu.make_weight(Q6_K, E * H, I, seed=73)
    rng = np.random.default_rng(T * 5 + k)
    eidx, ew = _routing(rng, T, E, k)
    X = (rng.standard_normal((T, H)) * 0.1).astype(np.float32)
    got = {}
    try:
        for fold in (1, 0):
            capi.set_option("moe_fold", fold)
            got[fold] = kquant.moe_ffn(gpu.dev(X), gw, uw, dw, gpu.dev(eidx.view(np.int32)), gpu.dev(ew), E).cpu().numpy()
            assert capi.last_kernel() == "moe_ffn_mtile"
    finally:
        capi.set_option("moe_fold", 1)
    want = kqo.moe_ffn(tgu, Q6_K, X, gp, up, dp, eidx, ew, H, I)
    rms = float(np.sqrt(np.mean(want.astype(np.float64) ** 2)))
    assert np.all(np.abs(got[1] - want) <= 1e-3 * rms + 1e-3 * np.abs(want))
    assert np.array_equal(got[1], got[0])


@pytest.mark.parametrize("family,kernel", [(0, "mtile_grouped"), (3, "mrow_grouped")])
@pytest.mark.parametrize("type_,N,K,per_slot", [(Q4_K, 768, 2048, False), (Q6_K, 2048, 768, True),
                                                 # K of one chunk: waves walk several tiles per staged X; ragged last tile
                                                 (Q6_K, 2000, 768, True), (Q4_K, 1104, 1024, False),
                                                 (Q6_K, 520, 512, False),
                                                 (Q5_K, 768, 2048, False), (Q5_K, 2048, 768, True), (Q5_K, 1104, 1024, False)])
def test_moe_matmul_grouped_ragged(gpu, kqo, type_, N, K, per_slot, family, kernel):
    """Ragged lists: some experts get many pairs, some none; repeated experts inside a token."""
    from backpack_amd import capi, kquant
    E, T, k = 12, 37, 4
    raw, packed, w = gpu.make_weight(type_, E * N, K, seed=61)
    rng = np.random.default_rng(62)
    eidx = rng.choice([0, 1, 1, 1, 5, 5, 7, 11], size=(T, k)).astype(np.uint32)   # experts 2,3,4,6,8,9,10 idle
    X = rng.standard_normal((T * k if per_slot else T, K)).astype(np.float32)
    if type_ == Q5_K and family == 3:
        kernel = "generic_indirect"      # no row kernel for the type
    capi.force_kernel(family)
    try:
        got = kquant.moe_matmul(gpu.dev(X), w, gpu.dev(eidx.view(np.int32)), E, x_per_slot=per_slot).cpu().numpy()
        assert capi.last_kernel() == kernel
    finally:
        capi.force_kernel(0)
    want = kqo.moe_matmul(type_, X, packed, eidx, N, K, x_per_slot=per_slot)
    rms = np.sqrt(np.mean(want.astype(np.float64) ** 2))
    assert np.all(np.abs(got - want) <= 1e-3 * rms + 1e-3 * np.abs(want))


def test_moe_matmul_grouped_many_pairs(gpu, kqo):
    """More pairs than the grouping pass keeps in registers (4 per thread of its one workgroup): the rest are
    counted first and placed behind the kept ones by a second read."""
    from backpack_amd import capi, kquant
    type_, N, K = Q4_K, 128, 256
    E, T, k = 20, 1100, 4
    raw, packed, w = gpu.make_weight(type_, E * N, K, seed=71)
    rng = np.random.default_rng(72)
    eidx = rng.integers(0, E, size=(T, k)).astype(np.uint32)
    eidx[::7, 0] = 3                                        # one crowded expert
    X = rng.standard_normal((T, K)).astype(np.float32)
    _say("moe grouped, many pairs", T * k)
    got = kquant.moe_matmul(gpu.dev(X), w, gpu.dev(eidx.view(np.int32)), E, x_per_slot=False).cpu().numpy()
    assert capi.last_kernel() == "mtile_grouped"
    want = kqo.moe_matmul(type_, X, packed, eidx, N, K, x_per_slot=False)
    rms = np.sqrt(np.mean(want.astype(np.float64) ** 2))
    assert np.all(np.abs(got - want) <= 1e-3 * rms + 1e-3 * np.abs(want))


@pytest.mark.parametrize("type_,N,K,per_slot", [(Q4_K, 768, 2048, False), (Q6_K, 2048, 768, True), (Q6_K, 300, 4096, False),
                                                 (Q5_K, 768, 2048, False), (Q5_K, 2048, 768, True), (Q5_K, 300, 4096, False)])
def test_moe_matmul_few_pairs_stream(gpu, kqo, type_, N, K, per_slot):
    """Decode-sized routing (fewer than two pairs per expert): one lanes-along-K matvec per pair."""
    from backpack_amd import capi, kquant
    E, T, k = 12, 3, 4
    raw, packed, w = gpu.make_weight(type_, E * N, K, seed=71)
    rng = np.random.default_rng(72)
    eidx = np.stack([rng.permutation(E)[:k] for _ in range(T)]).astype(np.uint32)
    X = rng.standard_normal((T * k if per_slot else T, K)).astype(np.float32)
    got = kquant.moe_matmul(gpu.dev(X), w, gpu.dev(eidx.view(np.int32)), E, x_per_slot=per_slot).cpu().numpy()
    assert capi.last_kernel() == "stream_grouped"
    want = kqo.moe_matmul(type_, X, packed, eidx, N, K, x_per_slot=per_slot)
    rms = np.sqrt(np.mean(want.astype(np.float64) ** 2))
    assert np.all(np.abs(got - want) <= 1e-3 * rms + 1e-3 * np.abs(want))
