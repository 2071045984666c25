"""Fused decode forms (bpk_kq_matmul_fused) against the oracle: the prologue the reference's
q4k_matmul_norm / q4k_down_gelu kernels apply, composed with the oracle matmul and the residual add.
One-launch shapes and the workspace path must compute the same function."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

Q4_K, Q6_K = 12, 14
NONE, NORM, SILU, GELU = range(4)


@pytest.fixture(scope="module")
def gpu():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from backpack_amd import capi
    capi.check(capi.lib().bpk_init(0))
    import gpu_util
    return gpu_util


def _case(gpu, kqo, type_, M, N, K, pro, with_res, with_bias, seed):
    rng = np.random.default_rng(seed)
    raw, packed, w = gpu.make_weight(type_, N, K, seed=seed)
    X = (rng.standard_normal((M, K if pro in (NONE, NORM) else 2 * K)) * 1.5).astype(np.float32)
    norm_w = (1 + 0.1 * rng.standard_normal(K)).astype(np.float32) if pro == NORM else None
    res = rng.standard_normal((M, N)).astype(np.float32) if with_res else None
    bias = rng.standard_normal(N).astype(np.float32) if with_bias else None
    xp = X if pro == NONE else kqo.prologue(pro, X, K, norm_w=norm_w, eps=1e-5)
    return w, packed, X, norm_w, res, bias, xp


def _check(gpu, kqo, type_, got, xp, packed, N, K, res, bias, label):
    # the residual enters after the contraction: compare got - residual with the oracle matmul of x'.
    # slack 1e-5: exp / tanh / rsqrt come from a different libm than the oracle's, which moves x' by
    # an ulp or two before the contraction.
    got = np.asarray(got, dtype=np.float64).reshape(-1, N)
    if res is not None:
        got = got - res.astype(np.float64)
    gpu.check_matmul(kqo, type_, got.astype(np.float32), xp, packed, N, K, bias=bias, label=label, slack=1e-5)


ONE_LAUNCH = [
    # type, M, N, K, prologue, residual, bias
    (Q4_K, 1, 384, 4096, NORM, False, False),     # norm -> qkv
    (Q4_K, 2, 200, 2048, NORM, True, True),
    (Q4_K, 1, 130, 1024, SILU, True, False),
    (Q4_K, 2, 96, 4096, GELU, True, False),
    (Q4_K, 1, 64, 512, NONE, True, True),         # residual only
    (Q6_K, 1, 256, 14336, SILU, True, False),     # act -> down -> residual, the decode FFN tail
    (Q6_K, 2, 100, 14336, SILU, True, False),
    (Q6_K, 1, 77, 4096, NORM, False, True),
    (Q6_K, 2, 64, 7168, NORM, True, False),       # norm across K slices of several waves
    (Q6_K, 1, 50, 28672, GELU, False, False),
    (Q6_K, 2, 40, 2048, GELU, True, True),
    (Q6_K, 1, 33, 768, NORM, True, False),
    (Q4_K, 1, 100, 14336, SILU, True, False),     # Q4_K long rows: K slices over 7 waves
    (Q4_K, 2, 90, 14336, NORM, True, True),       # ... the norm's sum of squares across the slices
    (Q4_K, 1, 70, 8192, GELU, False, False),      # ... 4 slices
    (Q4_K, 1, 40, 28672, NORM, False, False),     # ... 7 slices of 16 superblocks
    (13, 1, 200, 4096, NORM, True, False),        # Q5_K
    (13, 1, 120, 14336, SILU, True, False),
    (13, 2, 64, 1024, SILU, True, True),
]


@pytest.mark.parametrize("type_,M,N,K,pro,with_res,with_bias", ONE_LAUNCH)
def test_fused_one_launch(gpu, kqo, type_, M, N, K, pro, with_res, with_bias):
    from backpack_amd import capi, kquant
    print("fused", type_, M, N, K, pro, with_res, with_bias, flush=True)
    w, packed, X, norm_w, res, bias, xp = _case(gpu, kqo, type_, M, N, K, pro, with_res, with_bias, seed=N + K)
    y = kquant.matmul_fused(gpu.dev(X), w, pro, norm_w=gpu.dev(norm_w) if norm_w is not None else None, eps=1e-5,
                            residual=gpu.dev(res) if res is not None else None,
                            bias=gpu.dev(bias) if bias is not None else None, allow_workspace=False)
    assert capi.last_kernel() == "gemv_stream_fused"
    _check(gpu, kqo, type_, y.cpu().numpy(), xp, packed, N, K, res, bias, f"fused {type_} {M}x{N}x{K} pro={pro}")


def test_fused_residual_in_place_and_same_as_separate_launches(gpu, kqo):
    """x += down(silu(gate) * up): the residual is the output buffer; and the one-launch result equals the
    three-launch result of the workspace path on the same inputs to fp32 summation-order accuracy."""
    import torch
    from backpack_amd import capi, kquant
    N, K = 512, 14336
    w, packed, X, _, res, _, xp = _case(gpu, kqo, Q6_K, 1, N, K, SILU, True, False, seed=5)
    y = gpu.dev(res.copy())
    kquant.matmul_fused(gpu.dev(X), w, SILU, residual=y, out=y, allow_workspace=False)
    _check(gpu, kqo, Q6_K, y.cpu().numpy(), xp, packed, N, K, res, None, "in-place residual")
    capi.set_option("fused_separate", 1)      # prologue, matmul and add launches
    try:
        y2 = gpu.dev(res.copy())
        kquant.matmul_fused(gpu.dev(X), w, SILU, residual=y2, out=y2)
        assert capi.last_kernel() == "gemv_stream"
    finally:
        capi.set_option("fused_separate", 0)
    _check(gpu, kqo, Q6_K, y2.cpu().numpy(), xp, packed, N, K, res, None, "in-place residual, workspace path")
    scale = float(np.sqrt(np.mean((y.cpu().numpy() - res) ** 2)))
    assert float((y - y2).abs().max()) <= 2e-5 * scale


# verify batches (and one or two tokens the decode kernel declines): one launch of the tile kernel
TILE_FUSED = [
    # type, M, N, K, prologue, residual, bias
    (Q4_K, 1, 60, 32768, SILU, True, False),     # rows longer than the decode kernel's K slices hold
    (Q4_K, 5, 96, 2048, NORM, True, False),
    (Q6_K, 16, 64, 1024, NORM, False, False),    # 16 tokens: the Q6_K kernel with 16 token slots
    (Q6_K, 8, 64, 1024, GELU, False, False),
    (Q6_K, 2, 48, 28672, NORM, True, False),     # the two-token long-row decode kernel carries no norm
    (Q4_K, 3, 40, 512, NONE, True, False),
    (Q4_K, 4, 4096, 4096, NORM, False, False),   # norm -> q at its real shape: K cut over workgroups
    (Q4_K, 8, 4096, 4096, NONE, True, True),     # o + residual
    (Q4_K, 16, 6144, 4096, NORM, False, True),   # norm -> q|k|v
    (Q6_K, 4, 4096, 14336, SILU, True, False),   # act -> down -> residual, the FFN tail at its real shape
    (Q6_K, 8, 4096, 14336, SILU, True, False),
    (Q6_K, 16, 4096, 14336, NONE, True, False),  # (x = the gate|up epilogue's output)
    (Q6_K, 11, 1000, 4096, NORM, False, True),
    (Q6_K, 13, 300, 2048, NORM, True, True),
    (Q6_K, 7, 2000, 768, GELU, True, False),
    (13, 6, 700, 4096, NORM, True, False),       # Q5_K
    (13, 16, 200, 14336, SILU, True, True),
    (Q4_K, 9, 2300, 1280, NORM, True, False),    # ragged last tile, partial last chunk
]


@pytest.mark.parametrize("type_,M,N,K,pro,with_res,with_bias", TILE_FUSED)
def test_fused_tile_kernel_one_launch(gpu, kqo, type_, M, N, K, pro, with_res, with_bias):
    """The same function as the decode forms on the 16x16 tile kernel: the prologue in its conversion of X, the
    residual in its store.  No workspace; also checked against the three-launch path on the same inputs."""
    from backpack_amd import capi, kquant
    print("fused tile", type_, M, N, K, pro, with_res, with_bias, flush=True)
    w, packed, X, norm_w, res, bias, xp = _case(gpu, kqo, type_, M, N, K, pro, with_res, with_bias, seed=M + N + K)
    args = dict(norm_w=gpu.dev(norm_w) if norm_w is not None else None, eps=1e-5,
                bias=gpu.dev(bias) if bias is not None else None)
    y = kquant.matmul_fused(gpu.dev(X), w, pro, residual=gpu.dev(res) if res is not None else None,
                            allow_workspace=False, **args)
    assert capi.last_kernel() == "mtile_fused"
    got = y.cpu().numpy()
    _check(gpu, kqo, type_, got, xp, packed, N, K, res, bias, f"fused tile {type_} {M}x{N}x{K} pro={pro}")
    if with_res:      # in place: the residual is the output buffer
        y2 = gpu.dev(res.copy())
        kquant.matmul_fused(gpu.dev(X), w, pro, residual=y2, out=y2, allow_workspace=False, **args)
        assert np.array_equal(y2.cpu().numpy(), got)
    capi.set_option("fused_separate", 1)      # prologue, matmul and add launches
    try:
        y3 = kquant.matmul_fused(gpu.dev(X), w, pro, residual=gpu.dev(res) if res is not None else None, **args)
        assert capi.last_kernel() != "mtile_fused"
    finally:
        capi.set_option("fused_separate", 0)
    ref = y3.cpu().numpy()
    base = ref - res if res is not None else ref
    scale = float(np.sqrt(np.mean(base.astype(np.float64) ** 2)))
    assert float(np.abs(got - ref).max()) <= 5e-5 * scale + 1e-6 * float(np.abs(ref).max())


WORKSPACE = [
    (Q4_K, 20, 96, 2048, NORM, True),      # more than 16 tokens
    (Q6_K, 16, 64, 1024, GELU, False),     # Q6_K beyond 8 tokens with a two-operand prologue
    (Q6_K, 33, 64, 1024, GELU, False),
    (Q4_K, 17, 40, 512, NONE, True),
]


@pytest.mark.parametrize("type_,M,N,K,pro,with_res", WORKSPACE)
def test_fused_workspace_path(gpu, kqo, type_, M, N, K, pro, with_res):
    from backpack_amd import capi, kquant
    print("fused ws", type_, M, N, K, pro, with_res, flush=True)
    w, packed, X, norm_w, res, bias, xp = _case(gpu, kqo, type_, M, N, K, pro, with_res, False, seed=M + K)
    args = dict(norm_w=gpu.dev(norm_w) if norm_w is not None else None, eps=1e-5,
                residual=gpu.dev(res) if res is not None else None)
    with pytest.raises(capi.BpkError) as e:
        kquant.matmul_fused(gpu.dev(X), w, pro, allow_workspace=False, **args)
    assert e.value.code == -7
    y = kquant.matmul_fused(gpu.dev(X), w, pro, **args)
    assert capi.last_kernel() not in ("gemv_stream_fused", "mtile_fused")
    _check(gpu, kqo, type_, y.cpu().numpy(), xp, packed, N, K, res, None, f"fused ws {type_} {M}x{N}x{K}")


def test_fused_argument_checks(gpu):
    import ctypes as C
    from backpack_amd import capi, kquant
    raw, packed, w = gpu.make_weight(Q4_K, 8, 256, seed=1)
    x = gpu.dev(np.zeros((1, 256), np.float32))
    y = gpu.dev(np.zeros((1, 8), np.float32))
    L = capi.lib()

    def call(f):
        return L.bpk_kq_matmul_fused(Q4_K, x.data_ptr(), w.data.data_ptr(), None, y.data_ptr(), 1, 8, 256, 1, 36, 0,
                                     f, None, 0, None)
    assert call(None) == -3
    assert call(C.byref(capi.Fusion(7, None, 0.0, None, 0))) == -2
    assert call(C.byref(capi.Fusion(capi.PRO_RMS_NORM, None, 1e-5, None, 0))) == -3
    assert call(C.byref(capi.Fusion(capi.PRO_NONE, None, 0.0, None, 0))) == 0     # plain matmul
    assert L.bpk_kq_matmul_fused_workspace_bytes(3, 10, 256) == 3 * 256 * 4 + 2 * 3 * 10 * 4


# ---- epilogue: act(gate . x) * (up . x) out of the stacked gate|up matvec -------------------------
EPI = [
    # type, M, N outputs, K, epilogue, prologue, bias, expected kernel
    (Q4_K, 1, 14336, 4096, SILU, NONE, False, "gemv_stream_fused"),     # the decode FFN head at its real shape
    (Q4_K, 1, 14336, 4096, SILU, NORM, False, "gemv_stream_fused"),     # ... with ffn_norm folded in (eight-wave form)
    (Q4_K, 2, 300, 4096, GELU, NONE, True, "gemv_stream_fused"),
    (Q4_K, 1, 257, 2048, SILU, NORM, False, "gemv_stream_fused"),       # ffn_norm folded in as well
    (Q4_K, 1, 100, 8192, SILU, NONE, False, "gemv_stream_fused"),       # K slices over four waves
    (Q4_K, 2, 64, 14336, GELU, NORM, True, "gemv_stream_fused"),        # ... over seven, two tokens
    (13, 1, 500, 4096, SILU, NONE, False, "gemv_stream_fused"),         # Q5_K
    (Q4_K, 1, 33, 256, SILU, NONE, False, "gemv_stream_fused"),         # fewer pairs than waves
    (Q6_K, 1, 200, 2048, SILU, NONE, False, None),                      # workspace path: Q6_K gate|up
    (Q4_K, 5, 120, 1024, GELU, NORM, True, None),                       # ... more than two tokens, outputs not in tiles of 16
    (Q4_K, 5, 128, 1024, GELU, NORM, True, "mtile_fused"),              # verify batches: gate and up tiles meet in the workgroup
    (Q4_K, 16, 14336, 4096, SILU, NORM, False, "mtile_fused"),          # ... the FFN head at its real shape
    (Q4_K, 4, 14336, 4096, SILU, NONE, False, "mtile_fused"),
    (Q4_K, 8, 1040, 5376, GELU, NONE, True, "mtile_fused"),             # ... K cut over workgroups, a ragged last group
    (Q6_K, 8, 256, 2048, SILU, NONE, True, "mtile_fused"),
    (Q6_K, 12, 96, 1024, GELU, NORM, False, "mtile_fused"),             # ... the 16-slot Q6_K kernel
    (13, 3, 512, 4096, SILU, NORM, False, "mtile_fused"),               # Q5_K
    (Q6_K, 1, 208, 2048, SILU, NONE, False, "mtile_fused"),             # one token where the decode kernel has no pair mode
]


@pytest.mark.parametrize("type_,M,N,K,epi,pro,with_bias,kernel", EPI)
def test_fused_gate_up_epilogue(gpu, kqo, type_, M, N, K, epi, pro, with_bias, kernel):
    from backpack_amd import capi, kquant
    print("fused epilogue", type_, M, N, K, epi, pro, with_bias, flush=True)
    rng = np.random.default_rng(N + K + M)
    raw, packed, w = gpu.make_weight(type_, 2 * N, K, seed=N)            # gate rows, then up rows
    X = rng.standard_normal((M, K)).astype(np.float32)
    norm_w = (1 + 0.1 * rng.standard_normal(K)).astype(np.float32) if pro == NORM else None
    bias = (0.1 * rng.standard_normal(2 * N)).astype(np.float32) if with_bias else None
    xp = X if pro == NONE else kqo.prologue(pro, X, K, norm_w=norm_w, eps=1e-5)
    gate_up = kqo.matmul(type_, xp, packed, 2 * N, K, bias=bias)          # [M, 2N] = gate | up
    want = kqo.prologue(epi, gate_up, N)
    args = dict(norm_w=gpu.dev(norm_w) if norm_w is not None else None, eps=1e-5,
                bias=gpu.dev(bias) if bias is not None else None, epilogue=epi)
    if kernel is None:
        with pytest.raises(capi.BpkError) as e:
            kquant.matmul_fused(gpu.dev(X), w, pro, allow_workspace=False, **args)
        assert e.value.code == -7
    y = kquant.matmul_fused(gpu.dev(X), w, pro, allow_workspace=kernel is None, **args)
    if kernel is not None:
        assert capi.last_kernel() == kernel
    got = y.cpu().numpy()
    assert got.shape == (M, N)
    # the product of two fp32 matvec results, each good to ~1e-6 of its rms: 2e-4 of the output's scale
    # leaves room for the device's exponential as well
    rms = float(np.sqrt(np.mean(want.astype(np.float64) ** 2)))
    assert np.all(np.abs(got - want) <= 2e-4 * (rms + np.abs(want))), float(np.abs(got - want).max())


def test_fused_epilogue_argument_checks(gpu):
    import ctypes as C
    from backpack_amd import capi
    raw, packed, w = gpu.make_weight(Q4_K, 16, 256, seed=1)
    x = gpu.dev(np.zeros((1, 256), np.float32))
    y = gpu.dev(np.zeros((1, 8), np.float32))
    L = capi.lib()

    def call(f):
        return L.bpk_kq_matmul_fused(Q4_K, x.data_ptr(), w.data.data_ptr(), None, y.data_ptr(), 1, 8, 256, 1, 36, 0,
                                     C.byref(f), None, 0, None)
    assert call(capi.Fusion(capi.PRO_NONE, None, 0.0, None, 1)) == -2                  # unknown epilogue
    assert call(capi.Fusion(capi.PRO_NONE, None, 0.0, y.data_ptr(), capi.EPI_SILU_MUL)) == -2   # residual with epilogue
    assert call(capi.Fusion(capi.PRO_NONE, None, 0.0, None, capi.EPI_SILU_MUL)) == 0


def _bf16_rne(x32):
    u = np.ascontiguousarray(x32, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


@pytest.mark.parametrize("M,K,pro", [(1, 256, NONE), (37, 4096, NONE), (300, 1000, NONE),
                                      (5, 4096, NORM), (257, 768, NORM), (3, 300, NORM),
                                      (4, 14336, SILU), (130, 768, SILU), (2, 1000, SILU),
                                      (6, 2048, GELU), (129, 512, GELU)])
def test_prefill_rows_bf16(gpu, kqo, M, K, pro):
    """Activation rows of the prefill GEMM: plain conversion is the round-to-nearest-even bit pattern;
    the prologue forms are the oracle's fp32 prologue rounded the same way, to within one bf16 step where
    the device's exp / tanh / rsqrt differ from the oracle's libm in the last place."""
    from backpack_amd import kquant
    rng = np.random.default_rng(M * 7 + K + pro)
    X = (rng.standard_normal((M, K if pro in (NONE, NORM) else 2 * K)) * 1.5).astype(np.float32)
    if pro == NONE:   # ties, subnormals, signed zero, the largest finite value
        X.flat[:6] = np.array([1.00390625, 1.01171875, 1e-40, -0.0, 3.3895313e38, -1.00390625], dtype=np.float32)[:min(6, X.size)]
    norm_w = (1 + 0.1 * rng.standard_normal(K)).astype(np.float32) if pro == NORM else None
    got = kquant.prefill_rows_bf16(gpu.dev(X), K, prologue=pro, norm_w=gpu.dev(norm_w) if norm_w is not None else None,
                                   eps=1e-5)
    assert tuple(got.shape) == (M, K)
    got = got.view(__import__("torch").int16).cpu().numpy().view(np.uint16)
    ref32 = X if pro == NONE else kqo.prologue(pro, X, K, norm_w=norm_w, eps=1e-5)
    want = _bf16_rne(ref32).reshape(M, K)
    if pro == NONE:
        assert np.array_equal(got, want)
        return
    step = np.abs(got.astype(np.int32) - want.astype(np.int32))
    assert step.max() <= 1, f"{int((step > 1).sum())} elements more than one bf16 step away"
    assert (step > 0).mean() < 0.02, f"{(step > 0).mean():.3%} of the elements differ"


def test_prefill_rows_bf16_feeds_the_gemm_and_checks_arguments(gpu, kqo):
    """norm -> bf16 rows -> dequant-GEMM equals the oracle matmul of the rounded rows; argument errors."""
    from backpack_amd import capi, kquant
    M, N, K = 300, 520, 1024
    rng = np.random.default_rng(5)
    raw, packed, w = gpu.make_weight(Q4_K, N, K, seed=9)
    X = rng.standard_normal((M, K)).astype(np.float32)
    norm_w = (1 + 0.1 * rng.standard_normal(K)).astype(np.float32)
    xb = kquant.prefill_rows_bf16(gpu.dev(X), K, prologue=NORM, norm_w=gpu.dev(norm_w), eps=1e-5)
    got = kquant.matmul(xb, w).cpu().numpy()
    assert capi.last_kernel() == "gemm_bf16"
    bits = xb.view(__import__("torch").int16).cpu().numpy().view(np.uint16)
    Xw = (bits.astype(np.uint32) << 16).view(np.float32)
    cpu = kqo.matmul(Q4_K, Xw, packed, N, K)
    assert np.abs(got - cpu).max() <= 1e-2 * float(np.abs(cpu).max())
    L = capi.lib()
    x = gpu.dev(X)
    assert L.bpk_prefill_rows_bf16(7, x.data_ptr(), None, 0.0, M, K, xb.data_ptr(), None) == -2
    assert L.bpk_prefill_rows_bf16(NORM, x.data_ptr(), None, 1e-5, M, K, xb.data_ptr(), None) == -3
    assert L.bpk_prefill_rows_bf16(NONE, None, None, 0.0, M, K, xb.data_ptr(), None) == -3
    assert L.bpk_prefill_rows_bf16(NONE, x.data_ptr(), None, 0.0, M, 0, xb.data_ptr(), None) == -2
    assert L.bpk_prefill_rows_bf16(NONE, x.data_ptr(), None, 0.0, 0, K, xb.data_ptr(), None) == 0
