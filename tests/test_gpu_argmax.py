"""Greedy-sampling tail on the GPU (bpk_argmax_rows, bpk_kq_matmul_argmax): index work, exact."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

Q6_K = 14


@pytest.fixture(scope="module")
def gpu():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from backpack_amd import capi
    capi.check(capi.lib().bpk_init(0))
    import gpu_util
    return gpu_util


@pytest.mark.parametrize("M,N", [(1, 128256), (1, 1), (3, 4096), (16, 32000), (300, 1000), (2, 4097), (1, 262144)])
def test_argmax_rows_vs_oracle(gpu, kqo, M, N):
    from backpack_amd import kquant
    print("argmax", M, N, flush=True)
    rng = np.random.default_rng(M * 7 + N)
    lg = rng.standard_normal((M, N)).astype(np.float32)
    for _ in range(2):      # twice: the tickets must have been re-armed by the first launch
        idx, val = kquant.argmax_rows(gpu.dev(lg))
        assert np.array_equal(idx.cpu().numpy(), kqo.argmax_rows(lg))
        assert np.array_equal(val.cpu().numpy(), lg.max(axis=1))


def test_argmax_ties_and_degenerate_rows(gpu, kqo):
    from backpack_amd import kquant
    N = 20000
    rng = np.random.default_rng(0)
    rows = [np.zeros(N, np.float32), np.full(N, -2e30, np.float32), np.full(N, -np.inf, np.float32)]
    r = rng.standard_normal(N).astype(np.float32); r[[17, 9000, 19999]] = 9.0; rows.append(r)       # tie across parts
    r = rng.standard_normal(N).astype(np.float32); r[5] = np.nan; r[12345] = np.inf; rows.append(r)
    r = np.full(N, -5.0, np.float32); r[N - 1] = -4.0; rows.append(r)                                  # last element
    lg = np.stack(rows)
    idx, _ = kquant.argmax_rows(gpu.dev(lg))
    got = idx.cpu().numpy()
    assert np.array_equal(got, kqo.argmax_rows(lg))
    assert got.tolist() == [0, 0, 0, 17, 12345, N - 1]
    # a strided view: rows ld apart
    wide = gpu.dev(np.concatenate([lg, lg[:, ::-1]], axis=1))
    idx2, _ = kquant.argmax_rows(wide[:, :N])
    assert np.array_equal(idx2.cpu().numpy(), got)


def test_lm_head_with_argmax(gpu, kqo):
    """Q6_K lm_head rows -> logits -> pick, one call; the pick is the oracle's pick on the GPU's logits
    and the logits meet the matmul criteria."""
    from backpack_amd import kquant
    N, K = 40000, 1024
    raw, packed, w = gpu.make_weight(Q6_K, N, K, seed=9)
    for M in (1, 2, 5):
        X = np.random.default_rng(M).standard_normal((M, K)).astype(np.float32)
        logits, idx, val = kquant.matmul_argmax(gpu.dev(X), w)
        lg = logits.cpu().numpy()
        gpu.check_matmul(kqo, Q6_K, lg, X, packed, N, K, label=f"lm_head M={M}")
        assert np.array_equal(idx.cpu().numpy(), kqo.argmax_rows(lg))
        assert np.array_equal(val.cpu().numpy(), lg.max(axis=1))
        ref = kqo.matmul(Q6_K, X, packed, N, K)
        # the oracle's own pick agrees wherever its top two are further apart than the matmul tolerance
        top2 = np.sort(ref, axis=1)[:, -2:]
        clear = (top2[:, 1] - top2[:, 0]) > 1e-3 * np.abs(top2[:, 1])
        assert np.array_equal(idx.cpu().numpy()[clear], kqo.argmax_rows(ref)[clear])


def test_lm_head_pick_inside_the_matvec_launch(gpu, kqo):
    """One token over a vocabulary-sized Q6_K matrix: the row kernel leaves a partial pick per workgroup and
    its last workgroup reduces them.  Equal maxima (two identical weight rows), a repeated call (the ticket
    is re-armed), a bias, nothing above -1e30, and the same pick as the separate launch."""
    import torch
    from backpack_amd import capi, kquant
    N, K = 40000, 2048      # rows of 8 blocks: 16-byte aligned, as the row kernel wants them
    raw, packed, w = gpu.make_weight(Q6_K, N, K, seed=9)
    rows = w.data[: N * w.row_stride_bytes].view(N, w.row_stride_bytes)
    rows[31007] = rows[977]                       # identical rows: identical logits
    rows[39999] = rows[977]                       # ... and the last row of the last workgroup
    X = np.random.default_rng(3).standard_normal((1, K)).astype(np.float32)
    bias = np.zeros(N, np.float32)
    bias[[977, 31007, 39999]] = 1e4               # lift the three above everything else
    for rep in range(3):
        logits, idx, val = kquant.matmul_argmax(gpu.dev(X), w, bias=gpu.dev(bias))
        assert capi.last_kernel() == "gemv_rows_argmax"
        lg = logits.cpu().numpy()
        assert lg[0, 977] == lg[0, 31007] == lg[0, 39999]
        assert int(idx[0]) == 977 and float(val[0]) == lg[0, 977]
    # plain logits: the separate launch agrees
    logits, idx, val = kquant.matmul_argmax(gpu.dev(X), w)
    idx2, val2 = kquant.argmax_rows(logits)
    assert int(idx[0]) == int(idx2[0]) and float(val[0]) == float(val2[0])
    assert np.array_equal(idx.cpu().numpy(), kqo.argmax_rows(logits.cpu().numpy()))
    # nothing above -1e30: index 0, as the reference's scan from best = -1e30 leaves it
    low = gpu.dev(np.full(N, -3e30, np.float32))
    logits, idx, val = kquant.matmul_argmax(gpu.dev(X), w, bias=low)
    assert int(idx[0]) == 0 and float(val[0]) == np.float32(-1e30)
    # two tokens go to another kernel family and are followed by the pick's own launch
    X2 = np.random.default_rng(4).standard_normal((2, K)).astype(np.float32)
    logits, idx, val = kquant.matmul_argmax(gpu.dev(X2), w)
    assert capi.last_kernel() != "gemv_rows_argmax"
    assert np.array_equal(idx.cpu().numpy(), kqo.argmax_rows(logits.cpu().numpy()))
    # forced onto the row kernel, two tokens are picked inside the launch as well
    capi.force_kernel(2)
    try:
        l2, i2, v2 = kquant.matmul_argmax(gpu.dev(X2), w)
        assert capi.last_kernel() == "gemv_rows_argmax"
    finally:
        capi.force_kernel(0)
    assert np.array_equal(i2.cpu().numpy(), kqo.argmax_rows(l2.cpu().numpy()))
    assert np.array_equal(v2.cpu().numpy(), l2.cpu().numpy().max(axis=1))
