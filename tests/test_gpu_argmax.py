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
