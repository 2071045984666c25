"""MoE router stage on the GPU (bpk_moe_topk_softmax, bpk_moe_route) against the oracle's restatement
of topk_softmax.wgsl.  Selection is integer work: indices must match exactly on the same logits."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from backpack_amd import capi
    capi.check(capi.lib().bpk_init(0))
    import gpu_util
    return gpu_util


def _oracle(kqo, logits, k, normalize):
    T = logits.shape[0]
    idx = np.empty((T, k), np.uint32)
    wt = np.empty((T, k), np.float32)
    for t in range(T):
        idx[t], wt[t] = kqo.moe_topk_softmax(logits[t], k, normalize)
    return idx, wt


@pytest.mark.parametrize("T,E,k,normalize", [(1, 128, 8, True), (256, 128, 8, True), (7, 256, 8, False),
                                             (5, 1024, 16, True), (3, 60, 4, True), (9, 8, 8, True),
                                             (4, 64, 1, False), (2, 65, 2, True)])
def test_topk_softmax_vs_oracle(gpu, kqo, T, E, k, normalize):
    from backpack_amd import kquant
    print("topk", T, E, k, normalize, flush=True)
    rng = np.random.default_rng(T * 1000 + E)
    logits = (rng.standard_normal((T, E)) * 3).astype(np.float32)
    idx, wt = kquant.moe_topk_softmax(gpu.dev(logits), k, normalize)
    want_idx, want_wt = _oracle(kqo, logits, k, normalize)
    assert np.array_equal(idx.cpu().numpy().astype(np.uint32), want_idx)
    assert np.abs(wt.cpu().numpy() - want_wt).max() <= 2e-7 * max(1.0, float(np.abs(want_wt).max()))


def test_topk_ties_masks_and_degenerate_rows(gpu, kqo):
    """Ties go to the lowest index; -inf-like logits are never preferred; a row with nothing above
    -3.4e38 selects index 0 every time, as the reference's scan does."""
    from backpack_amd import kquant
    E, k = 128, 8
    rows = [np.zeros(E, np.float32),                                    # all equal: 0, 1, 2, ...
            np.where(np.arange(E) % 2 == 0, 1.0, 1.0).astype(np.float32),
            np.concatenate([np.full(E - 3, -3.4e38, np.float32), [5.0, 5.0, -1.0]]).astype(np.float32),
            np.full(E, -3.4e38, np.float32),                            # nothing selectable
            np.concatenate([[2.0], np.full(E - 1, -np.inf, np.float32)]).astype(np.float32),
            np.repeat(np.arange(E // 4, dtype=np.float32), 4)[::-1].copy()]   # runs of four equal values
    logits = np.stack(rows)
    idx, wt = kquant.moe_topk_softmax(gpu.dev(logits), k, True)
    want_idx, want_wt = _oracle(kqo, logits, k, True)
    got_idx = idx.cpu().numpy().astype(np.uint32)
    assert got_idx[0].tolist() == list(range(8))
    assert np.array_equal(got_idx, want_idx)
    got_wt = wt.cpu().numpy()
    both_nan = np.isnan(got_wt) & np.isnan(want_wt)
    assert np.all(both_nan | (np.abs(got_wt - want_wt) <= 2e-7))


@pytest.mark.parametrize("T,H,E,k", [(1, 2048, 128, 8), (256, 2048, 128, 8), (3, 4096, 256, 8), (2, 36, 10, 3),
                                     # many tokens: logits by tiles of 8 tokens x 16 experts (ragged in both), then the selection
                                     (70, 1024, 60, 4), (100, 36, 10, 3),
                                     # ... and more logits than the library's own buffer holds when none are asked for
                                     (9000, 64, 128, 8)])
def test_route_matvec_and_selection(gpu, kqo, T, H, E, k):
    """Logits against a float64 contraction; the selection must be the oracle's selection on the
    logits the GPU produced (a near-tie may legitimately order differently on other logits)."""
    from backpack_amd import kquant
    print("route", T, H, E, k, flush=True)
    rng = np.random.default_rng(H + E)
    x = rng.standard_normal((T, H)).astype(np.float32)
    w = (rng.standard_normal((E, H)) / np.sqrt(H)).astype(np.float32)
    idx, wt, logits = kquant.moe_route(gpu.dev(x), gpu.dev(w), k, True, want_logits=True)
    lg = logits.cpu().numpy()
    exact = x.astype(np.float64) @ w.astype(np.float64).T
    assert np.abs(lg - exact).max() <= 1e-5 * max(1.0, float(np.abs(exact).max()))
    want_idx, want_wt = _oracle(kqo, lg, k, True)
    assert np.array_equal(idx.cpu().numpy().astype(np.uint32), want_idx)
    assert np.abs(wt.cpu().numpy() - want_wt).max() <= 2e-7
    idx2, wt2 = kquant.moe_route(gpu.dev(x), gpu.dev(w), k, True)          # without the logits output
    assert np.array_equal(idx2.cpu().numpy(), idx.cpu().numpy()) and np.array_equal(wt2.cpu().numpy(), wt.cpu().numpy())


def test_route_feeds_the_expert_ffn(gpu, kqo):
    """router -> top-k -> expert FFN, all on the device, against the oracle chain on the GPU's logits."""
    from backpack_amd import kquant
    Q4_K, Q6_K = 12, 14
    T, E, k, H, I = 5, 16, 4, 512, 256
    rng = np.random.default_rng(3)
    x = rng.standard_normal((T, H)).astype(np.float32)
    wr = (rng.standard_normal((E, H)) / np.sqrt(H)).astype(np.float32)
    rg, pg, gate = gpu.make_weight(Q4_K, E * I, H, seed=1)
    ru, pu, up = gpu.make_weight(Q4_K, E * I, H, seed=2)
    rd, pd, down = gpu.make_weight(Q6_K, E * H, I, seed=3)
    xd = gpu.dev(x)
    idx, wt, logits = kquant.moe_route(xd, gpu.dev(wr), k, True, want_logits=True)
    out = kquant.moe_ffn(xd, gate, up, down, idx, wt, E).cpu().numpy()
    want_idx, want_wt = _oracle(kqo, logits.cpu().numpy(), k, True)
    want = kqo.moe_ffn(Q4_K, Q6_K, x, pg, pu, pd, want_idx, want_wt, H, I)
    scale = float(np.sqrt(np.mean(want.astype(np.float64) ** 2)))
    assert np.abs(out - want).max() <= 1e-3 * (scale + float(np.abs(want).max()))


def test_route_argument_checks(gpu):
    from backpack_amd import capi
    L = capi.lib()
    z = gpu.dev(np.zeros(4096, np.float32))
    p = z.data_ptr()
    assert L.bpk_moe_topk_softmax(p, 1, 2000, 8, 1, p, p, None) == -2      # more experts than the mask holds
    assert L.bpk_moe_topk_softmax(p, 1, 128, 17, 1, p, p, None) == -2      # k beyond MAX_K
    assert L.bpk_moe_topk_softmax(p, 1, 4, 8, 1, p, p, None) == -2         # k beyond n_experts
    assert L.bpk_moe_topk_softmax(None, 1, 128, 8, 1, p, p, None) == -3
    assert L.bpk_moe_route(p, p, 1, 30, 8, 2, 1, None, p, p, None) == -2   # hidden not a multiple of 4
    assert L.bpk_moe_route(p + 4, p, 1, 32, 8, 2, 1, None, p, p, None) == -4
    assert L.bpk_moe_topk_softmax(p, 0, 128, 8, 1, p, p, None) == 0        # no tokens: nothing to do
