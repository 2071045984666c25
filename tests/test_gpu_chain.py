"""Chains of decode matvecs in one launch (bpk_chain_*) against the oracle: every kernel form, the fused
forms, ops that feed each other inside a launch, sub-ranges, repeated runs and graph replay, the give-up
path of a wait, and what bpk_chain_create refuses.  The oracle of a chain is the oracle of its ops applied
one after the other (kqo.prologue, kqo.matmul, the residual add), as for bpk_kq_matmul_fused."""
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


def _say(*a):
    print(*a, flush=True)


FORMS = [
    # type, N, K: one per kernel form, ragged N (waves without rows, a last partial 64-row chunk)
    (Q4_K, 300, 2048),     # whole rows, one pass
    (Q4_K, 4100, 4096),    # whole rows, two passes; three rows for some waves, two for others
    (Q4_K, 1, 1024),
    (Q4_K, 130, 8192),     # K slices of eight superblocks
    (Q4_K, 90, 16640),     # K slices of sixteen (65 superblocks: the last slice is partial)
    (Q4_K, 140000, 256),   # more than 64 rows per wave: a wave stores its sums in several chunks
    (Q6_K, 200, 1536),     # whole rows, one pass
    (Q6_K, 300, 4096),     # whole rows, two passes
    (Q6_K, 150, 14336),    # K slices of eight superblocks, seven of the eight waves
    (Q6_K, 64, 16640),     # K slices of sixteen
    (Q6_K, 2048, 768),     # rows only 8-byte aligned (632-byte stride)
    (Q6_K, 17000, 4352),   # K slices, more than 64 rows per workgroup
]


def test_chain_every_form_independent_ops(gpu, kqo):
    """One launch over ops that do not feed each other: each must equal its own matvec."""
    import torch
    from backpack_amd import capi, kquant
    rng = np.random.default_rng(0)
    items = []
    ch = kquant.Chain()
    for i, (type_, N, K) in enumerate(FORMS):
        raw, packed, w = gpu.make_weight(type_, N, K, seed=300 + i)
        X = rng.standard_normal((1, K)).astype(np.float32)
        bias = rng.standard_normal(N).astype(np.float32) if i % 2 else None
        out = torch.full((1, N + 5), 9.25, device="cuda")
        ch.add(gpu.dev(X), w, out, bias=gpu.dev(bias) if bias is not None else None, y_offset=3 if i % 3 == 0 else 0)
        items.append((type_, N, K, packed, X, bias, out, 3 if i % 3 == 0 else 0))
    ch.build()
    for first, count in ((0, len(FORMS)), (0, 3), (3, len(FORMS) - 3), (5, 1)):
        for it in items:
            it[6].fill_(9.25)
        _say("chain forms", first, count)
        ch.run(first, count)
        torch.cuda.synchronize()
        ch.status()
        assert capi.last_kernel() == "chain"
        for k, (type_, N, K, packed, X, bias, out, yo) in enumerate(items):
            got = out.cpu().numpy()[0]
            if not (first <= k < first + count):
                assert np.all(got == 9.25), f"op {k} outside the launch was written"
                continue
            assert np.all(got[:yo] == 9.25) and np.all(got[yo + N:] == 9.25), f"op {k} wrote outside its outputs"
            gpu.check_matmul(kqo, type_, got[yo:yo + N], X, packed, N, K, bias=bias, label=f"chain op {k} {type_} {N}x{K}")


def _layer(gpu, kqo, hidden, inter, kv, seed, in_place):
    """o (+ residual) -> ffn norm -> gate|up -> silu*up -> down (+ residual) -> attn norm -> q|k|v, as one chain.
    Returns the chain, its buffers and the host copies the oracle needs."""
    import torch
    from backpack_amd import capi, kquant
    rng = np.random.default_rng(seed)
    W = {}
    for name, type_, N, K in (("o", Q4_K, hidden, hidden), ("gate_up", Q4_K, 2 * inter, hidden),
                              ("down", Q6_K, hidden, inter), ("qkv", Q4_K, hidden + 2 * kv, hidden)):
        raw, packed, w = gpu.make_weight(type_, N, K, seed=seed + len(name))
        W[name] = (type_, N, K, packed, w)
    host = dict(attn=(rng.standard_normal((1, hidden)) * 0.05).astype(np.float32),
                h0=rng.standard_normal((1, hidden)).astype(np.float32),
                ffn_norm=(1 + 0.1 * rng.standard_normal(hidden)).astype(np.float32),
                attn_norm=(1 + 0.1 * rng.standard_normal(hidden)).astype(np.float32))
    d = {k: gpu.dev(v) for k, v in host.items()}
    d["h1"] = d["h0"] if in_place else torch.zeros(1, hidden, device="cuda")
    d["h2"] = d["h0"] if in_place else torch.zeros(1, hidden, device="cuda")
    d["act"] = torch.zeros(1, inter, device="cuda")
    d["qkv"] = torch.zeros(1, hidden + 2 * kv, device="cuda")
    ch = kquant.Chain()
    ch.add(d["attn"], W["o"][4], d["h1"], residual=d["h0"])
    ch.add(d["h1"], W["gate_up"][4], d["act"], prologue=capi.PRO_RMS_NORM, norm_w=d["ffn_norm"], eps=1e-5,
           epilogue=capi.EPI_SILU_MUL)
    ch.add(d["act"], W["down"][4], d["h2"], residual=d["h1"])
    ch.add(d["h2"], W["qkv"][4], d["qkv"], prologue=capi.PRO_RMS_NORM, norm_w=d["attn_norm"], eps=1e-5)
    ch.build()
    return ch, d, host, W


def _check_layer(gpu, kqo, d, host, W, hidden, inter):
    """Every op against the oracle applied to the inputs the GPU itself produced for it."""
    h1, act, h2, qkv = (d[k].cpu().numpy() for k in ("h1", "act", "h2", "qkv"))
    t, N, K, packed, _ = W["o"]
    gpu.check_matmul(kqo, t, h1 - host["h0"], host["attn"], packed, N, K, label="o", slack=1e-5)
    t, N, K, packed, _ = W["gate_up"]
    xn = kqo.prologue(NORM, h1, K, norm_w=host["ffn_norm"], eps=1e-5)
    gu = kqo.matmul(t, xn, packed, N, K)
    want = kqo.prologue(SILU, gu, inter)
    rms = float(np.sqrt(np.mean(want.astype(np.float64) ** 2)))
    assert np.all(np.abs(act - want) <= 1e-3 * rms + 1e-3 * np.abs(want)), "gate|up with the activation folded in"
    t, N, K, packed, _ = W["down"]
    gpu.check_matmul(kqo, t, h2 - h1, act, packed, N, K, label="down", slack=1e-5)
    t, N, K, packed, _ = W["qkv"]
    xn = kqo.prologue(NORM, h2, K, norm_w=host["attn_norm"], eps=1e-5)
    gpu.check_matmul(kqo, t, qkv, xn, packed, N, K, label="qkv", slack=1e-5)


@pytest.mark.parametrize("hidden,inter,kv", [(1024, 2816, 256), (4096, 14336, 1024)])
def test_chain_decoder_layer_vs_oracle(gpu, kqo, hidden, inter, kv):
    """The stretch of a decoder layer between two attention blocks, every op fed by the one before, in one
    launch; at the Llama-3-8B shapes and at a small one (one-pass forms)."""
    import torch
    _say("chain layer", hidden, inter)
    ch, d, host, W = _layer(gpu, kqo, hidden, inter, kv, seed=hidden, in_place=False)
    ch.run()
    torch.cuda.synchronize()
    ch.status()
    _check_layer(gpu, kqo, d, host, W, hidden, inter)
    first = {k: d[k].clone() for k in ("h1", "act", "h2", "qkv")}
    # again, and in pieces: the same bits every time (the mailboxes' parity alternates from run to run)
    for pieces in ([(0, 4)], [(0, 1), (1, 3)], [(0, 2), (2, 2)], [(0, 1), (1, 1), (2, 1), (3, 1)]):
        for k in first:
            d[k].zero_()
        for a, n in pieces:
            ch.run(a, n)
        torch.cuda.synchronize()
        ch.status()
        for k in first:
            assert torch.equal(d[k], first[k]), f"{k} differs when launched as {pieces}"


def test_chain_in_place_equals_separate_calls(gpu, kqo):
    """x += o(attn); act = silu(gate(n(x))) * up(n(x)); x += down(act); qkv = W n(x) with one buffer for x: the chain
    against the same four bpk_kq_matmul_fused calls, and the chain replayed from a HIP graph."""
    import torch
    from backpack_amd import capi, kquant
    hidden, inter, kv = 4096, 14336, 1024
    ch, d, host, W = _layer(gpu, kqo, hidden, inter, kv, seed=77, in_place=True)

    def separate():
        x = gpu.dev(host["h0"])
        kquant.matmul_fused(d["attn"], W["o"][4], residual=x, out=x)
        act = kquant.matmul_fused(x, W["gate_up"][4], capi.PRO_RMS_NORM, norm_w=d["ffn_norm"], eps=1e-5,
                                  epilogue=capi.EPI_SILU_MUL)
        kquant.matmul_fused(act, W["down"][4], residual=x, out=x)
        qkv = kquant.matmul_fused(x, W["qkv"][4], capi.PRO_RMS_NORM, norm_w=d["attn_norm"], eps=1e-5)
        return x, act, qkv
    x_ref, act_ref, qkv_ref = separate()
    h0 = gpu.dev(host["h0"])

    def close(a, b):
        # the bound of the C++ host layer's chain test (tests/cpp/kernel_test.cpp, chain_of_a_decoder_layer_tail:
        # separate fused dispatches against the chain, atol = rtol = 1e-4 per element on outputs of unit scale; here
        # the outputs are not of unit scale, so the absolute part is 1e-4 of their rms), and 2e-5 of the largest element
        scale = float(b.abs().max())
        rms = float(b.double().pow(2).mean().sqrt())
        elementwise = bool(((a - b).abs() <= 1e-4 * rms + 1e-4 * b.abs()).all())
        return elementwise and float((a - b).abs().max()) <= 2e-5 * scale
    ch.run()
    torch.cuda.synchronize()
    ch.status()
    assert close(d["h0"], x_ref) and close(d["act"], act_ref) and close(d["qkv"], qkv_ref)
    want = {k: d[k].clone() for k in ("h0", "act", "qkv")}
    # graph replay: several times, with eager work and synchronisation between the replays
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        d["h0"].copy_(h0)
        ch.run()
        s.synchronize()
        g = torch.cuda.CUDAGraph()
        d["h0"].copy_(h0)
        with torch.cuda.graph(g, stream=s):
            ch.run()
        for rep in range(4):
            d["h0"].copy_(h0)
            d["act"].zero_()
            d["qkv"].zero_()
            g.replay()
            s.synchronize()
            for k in want:
                assert torch.equal(d[k], want[k]), f"replay {rep}: {k} differs from the eager run"
            _ = (d["qkv"] * 2).sum().item()
    ch.status()


def test_chain_wait_gives_up_and_recovers(gpu, kqo):
    """A wait that cannot be satisfied (the ops are kept from handing their outputs on) runs out after the
    bound, every workgroup leaves, the chain reports it and does nothing until it is reset."""
    import torch
    from backpack_amd import capi
    ch, d, host, W = _layer(gpu, kqo, 1024, 2816, 256, seed=5, in_place=False)
    ch.run()
    torch.cuda.synchronize()
    ch.status()
    good = d["qkv"].clone()
    capi.set_option("chain_hold", 1)
    capi.set_option("chain_spin_us", 3000)
    try:
        d["qkv"].zero_()
        ch.run()
        torch.cuda.synchronize()
    finally:
        capi.set_option("chain_hold", 0)
        capi.set_option("chain_spin_us", 0)
    with pytest.raises(capi.BpkError) as e:
        ch.status()
    assert e.value.code == -11 and "op 1" in str(e.value)
    assert float(d["qkv"].abs().max()) == 0.0, "an op behind the wait that ran out was computed"
    d["h1"].zero_()
    ch.run()                      # does nothing until the reset
    torch.cuda.synchronize()
    assert float(d["h1"].abs().max()) == 0.0
    ch.reset()
    ch.status()
    ch.run()
    torch.cuda.synchronize()
    ch.status()
    assert torch.equal(d["qkv"], good)


def test_chain_status_waits_for_launches_on_side_streams(gpu, kqo):
    """bpk_chain_status synchronises with the device itself: a launch issued on a non-blocking side stream that is
    still inside its bounded wait when status is called must be waited for and reported, without the caller
    synchronising first."""
    import torch
    from backpack_amd import capi
    ch, d, host, W = _layer(gpu, kqo, 1024, 2816, 256, seed=6, in_place=False)
    ch.run()
    torch.cuda.synchronize()
    ch.status()
    side = torch.cuda.Stream()
    capi.set_option("chain_hold", 1)
    with pytest.raises(capi.BpkError) as e:        # the hook is refused without a short bound on the waits
        ch.run()
    assert e.value.code == -2 and "chain_spin_us" in str(e.value)
    capi.set_option("chain_spin_us", 50000)        # 50 ms: far longer than the host needs to reach status()
    try:
        with torch.cuda.stream(side):
            ch.run()
    finally:
        capi.set_option("chain_hold", 0)
        capi.set_option("chain_spin_us", 0)
    with pytest.raises(capi.BpkError) as e:
        ch.status()                                # no synchronize in between
    assert e.value.code == -11
    ch.reset()
    ch.run()
    ch.status()
    with pytest.raises(capi.BpkError):
        capi.set_option("chain_spin_us", 20000000)


def test_chain_create_refusals(gpu):
    import torch
    from backpack_amd import capi, kquant
    raw, packed, w4 = gpu.make_weight(Q4_K, 64, 512, seed=1)
    raw, packed, w6 = gpu.make_weight(Q6_K, 64, 512, seed=2)
    x = torch.zeros(1, 512, device="cuda")
    y = torch.zeros(1, 640, device="cuda")

    def build(*ops):
        ch = kquant.Chain()
        for o in ops:
            ch.add(*o[0], **o[1])
        return ch.build()
    # an epilogue on a Q6_K matrix has no kernel form
    with pytest.raises(capi.BpkError) as e:
        build(((x, w6, y), dict(epilogue=capi.EPI_SILU_MUL)))
    assert e.value.code == -2
    # an input that straddles the end of an earlier op's outputs
    with pytest.raises(capi.BpkError) as e:
        build(((x, w4, y), {}), ((y[:, 32:544], w4, torch.zeros(1, 64, device="cuda")), {}))
    assert e.value.code == -2 and "part of the outputs" in str(e.value)
    # two ops that write the same buffer with nothing ordering them: fine as two launches, refused as one
    ch = build(((x, w4, y), {}), ((x, w6, y), {}))
    ch.run(0, 1)
    ch.run(1, 1)
    with pytest.raises(capi.BpkError) as e:
        ch.run(0, 2)
    assert e.value.code == -2 and "orders" in str(e.value)
    torch.cuda.synchronize()
    ch.status()
    # misaligned x
    xx = torch.zeros(1, 516, device="cuda")
    with pytest.raises(capi.BpkError) as e:
        build(((xx[:, 1:513], w4, y), {}))
    assert e.value.code == -4
    # Q5_K is not served
    raw, packed, w5 = gpu.make_weight(13, 64, 512, seed=4)
    with pytest.raises(capi.BpkError) as e:
        build(((x, w5, y), {}))
    assert e.value.code == -1
    # a launch of more ops than a launch walks, and a range outside the chain
    ch = build(((x, w4, y), {}))
    with pytest.raises(capi.BpkError):
        ch.run(0, 2)
    with pytest.raises(capi.BpkError):
        ch.run(1, 1)
