"""GGUF file -> device weights -> matmul, through the C ABI: the bytes a file
holds must come out of the GPU bit for bit, and a matmul on weights loaded that
way must meet the same criteria as one on weights uploaded from memory."""
import numpy as np
import pytest

import gguf_writer as gw

pytestmark = pytest.mark.gpu

Q4_K, Q6_K = 12, 14


@pytest.fixture(scope="module")
def gpu():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from backpack_amd import capi
    capi.check(capi.lib().bpk_init(0))
    import gpu_util
    return gpu_util


def test_weights_from_file_match_the_file_and_the_oracle(gpu, kqo, tmp_path):
    from backpack_amd import kquant, synth
    from backpack_amd.gguf import GGUFFile
    K = 1024
    parts = {"blk.0.attn_q.weight": (Q4_K, 96, 11), "blk.0.attn_k.weight": (Q4_K, 32, 12),
             "blk.0.attn_v.weight": (Q4_K, 32, 13), "output.weight": (Q6_K, 70, 14)}
    raws = {n: synth.make_raw(t, N, K, seed) for n, (t, N, seed) in parts.items()}
    tensors = [(n, (K, parts[n][1]), parts[n][0], raws[n].tobytes()) for n in parts]
    tensors.insert(2, ("blk.0.attn_norm.weight", (K,), 0, np.ones(K, np.float32).tobytes()))
    path = str(tmp_path / "w.gguf")
    gw.write(path, [("general.architecture", gw.STRING, "qwen3")], tensors)
    print("gguf weights", path, flush=True)
    with GGUFFile(path) as g:
        qkv = kquant.from_gguf(g, ["blk.0.attn_q.weight", "blk.0.attn_k.weight", "blk.0.attn_v.weight"])
        head = kquant.from_gguf(g, "output.weight")
    # the mapping is gone; the device copies must stand on their own
    assert (qkv.type, qkv.N, qkv.K, head.type, head.N) == (Q4_K, 160, K, Q6_K, 70)
    raw_qkv = np.concatenate([raws[n].reshape(-1) for n in list(parts)[:3]])
    for w, raw, type_ in ((qkv, raw_qkv, Q4_K), (head, raws["output.weight"], Q6_K)):
        got = kquant.dequant_rows(w).cpu().numpy()
        want = kqo.dequant(type_, raw, w.N, K)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
        packed = synth.pack_rows(type_, raw, w.N, K)
        for M in (1, 5):
            X = np.random.default_rng(M).standard_normal((M, K)).astype(np.float32)
            y = kquant.matmul(gpu.dev(X), w).cpu().numpy()
            gpu.check_matmul(kqo, type_, y, X, packed, w.N, K, label=f"gguf {type_} M={M}")


@pytest.mark.parametrize("type_,K,N_parts", [(Q6_K, 768, (50000, 3093, 67000)), (Q4_K, 2048, (40000, 30000))])
def test_upload_larger_than_the_stage_keeps_every_row(gpu, kqo, tmp_path, type_, K, N_parts):
    """The upload moves rows in 32 MiB pieces through two pinned buffers; rows on either side of every
    piece boundary, of every part boundary and at the ends must arrive intact (Q6_K with an odd block
    count also exercises the padded row stride)."""
    from backpack_amd import capi, kquant
    from backpack_amd.gguf import GGUFFile
    rng = np.random.default_rng(3)
    nb = K // 256
    row_bytes = nb * (144 if type_ == Q4_K else 210)
    raws = []
    for N in N_parts:
        r = rng.integers(0, 256, size=(N, row_bytes), dtype=np.uint8)
        blocks = r.reshape(N, nb, -1)
        if type_ == Q4_K:       # keep the fp16 scale fields finite
            blocks[:, :, 1] &= 0x3B
            blocks[:, :, 3] &= 0x3B
        else:
            blocks[:, :, 209] &= 0x3B
        raws.append(r)
    names = [f"part{i}.weight" for i in range(len(N_parts))]
    path = str(tmp_path / "big.gguf")
    gw.write(path, [], [(n, (K, r.shape[0]), type_, r.tobytes()) for n, r in zip(names, raws)])
    print("big upload", type_, K, N_parts, flush=True)
    with GGUFFile(path) as g:
        w = kquant.from_gguf(g, names)
    raw = np.concatenate(raws)
    N = raw.shape[0]
    _, rs = capi.layout(type_, K)
    per_piece = (32 << 20) // (rs * 4)
    assert N * rs * 4 > 2 * (32 << 20), "the case must span more than two pieces"
    marks = {0, N - 1}
    for b in list(range(per_piece, N, per_piece)) + list(np.cumsum(N_parts)[:-1]):
        marks.update({int(b) - 1, int(b)})
    rows = np.array(sorted(marks), dtype=np.int32)
    got = kquant.dequant_rows(w, gpu.dev(rows)).cpu().numpy()
    want = kqo.dequant(type_, np.ascontiguousarray(raw[rows]), len(rows), K)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # and windows of 4096 rows spread over the whole matrix
    every = kquant.dequant_rows(w)
    step = 4096
    for r0 in range(0, N, N // 7):
        blk = kqo.dequant(type_, np.ascontiguousarray(raw[r0:r0 + step]), min(step, N - r0), K)
        assert np.array_equal(every[r0:r0 + step].cpu().numpy().view(np.uint32), blk.view(np.uint32))
