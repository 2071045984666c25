"""Seeded synthetic GGUF k-quant superblocks and model shape tables.

The generators build raw (unpadded) GGUF rows from the *decoded* fields, i.e.
they draw the 6-bit scales, the quants and the fp16 super-scales and then pack
them the way the format stores them, so a test can check a dequantiser against
the drawn fields directly.

Distributions (the benchmark's workload definition):
  Q4_K  4-bit quants uniform 0..15; 8 scales and 8 mins uniform 0..63;
        d, dmin = fp16(|N(0, sigma)|), sigma = 0.01
  Q6_K  6-bit stored quants uniform 0..63 (the -32 is applied on decode);
        16 int8 scales uniform -64..63; d = fp16(|N(0, sigma)|)
PRNG: numpy PCG64 seeded with the given integer.
"""
from __future__ import annotations

import numpy as np

Q4_K = 12
Q6_K = 14
QK_K = 256
Q5_K = 13
BLOCK_BYTES = {Q4_K: 144, Q5_K: 176, Q6_K: 210}
SIGMA = 0.01


def n_blocks(K: int) -> int:
    return (K + QK_K - 1) // QK_K


def row_stride_words(type_: int, K: int) -> int:
    """Words per packed row: Q4_K 36 per block, Q6_K 210*nb bytes rounded up to 4."""
    return (n_blocks(K) * BLOCK_BYTES[type_] + 3) // 4


def pack_rows(type_: int, raw: np.ndarray, N: int, K: int) -> np.ndarray:
    """Raw GGUF rows -> padded u32 rows (zero pad bytes), as uploaded to the GPU."""
    rb = n_blocks(K) * BLOCK_BYTES[type_]
    rs = row_stride_words(type_, K)
    out = np.zeros((N, rs * 4), dtype=np.uint8)
    out[:, :rb] = np.ascontiguousarray(raw, dtype=np.uint8).reshape(N, rb)
    return out.reshape(-1).view(np.uint32)


def q4k_fields(rng: np.random.Generator, N: int, nb: int):
    d = np.abs(rng.normal(0.0, SIGMA, size=(N, nb))).astype(np.float16)
    dmin = np.abs(rng.normal(0.0, SIGMA, size=(N, nb))).astype(np.float16)
    sc = rng.integers(0, 64, size=(N, nb, 8), dtype=np.uint8)
    mn = rng.integers(0, 64, size=(N, nb, 8), dtype=np.uint8)
    q = rng.integers(0, 16, size=(N, nb, 256), dtype=np.uint8)
    return d, dmin, sc, mn, q


def q4k_encode(d, dmin, sc, mn, q) -> np.ndarray:
    """Decoded fields -> raw 144-byte superblocks, shape (N, nb, 144)."""
    N, nb = d.shape
    blk = np.zeros((N, nb, 144), dtype=np.uint8)
    blk[..., 0:2] = d.reshape(N, nb, 1).view(np.uint8)
    blk[..., 2:4] = dmin.reshape(N, nb, 1).view(np.uint8)
    lo_sc, hi_sc = sc[..., :4], sc[..., 4:]
    lo_mn, hi_mn = mn[..., :4], mn[..., 4:]
    blk[..., 4:8] = lo_sc | ((hi_sc >> 4) << 6)
    blk[..., 8:12] = lo_mn | ((hi_mn >> 4) << 6)
    blk[..., 12:16] = (hi_sc & 15) | ((hi_mn & 15) << 4)
    # element sb*32+i lives in byte (sb//2)*32+i, low nibble for even sb
    qq = q.reshape(N, nb, 4, 2, 32)
    blk[..., 16:144] = (qq[:, :, :, 0, :] | (qq[:, :, :, 1, :] << 4)).reshape(N, nb, 128)
    return blk


def q4k_decode_f64(d, dmin, sc, mn, q) -> np.ndarray:
    """Exact real value of every weight in float64: d*sc*q - dmin*mn."""
    N, nb = d.shape
    dd = d.astype(np.float64)[..., None, None]
    mm = dmin.astype(np.float64)[..., None, None]
    qq = q.reshape(N, nb, 8, 32).astype(np.float64)
    w = dd * sc.astype(np.float64)[..., None] * qq - mm * mn.astype(np.float64)[..., None]
    return w.reshape(N, nb * 256)


def q5k_fields(rng: np.random.Generator, N: int, nb: int):
    d, dmin, sc, mn, _ = q4k_fields(rng, N, nb)
    q = rng.integers(0, 32, size=(N, nb, 256), dtype=np.uint8)
    return d, dmin, sc, mn, q


def q5k_encode(d, dmin, sc, mn, q) -> np.ndarray:
    """Decoded fields -> raw 176-byte superblocks: the Q4_K header, 32 bytes of fifth bits (bit sb of
    byte i belongs to element i of sub-block sb), then the Q4_K nibble bytes."""
    N, nb = d.shape
    low = q4k_encode(d, dmin, sc, mn, q & 15)
    blk = np.zeros((N, nb, 176), dtype=np.uint8)
    blk[..., 0:16] = low[..., 0:16]
    hi = (q >> 4).reshape(N, nb, 8, 32)
    qh = np.zeros((N, nb, 32), dtype=np.uint8)
    for sb in range(8):
        qh |= hi[:, :, sb, :] << sb
    blk[..., 16:48] = qh
    blk[..., 48:176] = low[..., 16:144]
    return blk


def q6k_fields(rng: np.random.Generator, N: int, nb: int):
    d = np.abs(rng.normal(0.0, SIGMA, size=(N, nb))).astype(np.float16)
    sc = rng.integers(-64, 64, size=(N, nb, 16), dtype=np.int8)
    q = rng.integers(0, 64, size=(N, nb, 256), dtype=np.uint8)  # stored value
    return d, sc, q


def q6k_encode(d, sc, q) -> np.ndarray:
    """Decoded fields -> raw 210-byte superblocks, shape (N, nb, 210)."""
    N, nb = d.shape
    blk = np.zeros((N, nb, 210), dtype=np.uint8)
    # element 128h + 32t + l: t=0,2 share ql[64h+l] (low, high nibble),
    # t=1,3 share ql[64h+32+l]; bits 2t..2t+1 of qh[32h+l] hold the top two bits
    v = q.reshape(N, nb, 2, 4, 32)
    lo, hi = v & 15, v >> 4
    ql = np.zeros((N, nb, 2, 64), dtype=np.uint8)
    ql[..., 0:32] = lo[:, :, :, 0, :] | (lo[:, :, :, 2, :] << 4)
    ql[..., 32:64] = lo[:, :, :, 1, :] | (lo[:, :, :, 3, :] << 4)
    qh = hi[:, :, :, 0, :] | (hi[:, :, :, 1, :] << 2) | (hi[:, :, :, 2, :] << 4) | (hi[:, :, :, 3, :] << 6)
    blk[..., 0:128] = ql.reshape(N, nb, 128)
    blk[..., 128:192] = qh.reshape(N, nb, 64)
    blk[..., 192:208] = sc.view(np.uint8)
    blk[..., 208:210] = d.reshape(N, nb, 1).view(np.uint8)
    return blk


def q6k_decode_f64(d, sc, q) -> np.ndarray:
    """Exact real value: d * scale[16-element group] * (q - 32)."""
    N, nb = d.shape
    dd = d.astype(np.float64)[..., None, None]
    qq = q.reshape(N, nb, 16, 16).astype(np.float64) - 32.0
    w = dd * sc.astype(np.float64)[..., None] * qq
    return w.reshape(N, nb * 256)


def make_raw(type_: int, N: int, K: int, seed: int = 0) -> np.ndarray:
    """Raw GGUF bytes of an N x K matrix, shape (N, nb*block_bytes) uint8."""
    rng = np.random.default_rng(seed)
    nb = n_blocks(K)
    if type_ == Q4_K:
        blk = q4k_encode(*q4k_fields(rng, N, nb))
    elif type_ == Q5_K:
        blk = q5k_encode(*q5k_fields(rng, N, nb))
    elif type_ == Q6_K:
        blk = q6k_encode(*q6k_fields(rng, N, nb))
    else:
        raise ValueError(f"unsupported k-quant type {type_}")
    return blk.reshape(N, -1)


def make_packed(type_: int, N: int, K: int, seed: int = 0) -> np.ndarray:
    return pack_rows(type_, make_raw(type_, N, K, seed), N, K)


# --------------------------------------------------------------------------- #
# model shape tables (N = output rows, K = input columns)
LLAMA3_8B = {
    "n_layers": 32,
    "hidden": 4096,
    # name, type, N, K — q|k|v and gate|up are row-concatenated like the
    # reference's fuseKQ does for uniform k-quant models
    "layer": [
        ("qkv", Q4_K, 4096 + 1024 + 1024, 4096),
        ("o", Q4_K, 4096, 4096),
        ("gate_up", Q4_K, 2 * 14336, 4096),
        ("down", Q6_K, 4096, 14336),
    ],
    "layer_unfused": [
        ("q", Q4_K, 4096, 4096), ("k", Q4_K, 1024, 4096), ("v", Q4_K, 1024, 4096),
        ("o", Q4_K, 4096, 4096), ("gate", Q4_K, 14336, 4096), ("up", Q4_K, 14336, 4096),
        ("down", Q6_K, 4096, 14336),
    ],
    "lm_head": ("lm_head", Q6_K, 128256, 4096),
}

QWEN3_30B_A3B = {
    "n_experts": 128,
    "top_k": 8,
    "hidden": 2048,
    "inter": 768,
    "gate_up_type": Q4_K,
    "down_type": Q6_K,
}


def weight_bytes(type_: int, N: int, K: int) -> int:
    """Algorithmic weight bytes (unpadded GGUF size)."""
    return N * n_blocks(K) * BLOCK_BYTES[type_]


def make_packed_device(type_: int, N: int, K: int, seed: int = 0, device="cuda"):
    """Same distributions as make_packed, generated on the GPU with torch's
    Philox generator (for multi-gigabyte benchmark weight sets).  Returns a
    uint8 tensor of N*row_stride_words*4 + 16 bytes (16 zero bytes of slack)."""
    import torch
    g = torch.Generator(device=device).manual_seed(seed)
    nb = n_blocks(K)
    bb = BLOCK_BYTES[type_]
    rs = row_stride_words(type_, K) * 4
    rows = torch.zeros((N, rs), dtype=torch.uint8, device=device)
    blk = torch.randint(0, 256, (N, nb, bb), dtype=torch.uint8, device=device, generator=g)

    def half_scales(cnt):
        v = (torch.randn((N, nb, cnt), device=device, generator=g) * SIGMA).abs().to(torch.float16)
        return v.view(torch.uint8).reshape(N, nb, 2 * cnt)

    if type_ in (Q4_K, Q5_K):
        blk[:, :, 0:4] = half_scales(2)          # 12 scale bytes, the quants (and Q5_K's fifth bits) stay uniform
    elif type_ == Q6_K:
        sc = torch.randint(-64, 64, (N, nb, 16), dtype=torch.int8, device=device, generator=g)
        blk[:, :, 192:208] = sc.view(torch.uint8)
        blk[:, :, 208:210] = half_scales(1)
    else:
        raise ValueError(f"unsupported k-quant type {type_}")
    rows[:, : nb * bb] = blk.reshape(N, nb * bb)
    return torch.cat([rows.reshape(-1), torch.zeros(16, dtype=torch.uint8, device=device)])
