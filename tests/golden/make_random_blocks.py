"""Writes tests/golden/random_blocks.npz: rows of uniformly random bytes (every
field of the block exercised, fp16 scales forced finite but including
subnormals) with the COMPILED REFERENCE's dequantised output and packed layout.

    make -C oracle && python tests/golden/make_random_blocks.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import kqo  # noqa: E402


def finite_fp16(raw, offs, bb):
    """Clear one exponent bit of any inf/NaN fp16 at byte offsets `offs`."""
    blocks = raw.reshape(raw.shape[0], -1, bb)
    for o in offs:
        hi = blocks[:, :, o + 1]
        bad = (hi & 0x7C) == 0x7C
        hi[bad] &= 0xBF
    return raw


def main():
    assert kqo.ref() is not None
    rng = np.random.default_rng(20240)
    out = {}
    for name, type_, bb, offs, N, K in (("q4k", kqo.Q4_K, 144, (0, 2), 6, 768),
                                        ("q6k", kqo.Q6_K, 210, (208,), 5, 768)):
        nb = K // 256
        raw = rng.integers(0, 256, size=(N, nb * bb), dtype=np.uint8)
        # a few subnormal and zero super-scales
        blocks = raw.reshape(N, nb, bb)
        for o in offs:
            blocks[0, 0, o + 1] &= 0x83   # exponent field 0 -> subnormal
            blocks[1, 1, o:o + 2] = 0     # exactly zero
        raw = finite_fp16(raw, offs, bb)
        packed, nbr, rs = kqo.ref_pack(type_, raw, N, K)
        out[f"{name}/raw"] = raw
        out[f"{name}/packed"] = packed
        out[f"{name}/desc"] = np.array([type_, N, K, nbr, rs], dtype=np.int64)
        out[f"{name}/deq_bits"] = kqo.ref_dequant(type_, raw, N, K).view(np.uint32)
    np.savez_compressed(os.path.join(HERE, "random_blocks.npz"), **out)
    print("wrote random_blocks.npz")


if __name__ == "__main__":
    main()
