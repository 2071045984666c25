"""Writes tests/golden/recipes.npz: the reference's eleven Q4_K/Q5_K/Q6_K known-answer
cases with inputs regenerated from their closed forms and expected outputs
computed by the COMPILED REFERENCE (oracle/_ref/libbp_ref.so -> dequant_kquant)
followed by the test-suite's sequential fp32 dot, written here as a plain
float32 loop that shares no code with the oracle.

Run in the container that has the reference checkout:
    make -C oracle && python tests/golden/make_recipes.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, os.path.dirname(HERE))

from oracle import kqo  # noqa: E402
import recipes  # noqa: E402


def seq_dot(x, w, b0):
    a = np.float32(b0)
    for k in range(len(x)):
        a = np.float32(a + np.float32(x[k] * w[k]))
    return a


def main():
    assert kqo.ref() is not None, "build oracle/_ref first (make -C oracle)"
    out = {}
    for name, r in recipes.build(kqo).items():
        N, K = r["N"], r["K"]
        deq = kqo.ref_dequant(r["type"], r["raw"], N, K)
        packed, nb, rs = kqo.ref_pack(r["type"], r["raw"], N, K)
        out[f"{name}/raw"] = r["raw"]
        out[f"{name}/packed"] = packed
        out[f"{name}/desc"] = np.array([r["type"], r["M"], N, K, nb, rs], dtype=np.int64)
        out[f"{name}/deq"] = deq
        if "rows" in r:
            rows = np.array(r["rows"], dtype=np.int32)
            out[f"{name}/rows"] = rows
            out[f"{name}/expected"] = deq[rows]
        else:
            x, bias = r["x"], r["bias"]
            exp = np.zeros((r["M"], N), dtype=np.float32)
            for m in range(r["M"]):
                for n in range(N):
                    exp[m, n] = seq_dot(x[m], deq[n], bias[n])
            out[f"{name}/x"] = x
            out[f"{name}/bias"] = bias
            out[f"{name}/expected"] = exp
        out[f"{name}/tol"] = np.array([r["atol"], r["rtol"]], dtype=np.float32)
    np.savez_compressed(os.path.join(HERE, "recipes.npz"), **out)
    print("wrote recipes.npz with", len(out), "arrays")


if __name__ == "__main__":
    main()
