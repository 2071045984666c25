"""Builds backpack_amd/libbpk_kquant.so from backpack_amd/csrc/*.hip with hipcc
for gfx950.  Run as `python -m backpack_amd.build`; hipcc cross-compiles, so no
GPU is needed."""
from __future__ import annotations

import concurrent.futures as cf
import glob
import os
import re
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "build")
LIB = os.path.join(HERE, "libbpk_kquant.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-fno-gpu-rdc", "-Wall", "-Wno-unused-command-line-argument",
    # keep the compiler from forming packed-fp32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


# A source that carries this marker issues global loads from inline asm and waits
# for them by hand; that is only sound while the loaded registers stay where they
# are, so such a file must compile without any register spill or scratch use.
NO_SPILL_MARKER = "KQ_REQUIRES_NO_SPILL"


def _compile(src: str) -> str:
    obj = os.path.join(OBJ, os.path.basename(src).replace(".hip", ".o"))
    extra = os.environ.get("BPK_EXTRA_FLAGS", "").split()   # experiments only
    with open(src) as f:
        guarded = NO_SPILL_MARKER in f.read()
    if guarded:
        extra.append("-Rpass-analysis=kernel-resource-usage")
    cmd = [HIPCC, *FLAGS, *extra, "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    lines = r.stderr.splitlines()
    if guarded:
        # (scalar registers spilled into lanes of a reserved vector register are harmless here: no register
        # with a load in flight moves; vector spills and scratch memory are what must not happen)
        bad = [l for l in lines if re.search(r"(VGPRs Spill|ScratchSize[^:]*):\s*[1-9]", l)]
        if bad and r.returncode == 0:
            raise RuntimeError(f"{src} must not spill registers (hand-waited loads):\n" + "\n".join(bad[:8]))
        lines = [l for l in lines if "kernel-resource-usage" not in l and not re.match(r"^\s*\d*\s*\|", l)]
    err = "\n".join(l for l in lines if "packed-fp32-ops" not in l)
    if r.returncode:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build_library(jobs: int = 8) -> str:
    os.makedirs(OBJ, exist_ok=True)
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    with cf.ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(_compile, srcs))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    return LIB


if __name__ == "__main__":
    print(build_library())
