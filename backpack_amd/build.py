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
# are, so such a file must compile without any register spill or scratch use, and
# its generated code is read: see check_ring_registers.
NO_SPILL_MARKER = "KQ_REQUIRES_NO_SPILL"

# The compiler the hand-waited kernels were validated with on the GPU (first line of `hipcc --version`, up to
# the build number).  Another compiler may place registers differently; the checks below still run, but the
# GPU parity tests (tests/test_gpu_parity.py::test_matmul_vs_oracle and test_gemv_stream_shapes, which between
# them reach every instantiation of the lanes-along-K kernels) have not been run against its code.
VALIDATED_HIPCC = "HIP version: 7.2.26015"


def hipcc_version() -> str:
    try:
        r = subprocess.run([HIPCC, "--version"], capture_output=True, text=True)
        return r.stdout.splitlines()[0].strip() if r.stdout else ""
    except OSError:
        return ""


def check_compiler() -> None:
    """Refuses a compiler other than the validated one unless BPK_ALLOW_UNVALIDATED_HIPCC=1 (then it warns);
    BPK_TRACKED_LOADS=1 builds the hand-waited kernels with ordinary compiler-tracked loads instead."""
    v = hipcc_version()
    if v.startswith(VALIDATED_HIPCC) or os.environ.get("BPK_TRACKED_LOADS") == "1":
        return
    msg = (f"hipcc reports '{v}', the hand-waited decode kernels were validated with '{VALIDATED_HIPCC}*'. "
           "Run the GPU parity tests after building; set BPK_ALLOW_UNVALIDATED_HIPCC=1 to build anyway, or "
           "BPK_TRACKED_LOADS=1 to build those kernels with compiler-tracked loads (slower, no such dependence).")
    if os.environ.get("BPK_ALLOW_UNVALIDATED_HIPCC") == "1":
        sys.stderr.write("warning: " + msg + "\n")
    else:
        raise RuntimeError(msg)


_REG = re.compile(r"\bv\[(\d+):(\d+)\]|\bv(\d+)\b")


def _regs(text: str) -> set[int]:
    out: set[int] = set()
    for a, b, c in _REG.findall(text):
        if c:
            out.add(int(c))
        else:
            out.update(range(int(a), int(b) + 1))
    return out


def check_ring_registers(asm_path: str) -> list[str]:
    """In every function of the generated code, the vector registers written by the marked ring loads must be
    exactly those the marked ring waits pass through: a register that was copied between its load and its
    wait (a split live range, a copy on a back edge) leaves a load whose register no wait names, or a wait
    on a register no load writes."""
    problems = []
    func, loads, waits = None, set(), set()

    def close():
        if func and (loads or waits) and loads != waits:
            problems.append(f"{func}: ring loads write v{sorted(loads - waits)} that no ring wait covers, "
                            f"ring waits name v{sorted(waits - loads)} that no ring load writes")
    with open(asm_path) as f:
        for line in f:
            m = re.match(r"^([A-Za-z_][\w.$]*):\s*(;.*)?$", line)
            if m and not m.group(1).startswith(".L"):
                close()
                func, loads, waits = m.group(1), set(), set()
                continue
            if "; ringld" in line:
                # global_load_dwordx4 v[a:b], v[c:d], off ; ringld  -> the first operand is the destination
                dest = line.split(",")[0]
                loads |= _regs(dest.split(None, 1)[1] if len(dest.split(None, 1)) > 1 else "")
            elif "; ringwait" in line:
                waits |= _regs(line.split("; ringwait", 1)[1])
    close()
    return problems


# A source that carries this marker keeps its hand-waited loads in straight-line code: every kernel's listing, read top
# to bottom, is the order of execution as far as the ring is concerned (loads ahead of the loop, then wait, use and
# refill of one slot after another in the loop's body).  Its generated code also passes check_ring_order.
STRAIGHT_LINE_MARKER = "KQ_RING_STRAIGHT_LINE"


def check_ring_order(asm_path: str) -> list[str]:
    """Reads every function top to bottom with the set of registers that have a marked load in flight: a marked
    wait may only name registers of that set (and takes them out), a marked load may not write a register still
    in it, and no other instruction may mention one (a copy, a spill, a reuse as a temporary).  Stricter than
    check_ring_registers, which compares sets per function; only meaningful for listings whose text order is
    the order of execution."""
    problems = []
    func, flying, n = None, set(), 0
    with open(asm_path) as f:
        for line in f:
            n += 1
            m = re.match(r"^([A-Za-z_][\w.$]*):\s*(;.*)?$", line)
            if m and not m.group(1).startswith(".L"):
                func, flying = m.group(1), set()
                continue
            if not line.startswith("\t") or line.lstrip().startswith((".", ";")):
                continue
            code = line.split(";", 1)[0]
            if "; ringld" in line:
                parts = code.split(",")
                dest = _regs(parts[0].split(None, 1)[1] if len(parts[0].split(None, 1)) > 1 else "")
                if dest & flying:
                    problems.append(f"{func}, line {n}: v{sorted(dest & flying)} loaded again before its wait")
                addr = _regs(",".join(parts[1:]))
                if addr & flying:
                    problems.append(f"{func}, line {n}: a load's address uses v{sorted(addr & flying)}, which is in flight")
                flying |= dest
            elif "; ringwait" in line:
                named = _regs(line.split("; ringwait", 1)[1])
                if named - flying:
                    problems.append(f"{func}, line {n}: a wait names v{sorted(named - flying)}, which no load in flight writes")
                flying -= named
            elif _regs(code) & flying:
                problems.append(f"{func}, line {n}: '{code.strip()[:60]}' touches v{sorted(_regs(code) & flying)} with a load in flight")
    return problems


# A source that carries this marker has kernels whose arguments are scalars and few enough to arrive in scalar
# registers with the wave (kernel-argument preloading, up to 16 dwords); kernels with struct arguments are unaffected.
PRELOAD_MARKER = "KQ_KERNARG_PRELOAD"


def _compile(src: str) -> str:
    base = os.path.basename(src).replace(".hip", "")
    obj = os.path.join(OBJ, base + ".o")
    extra = os.environ.get("BPK_EXTRA_FLAGS", "").split()   # experiments only
    with open(src) as f:
        text = f.read()
    guarded = NO_SPILL_MARKER in text
    if PRELOAD_MARKER in text and os.environ.get("BPK_NO_KERNARG_PRELOAD") != "1":
        extra += ["-mllvm", "-amdgpu-kernarg-preload-count=16"]
    tracked = os.environ.get("BPK_TRACKED_LOADS") == "1"
    if guarded:
        extra.append("-Rpass-analysis=kernel-resource-usage")
        if tracked:
            extra.append("-DKQ_TRACKED_LOADS")
    cmd = [HIPCC, *FLAGS, *extra, "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    lines = r.stderr.splitlines()
    if guarded:
        # (scalar registers spilled into lanes of a reserved vector register are harmless here: no register
        # with a load in flight moves; vector spills and scratch memory are what must not happen)
        bad = [l for l in lines if re.search(r"(VGPRs Spill|ScratchSize[^:]*):\s*[1-9]", l)]
        if bad and r.returncode == 0 and not tracked:
            raise RuntimeError(f"{src} must not spill registers (hand-waited loads):\n" + "\n".join(bad[:8]))
        lines = [l for l in lines if "kernel-resource-usage" not in l and not re.match(r"^\s*\d*\s*\|", l)]
    err = "\n".join(l for l in lines if "packed-fp32-ops" not in l)
    if r.returncode:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    if guarded and not tracked:
        # the device code as text, for the register check
        asm = os.path.join(OBJ, base + ".s")
        ra = subprocess.run([HIPCC, *FLAGS, *[e for e in extra if not e.startswith("-Rpass")], "-S", "--cuda-device-only",
                             src, "-o", asm], capture_output=True, text=True)
        if ra.returncode:
            raise RuntimeError(f"hipcc -S failed on {src}:\n{ra.stderr}")
        problems = check_ring_registers(asm)
        if STRAIGHT_LINE_MARKER in text:
            problems += check_ring_order(asm)
        if problems:
            raise RuntimeError(f"{src}: registers of hand-waited loads were moved between load and wait:\n" +
                               "\n".join(problems[:8]))
    return obj


def build_library(jobs: int = 8) -> str:
    os.makedirs(OBJ, exist_ok=True)
    check_compiler()
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
