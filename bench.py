#!/usr/bin/env python3
"""Benchmark of the k-quant decode path on one MI355X.

A step is one pass of the Llama-3-8B-shaped decode layer set at M = 1 in the
Q4_K_M mix: per layer q|k|v (Q4_K 6144x4096), o (Q4_K 4096x4096), gate|up
(Q4_K 28672x4096), down (Q6_K 4096x14336), 32 layers with distinct weights,
plus a Q6_K lm_head 128256x4096 — 129 launches reading 4 841 250 816 weight
bytes, far beyond the 256 MB last-level cache, all resident in HBM before the
timed region.  Launches go to one stream in order; by default the step is
recorded once into a HIP graph and replayed, like the reference's pre-recorded
per-token command buffer (runtime/model_runner.cpp:5725-5759).

Prints ONE JSON line.  `value` is weight+activation bytes of the step divided by
wall time.  `roofline` covers the dominant kernel (the Q4_K GEMV on gate|up,
44 % of the bytes), timed with HIP events on the launch stream over its own
region of 32 distinct matrices.  `cpu_baseline` times the reference's CPU path
(dequantise to fp32, sequential fp32 dot) on a bounded sample on the host.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, published
COPY_RATE_GBS = 6350.0          # what a plain streaming read reaches on this pool's MI355X (6.0-6.7 TB/s measured)
METRIC = "Q4_K M=1 matvec HBM GB/s (% of peak); M=2048 dequant-GEMM TFLOPS (% MFMA)"

# HBM bytes per launch of the dominant kernel are NOT measured in this run: they are read from the committed
# rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE summary named below (FETCH_SIZE x 2.000 KiB + WRITE_SIZE x 1.000 KiB, the
# factors being what the same counters read for a 256 MiB copy kernel), from its line
# "traffic_bytes <kernel family> <shape> <bytes>"; no such line for the kernel that ran -> null.
TRAFFIC_PROFILE = "profiles/decode_gemv_hbm_traffic_pmc.txt"


def profiled_traffic(kernel, shape):
    try:
        with open(os.path.join(ROOT, TRAFFIC_PROFILE)) as f:
            for line in f:
                t = line.split()
                if len(t) == 4 and t[0] == "traffic_bytes" and t[1] == kernel and t[2] == shape:
                    return int(t[3])
    except OSError:
        pass
    return None


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of replaying a HIP graph")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--layers", type=int, default=32, help="layers in the set (32 = the named workload)")
    ap.add_argument("--prefill", action="store_true",
                    help="(kept for old command lines: the M=2048 / M=512 prefill GEMM leg now runs by default)")
    ap.add_argument("--no-prefill", action="store_true", help="skip the prefill GEMM leg")
    ap.add_argument("--verify", action="store_true", help="(kept for old command lines: the verify leg runs by default)")
    ap.add_argument("--moe", action="store_true", help="(kept for old command lines: the MoE leg runs by default)")
    ap.add_argument("--no-verify", action="store_true",
                    help="skip the layer set at M = 2, 4, 8, 16 (speculative-decode verify batches)")
    ap.add_argument("--no-moe", action="store_true",
                    help="skip the Qwen3-30B-A3B-shaped routed-expert FFN at T = 1 and T = 256")
    ap.add_argument("--all", action="store_true", help="also --fused")
    ap.add_argument("--no-config0", action="store_true", help="skip the single 4096x4096 matvec (cold / hot)")
    ap.add_argument("--fused", action="store_true",
                    help="also time the layer set with RMSNorm folded into qkv and act*mul + residual into down")
    ap.add_argument("--load", action="store_true",
                    help="also write a GGUF file of Q4_K / Q6_K matrices and time file -> device weights")
    ap.add_argument("--gemm-tile", type=int, default=0,
                    help="force the prefill GEMM tile (0 = the library's own choice)")
    ap.add_argument("--gemm-split", type=int, default=0,
                    help="256-tile prefill GEMM: 1 = one tile per workgroup, 2 = equal shares per CU (0 = automatic)")
    ap.add_argument("--prefill-only", action="store_true",
                    help="run only the M=2048 prefill GEMM leg and print its figures (for profiling)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="first run one 256 MiB device-to-device copy kernel: under rocprofv3 --pmc its "
                         "FETCH_SIZE / WRITE_SIZE readings give the counters' scale")
    return ap.parse_args()


def build_layer_set(n_layers):
    import torch
    from backpack_amd import kquant, synth
    spec = synth.LLAMA3_8B
    mats = []   # (name, KQuantPacked, x, y)
    xs, ys = {}, {}
    seed = 0
    for layer in range(n_layers):
        for name, type_, N, K in spec["layer"]:
            data = synth.make_packed_device(type_, N, K, seed=seed)
            seed += 1
            nb, rs = synth.n_blocks(K), synth.row_stride_words(type_, K)
            w = kquant.KQuantPacked(data, type_, N, K, rs, nb)
            if K not in xs:
                g = torch.Generator(device="cuda").manual_seed(1000 + K)
                xs[K] = torch.randn(1, K, device="cuda", generator=g)
            if N not in ys:
                ys[N] = torch.empty(1, N, device="cuda")
            mats.append((name, w, xs[K], ys[N]))
    name, type_, N, K = spec["lm_head"]
    data = synth.make_packed_device(type_, N, K, seed=seed)
    w = kquant.KQuantPacked(data, type_, N, K, synth.row_stride_words(type_, K), synth.n_blocks(K))
    ys[N] = torch.empty(1, N, device="cuda")
    mats.append((name, w, xs[K], ys[N]))
    return mats


def algorithmic_bytes(mats, M=1):
    from backpack_amd import synth
    wb = sum(synth.weight_bytes(w.type, w.N, w.K) for _, w, _, _ in mats)
    act = sum((w.K + w.N) * 4 * M for _, w, _, _ in mats)
    return wb, act


def run_region(mats, steps, warmup, use_graph, per_step=None):
    """Times `steps` passes over mats with HIP events on the launch stream.  per_step: a list that receives
    the duration of every pass of a second, separately timed round of `steps` passes (an event pair each)."""
    import torch
    from backpack_amd import kquant

    def one_pass():
        for _, w, x, y in mats:
            kquant.matmul(x, w, out=y)

    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        one_pass()
        stream.synchronize()
        if use_graph:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                one_pass()
            step = graph.replay
        else:
            step = one_pass
        for _ in range(warmup):
            step()
        stream.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        e0.record(stream)
        for _ in range(steps):
            step()
        e1.record(stream)
        stream.synchronize()
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        if per_step is not None:
            evs = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
            evs[0].record(stream)
            for i in range(steps):
                step()
                evs[i + 1].record(stream)
            stream.synchronize()
            per_step.extend(evs[i].elapsed_time(evs[i + 1]) * 1e-3 for i in range(steps))
    return e0.elapsed_time(e1) * 1e-3, wall


def cpu_baseline():
    """The reference's CPU path on a bounded sample of the same workload (half of
    the layers + lm_head, about ten seconds of work), single thread, then the
    same rows split over all host threads."""
    import concurrent.futures as cf

    import numpy as np
    from backpack_amd import synth
    from oracle import kqo

    use_ref = kqo.ref() is not None
    spec = synth.LLAMA3_8B
    n_layers = 16
    sample = list(spec["layer"]) * n_layers + [spec["lm_head"]]
    rng = np.random.default_rng(0)
    total_bytes, t_deq, t_dot = 0, 0.0, 0.0
    # every core this job may use: the scheduler affinity, cut down to the control group's CPU quota where
    # one is set (threads beyond it would only take turns); the host's own count is reported beside it
    try:
        cores = len(os.sched_getaffinity(0))
    except AttributeError:
        cores = os.cpu_count() or 1
    quota = None
    try:
        with open("/sys/fs/cgroup/cpu.max") as f:
            q, period = f.read().split()[:2]
            if q != "max":
                quota = max(1, int(int(q) / int(period)))
    except (OSError, ValueError):
        pass
    if quota:
        cores = min(cores, quota)
    cores = max(1, min(cores, 256))
    t_par = 0.0
    for i, (name, type_, N, K) in enumerate(sample):
        # the CPU leg only needs bytes of the right shape: uniform random
        # blocks with fixed small fp16 super-scales (no NaNs), cheap to make
        bb = synth.BLOCK_BYTES[type_]
        nb = synth.n_blocks(K)
        raw = rng.integers(0, 256, size=(N, nb, bb), dtype=np.uint8)
        for off in ((0, 2) if type_ == synth.Q4_K else (208,)):
            raw[:, :, off] = 0x1F
            raw[:, :, off + 1] = 0x20
        raw = raw.reshape(N, nb * bb)
        x = rng.standard_normal((1, K)).astype(np.float32)
        _, td, tm = kqo.matmul_timed(type_, x, raw, N, K, use_ref=use_ref)
        t_deq += td
        t_dot += tm
        total_bytes += N * nb * bb
        # all-core leg: contiguous row slabs, one per thread (ctypes drops the GIL)
        slabs = np.array_split(np.arange(N), cores)
        t0 = time.perf_counter()
        with cf.ThreadPoolExecutor(cores) as ex:
            list(ex.map(lambda s: kqo.matmul_timed(type_, x, raw[s[0]:s[-1] + 1], len(s), K, use_ref=use_ref),
                        [s for s in slabs if len(s)]))
        t_par += time.perf_counter() - t0
        del raw
    one = total_bytes / (t_deq + t_dot) / 1e9
    return {
        "value": round(one, 4), "unit": "GB/s", "cores": 1,
        "kind": "reference" if use_ref else "port",
        "sample": f"{n_layers} of the 32 layers (qkv, o, gate_up, down) + lm_head of the same workload, "
                  f"{total_bytes} weight bytes; dequant {t_deq:.2f} s + dot {t_dot:.2f} s",
        "dequant_s": round(t_deq, 3), "dot_s": round(t_dot, 3),
        "all_cores": {"value": round(total_bytes / t_par / 1e9, 4), "unit": "GB/s", "cores": cores,
                      "nproc": os.cpu_count(), "cgroup_cpu_quota": quota,
                      "note": "threads = the cores this job may use (affinity, cut to the cgroup quota)"},
    }


def main():
    args = parse()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: this path has no multi-GPU leg (asked for --gpus {args.gpus}); "
              "it shards by output rows with no exchange, so N GPUs run N independent copies of this "
              "benchmark on 1/N of the rows.", file=sys.stderr)
        sys.exit(2)
    import torch
    from backpack_amd import capi, synth
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    capi.check(capi.lib().bpk_init(0))

    if args.calibrate_copy:
        src = torch.zeros(256 << 20, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        dst.copy_(src)          # one elementwise copy kernel: reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst
        torch.cuda.empty_cache()

    if args.gemm_tile:
        capi.set_option("gemm_tile", args.gemm_tile)
    if args.gemm_split:
        capi.set_option("gemm_split", args.gemm_split)
    mats = build_layer_set(args.layers)
    if args.prefill_only:
        torch.cuda.synchronize()
        print(json.dumps({"prefill": prefill_leg(mats, 2048)}))
        return

    torch.cuda.synchronize()
    wb, act = algorithmic_bytes(mats)
    use_graph = not args.no_graph

    step_s = []
    sec, wall = run_region(mats, args.steps, args.warmup, use_graph, per_step=step_s)
    step_s.sort()
    ms_per_step = sec / args.steps * 1e3
    gbs = (wb + act) / (sec / args.steps) / 1e9

    # dominant kernel: the Q4_K GEMV on gate|up, every layer's own matrix
    dom = [m for m in mats if m[0] == "gate_up"]
    dom_steps = min(max(args.steps, 10), 50)
    dom_pass = []
    dsec, _ = run_region(dom, dom_steps, min(args.warmup, 5), use_graph, per_step=dom_pass)
    dom_pass.sort()
    launches = len(dom) * dom_steps
    dom_w = dom[0][1]
    dom_bytes = synth.weight_bytes(dom_w.type, dom_w.N, dom_w.K) + (dom_w.K + dom_w.N) * 4
    dom_gbs = dom_bytes / (dsec / launches) / 1e9
    dom_kernel = capi.last_kernel()     # the library's name of the kernel family that served these launches
    dom_shape = f"{dom_w.N}x{dom_w.K}"
    traffic = profiled_traffic(dom_kernel, dom_shape)
    roofline = {
        "kernel": f"{dom_kernel} (gate|up {dom_shape} Q4_K, M=1; instantiation: see profiles/decode_layer_set_kernel_trace.txt)",
        "bound": "hbm", "achieved": round(dom_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": round(dom_gbs / HBM_PEAK_GBS, 4),
        "bytes_per_launch": dom_bytes, "us_per_launch": round(dsec / launches * 1e6, 3),
        # per launch, from passes of 32 launches each timed by an event pair
        "us_per_launch_min": round(dom_pass[0] / len(dom) * 1e6, 3),
        "us_per_launch_median": round(dom_pass[len(dom_pass) // 2] / len(dom) * 1e6, 3),
        "launches_timed": launches,
        "traffic": traffic,
        "traffic_source": f"not measured in this run: rocprofv3 --pmc summary {TRAFFIC_PROFILE}, line for {dom_kernel} {dom_shape}",
        "frac_of_measured_copy_rate": round(dom_gbs / COPY_RATE_GBS, 4),
    }

    # per-shape breakdown (extra information, same protocol)
    shapes = {}
    for name in ("qkv", "o", "down", "lm_head"):
        sel = [m for m in mats if m[0] == name]
        reps = 20 * (8 if name == "lm_head" else 1)
        s, _ = run_region(sel, reps, 2, use_graph)
        w = sel[0][1]
        b = synth.weight_bytes(w.type, w.N, w.K) + (w.K + w.N) * 4
        shapes[name] = {"us": round(s / (len(sel) * reps) * 1e6, 2),
                        "GBps": round(b / (s / (len(sel) * reps)) / 1e9, 1)}
    shapes["gate_up"] = {"us": roofline["us_per_launch"], "GBps": roofline["achieved"]}

    out = {
        "metric": METRIC, "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "Llama-3-8B-shaped decode layer set, M=1, Q4_K_M mix "
                               f"({args.layers} layers x [qkv, o, gate_up, down] + lm_head)",
                   "weights": "GGUF Q4_K / Q6_K superblocks, read as packed bytes", "activations": "f32",
                   "accumulation": "f32", "launches_per_step": len(mats), "weight_bytes": wb, "activation_bytes": act,
                   "graph_replay": use_graph},
        "pct_of_hbm_peak": round(gbs / HBM_PEAK_GBS * 100, 2),
        "pct_of_measured_copy_rate": round(gbs / COPY_RATE_GBS * 100, 2),
        "ms_per_step_min": round(step_s[0] * 1e3, 4), "ms_per_step_median": round(step_s[len(step_s) // 2] * 1e3, 4),
        "tokens_per_s_equiv": round(args.steps / sec, 1),
        "host_wall_ms_per_step": round(wall / args.steps * 1e3, 4),
        "roofline": roofline,
        "per_shape": shapes,
    }
    if not args.no_config0:
        out["config0"] = config0_leg()
    if not args.no_verify:
        out["verify"] = verify_leg(mats, wb, use_graph)
    if not args.no_moe:
        out["moe"] = moe_leg()
    if args.fused or args.all:
        out["fused"] = fused_leg(mats, use_graph)
    if args.load:
        out["gguf_load"] = load_leg()
    if not args.no_prefill:
        # the second half of the metric: M=2048 dequant-GEMM TFLOP/s and its fraction of the bf16 MFMA peak
        out["prefill"] = prefill_leg(mats, 2048)
        out["prefill_m512"] = prefill_leg(mats, 512)
        out["gemm_tflops_m2048"] = out["prefill"]["layer_set"]["TFLOPs"]
        out["gemm_pct_of_mfma_peak"] = out["prefill"]["layer_set"]["pct_of_bf16_mfma_peak"]
        out["gemm_accuracy"] = out["prefill"]["accuracy"]
    if not args.no_cpu:
        del mats, dom
        torch.cuda.empty_cache()
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out))


def fused_leg(mats, use_graph):
    """The decode layer set with the dispatches around its matvecs folded in: qkv and gate|up read x through
    RMSNorm, gate|up writes silu(gate)*up directly, o and down add the residual in place.  Timed three ways
    on the same weights: plain matvecs only (what the headline measures), fused (one launch each), and the
    same function as separate launches (norm, act*mul, add beside the matvecs)."""
    import torch
    from backpack_amd import capi, kquant
    hidden = next(w.K for n, w, _, _ in mats if n == "qkv")
    inter = next(w.K for n, w, _, _ in mats if n == "down")
    norm_w = torch.ones(hidden, device="cuda")
    gate_up = next(y for n, _, _, y in mats if n == "gate_up")
    resid = torch.zeros(1, hidden, device="cuda")
    ws = torch.empty(capi.lib().bpk_kq_matmul_fused_workspace_bytes(1, max(w.N for _, w, _, _ in mats), inter),
                     dtype=torch.uint8, device="cuda")

    act = torch.zeros(1, inter, device="cuda")

    def fused_pass():
        # a layer's four matvecs with the five dispatches around them folded in: attn_norm -> qkv,
        # o -> + residual, ffn_norm -> gate|up -> act * up, down -> + residual
        for name, w, x, y in mats:
            if name == "qkv":
                kquant.matmul_fused(x, w, capi.PRO_RMS_NORM, norm_w=norm_w, eps=1e-5, out=y, workspace=ws)
            elif name == "o":
                kquant.matmul_fused(x, w, residual=resid, out=resid, workspace=ws)
            elif name == "gate_up":
                kquant.matmul_fused(x, w, capi.PRO_RMS_NORM, norm_w=norm_w, eps=1e-5, out=act, workspace=ws,
                                    epilogue=capi.EPI_SILU_MUL)
            elif name == "down":
                kquant.matmul_fused(act, w, residual=resid, out=resid, workspace=ws)
            else:
                kquant.matmul(x, w, out=y)

    def timed(one_pass, steps=20, warmup=3):
        stream = torch.cuda.Stream()
        with torch.cuda.stream(stream):
            one_pass()
            stream.synchronize()
            step = one_pass
            if use_graph:
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph, stream=stream):
                    one_pass()
                step = graph.replay
            for _ in range(warmup):
                step()
            stream.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            for _ in range(steps):
                step()
            e1.record(stream)
            stream.synchronize()
        return e0.elapsed_time(e1) / steps

    res = {"plain_ms": round(timed(lambda: [kquant.matmul(x, w, out=y) for _, w, x, y in mats]), 4)}
    res["fused_ms"] = round(timed(fused_pass), 4)
    res["kernel"] = capi.last_kernel()
    capi.set_option("fused_separate", 1)
    try:
        res["separate_ms"] = round(timed(fused_pass), 4)
    finally:
        capi.set_option("fused_separate", 0)
    # The same fused function as chains: one launch per stretch between two attention blocks
    # (o, gate|up, down and the next layer's q|k|v, the last stretch ending in lm_head), 1 + n_layers launches.
    # Every op reads what the op before it wrote (x += o(attn); act; x += down(act); qkv = W n(x)), handed on
    # inside the launch.
    attn = torch.randn(1, hidden, device="cuda") * 0.05
    xres = torch.randn(1, hidden, device="cuda")
    x0 = xres.clone()
    order = [m for m in mats]
    ch = kquant.Chain()
    cuts = []
    for name, w, x, y in order:
        if name in ("qkv", "lm_head"):
            ch.add(xres, w, y, prologue=capi.PRO_RMS_NORM, norm_w=norm_w, eps=1e-5)
            cuts.append(len(ch))            # a launch ends behind every q|k|v (attention follows) and behind lm_head
        elif name == "o":
            ch.add(attn, w, xres, residual=xres)
        elif name == "gate_up":
            ch.add(xres, w, act, prologue=capi.PRO_RMS_NORM, norm_w=norm_w, eps=1e-5, epilogue=capi.EPI_SILU_MUL)
        else:
            ch.add(act, w, xres, residual=xres)
    ch.build()

    def chain_pass():
        xres.copy_(x0)                      # (the residual stream would grow without bound over replays otherwise)
        a = 0
        for b in cuts:
            ch.run(a, b - a)
            a = b
    res["chain_ms"] = round(timed(chain_pass), 4)
    ch.status()
    res["chain_launches"] = len(cuts)
    # the greedy pick behind lm_head rides in the lm_head launch (bpk_kq_matmul_argmax): the launch with and
    # without it, graphs of 20 over the layer set's lm_head
    _, w_lm, x_lm, logits = next(m for m in mats if m[0] == "lm_head")
    idx = torch.empty(1, dtype=torch.int32, device="cuda")
    val = torch.empty(1, dtype=torch.float32, device="cuda")
    stream = lambda: torch.cuda.current_stream().cuda_stream

    def lm_plain():
        for _ in range(20):
            kquant.matmul(x_lm, w_lm, out=logits)

    def lm_pick():
        for _ in range(20):
            capi.check(capi.lib().bpk_kq_matmul_argmax(w_lm.type, x_lm.data_ptr(), w_lm.data.data_ptr(), None, logits.data_ptr(),
                                                       1, w_lm.N, w_lm.K, w_lm.n_blocks, w_lm.row_stride_words,
                                                       idx.data_ptr(), val.data_ptr(), stream()))
    res["lm_head_us"] = round(timed(lm_plain) * 1e3 / 20, 2)
    res["lm_head_with_pick_us"] = round(timed(lm_pick) * 1e3 / 20, 2)
    res["pick"] = capi.last_kernel()
    n = sum(1 for name, *_ in mats if name == "qkv")
    res["launches_saved"] = 5 * n     # per layer: two norms, act*mul, two residual adds
    return res


def load_leg(n_layers=8):
    """GGUF file -> device weights: a file of n_layers x [gate, up (Q4_K, stacked into one weight), down
    (Q6_K)] at the layer set's shapes is written to the temporary directory, opened, and every weight is
    created from it.  Two passes: the second finds the file in the page cache and the upload stage warm."""
    import tempfile
    import struct
    import numpy as np
    import torch
    from backpack_amd import capi, kquant, synth
    from backpack_amd.gguf import GGUFFile
    H, I = 4096, 14336
    rng = np.random.default_rng(0)

    def raw(type_, N, K):
        nb = K // 256
        bb = 144 if type_ == synth.Q4_K else 210
        return rng.integers(0, 256, size=N * nb * bb, dtype=np.uint8)
    tensors = []
    for l in range(n_layers):
        tensors += [(f"blk.{l}.ffn_gate.weight", (H, I), synth.Q4_K), (f"blk.{l}.ffn_up.weight", (H, I), synth.Q4_K),
                    (f"blk.{l}.ffn_down.weight", (I, H), synth.Q6_K)]

    def s(b):
        return struct.pack("<Q", len(b)) + b
    with tempfile.TemporaryDirectory() as d:
        path = d + "/load.gguf"
        head = struct.pack("<IIQQ", 0x46554747, 3, len(tensors), 0)
        datas, pos = [], 0
        for name, dims, type_ in tensors:
            body = raw(type_, dims[1], dims[0])
            pos = (pos + 31) // 32 * 32
            head += s(name.encode()) + struct.pack("<IQQIQ", 2, dims[0], dims[1], type_, pos)
            datas.append((pos, body))
            pos += body.size
        data_offset = (len(head) + 31) // 32 * 32
        with open(path, "wb") as f:
            f.write(head)
            for off, body in datas:
                f.seek(data_offset + off)
                f.write(body.tobytes())
        total = sum(b.size for _, b in datas)
        del datas
        res = {"file_bytes": data_offset + pos, "weight_bytes": total}
        for label in ("first_pass", "second_pass"):
            t0 = time.perf_counter()
            ws = []
            with GGUFFile(path) as g:
                for l in range(n_layers):
                    ws.append(kquant.from_gguf(g, [f"blk.{l}.ffn_gate.weight", f"blk.{l}.ffn_up.weight"]))
                    ws.append(kquant.from_gguf(g, f"blk.{l}.ffn_down.weight"))
            torch.cuda.synchronize()
            sec = time.perf_counter() - t0
            res[label] = {"s": round(sec, 3), "GBps": round(total / sec / 1e9, 2)}
            del ws
    return res


def config0_leg():
    """One Q4_K matvec, M=1, K=N=4096 (a decode projection): cold = 64 distinct
    matrices per pass (604 MB, beyond the last-level cache), hot = one matrix
    launched back to back; graph replay, HIP events around each pass."""
    import torch
    from backpack_amd import kquant, synth
    N = K = 4096
    mk = lambda seed: kquant.KQuantPacked(synth.make_packed_device(synth.Q4_K, N, K, seed=seed), synth.Q4_K, N, K,
                                          synth.row_stride_words(synth.Q4_K, K), synth.n_blocks(K))
    ws = [mk(1000 + i) for i in range(64)]
    x = torch.randn(1, K, device="cuda", generator=torch.Generator(device="cuda").manual_seed(0))
    y = torch.empty(1, N, device="cuda")
    nbytes = synth.weight_bytes(synth.Q4_K, N, K) + (K + N) * 4
    res = {}
    for label, mats in (("cold", ws), ("hot", [ws[0]] * 64)):
        sel = [("m", w, x, y) for w in mats]
        times = []
        for _ in range(5):
            s, _ = run_region(sel, 4, 1, True)
            times.append(s / (4 * len(sel)))
        times.sort()
        res[label] = {"us_min": round(times[0] * 1e6, 2), "us_median": round(times[len(times) // 2] * 1e6, 2),
                      "GBps": round(nbytes / times[len(times) // 2] / 1e9, 1), "launches_timed": 5 * 4 * len(sel)}
    res["bytes_per_launch"] = nbytes
    return res


def verify_leg(mats, wb, use_graph):
    """The decode layer set at M = 2..16 tokens: the same weight bytes per step;
    the aim is a step time that stays near the M = 1 time."""
    import torch
    from backpack_amd import capi
    res = {}
    for M in (2, 4, 8, 16):
        xs, ys, ms = {}, {}, []
        for name, w, x, y in mats:
            if w.K not in xs:
                xs[w.K] = torch.randn(M, w.K, device="cuda")
            if w.N not in ys:
                ys[w.N] = torch.empty(M, w.N, device="cuda")
            ms.append((name, w, xs[w.K], ys[w.N]))
        sec, _ = run_region(ms, 10, 2, use_graph)
        act = sum((w.K + w.N) * 4 * M for _, w, _, _ in ms)
        res[f"M{M}"] = {"ms_per_step": round(sec / 10 * 1e3, 4), "GBps": round((wb + act) / (sec / 10) / 1e9, 1),
                        "kernel": capi.last_kernel()}
    return res


def moe_leg():
    """Routed-expert FFN, Qwen3-30B-A3B shape: 128 experts, top-8, hidden 2048,
    expert FFN 768, Q4_K gate/up and Q6_K down; one layer, T = 1 and T = 256.
    Bytes = each touched expert's three matrices once."""
    import torch
    from backpack_amd import capi, kquant, synth
    c = synth.QWEN3_30B_A3B
    E, k, H, I = c["n_experts"], c["top_k"], c["hidden"], c["inter"]

    def stacked(type_, N, K, seed):
        data = synth.make_packed_device(type_, E * N, K, seed=seed)
        return kquant.KQuantPacked(data, type_, E * N, K, synth.row_stride_words(type_, K), synth.n_blocks(K))
    # several layers' worth of distinct expert stacks so that replays do not run from cache
    layers = [(stacked(c["gate_up_type"], I, H, 10 + 3 * l), stacked(c["gate_up_type"], I, H, 11 + 3 * l),
               stacked(c["down_type"], H, I, 12 + 3 * l)) for l in range(4)]
    per_expert = 2 * synth.weight_bytes(c["gate_up_type"], I, H) + synth.weight_bytes(c["down_type"], H, I)
    res = {}
    g = torch.Generator(device="cpu").manual_seed(7)
    for T in (1, 256):
        idx = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32).cuda()
        wt = torch.softmax(torch.randn(T, k, generator=g), dim=-1).cuda()
        x = torch.randn(T, H, device="cuda")
        touched = int(torch.unique(idx).numel())
        for gu, up, dn in layers:
            kquant.moe_ffn(x, gu, up, dn, idx, wt, E)
        torch.cuda.synchronize()
        reps = 20
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            for gu, up, dn in layers:
                kquant.moe_ffn(x, gu, up, dn, idx, wt, E)
        e1.record()
        torch.cuda.synchronize()
        sec = e0.elapsed_time(e1) * 1e-3 / (reps * len(layers))
        ffn_kernel = capi.last_kernel()
        nbytes = touched * per_expert
        flops = 2.0 * T * k * 3 * H * I
        # the router stage in front of it: fp32 router matvec + top-k softmax, timed in a replayed graph
        wr = torch.randn(E, H, device="cuda") / H ** 0.5
        ridx = torch.empty((T, k), dtype=torch.int32, device="cuda")
        rwt = torch.empty((T, k), dtype=torch.float32, device="cuda")
        rs = torch.cuda.Stream()
        with torch.cuda.stream(rs):
            def route():
                capi.check(capi.lib().bpk_moe_route(x.data_ptr(), wr.data_ptr(), T, H, E, k, 1, None, ridx.data_ptr(),
                                                    rwt.data_ptr(), rs.cuda_stream))
            route()
            rs.synchronize()
            rg = torch.cuda.CUDAGraph()
            with torch.cuda.graph(rg, stream=rs):
                for _ in range(50):
                    route()
            rg.replay()
            rs.synchronize()
            r0, r1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            r0.record(rs)
            for _ in range(10):
                rg.replay()
            r1.record(rs)
            rs.synchronize()
        route_us = r0.elapsed_time(r1) * 1e3 / 500
        res[f"T{T}"] = {"us_per_layer": round(sec * 1e6, 2), "route_us": round(route_us, 2),
                        "experts_touched": touched, "weight_bytes": nbytes,
                        "GBps": round(nbytes / sec / 1e9, 1), "TFLOPs": round(flops / sec / 1e12, 2),
                        "kernel": ffn_kernel}
    return res


def prefill_leg(mats, M=2048):
    """The bf16 dequant-GEMM over the layer set at M tokens: ONE PASS = every one of the set's distinct matrices
    (32 layers x [qkv, o, gate_up, down] + lm_head, the weights the decode leg holds) multiplied once, in layer
    order, on one stream; timed over whole passes.  Per-shape figures come from passes over one shape's 32
    matrices.  `accuracy`: the output of one gate|up launch against fp64 contractions of (a) the exactly
    dequantised weights (bpk_kq_dequant_rows, bit-identical to the reference's dequant) and (b) those weights
    rounded to bf16, on sampled rows, computed with torch on the GPU."""
    import torch
    from backpack_amd import kquant
    xs, ys = {}, {}
    for _, w, _, _ in mats:
        if w.K not in xs:
            xs[w.K] = torch.randn(M, w.K, device="cuda", generator=torch.Generator(device="cuda").manual_seed(w.K)).to(torch.bfloat16)
        if w.N not in ys:
            ys[w.N] = torch.empty(M, w.N, device="cuda")

    def run(sel, passes, warm):
        stream = torch.cuda.Stream()
        with torch.cuda.stream(stream):
            for _ in range(warm):
                for _, w, _, _ in sel:
                    kquant.matmul(xs[w.K], w, out=ys[w.N])
            stream.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            for _ in range(passes):
                for _, w, _, _ in sel:
                    kquant.matmul(xs[w.K], w, out=ys[w.N])
            e1.record(stream)
            stream.synchronize()
        return e0.elapsed_time(e1) * 1e-3 / passes

    res = {}
    for name in ("qkv", "o", "gate_up", "down", "lm_head"):
        sel = [m for m in mats if m[0] == name]
        s = run(sel, 2 if name != "lm_head" else 6, 1) / len(sel)
        w = sel[0][1]
        res[name] = {"ms": round(s * 1e3, 3), "TFLOPs": round(2.0 * M * w.N * w.K / s / 1e12, 1)}
    passes = 3
    sec = run(mats, passes, 1)
    flops = sum(2.0 * M * w.N * w.K for _, w, _, _ in mats)
    tf = flops / sec / 1e12
    res["layer_set"] = {"TFLOPs": round(tf, 1), "pct_of_bf16_mfma_peak": round(tf / MFMA_BF16_PEAK_TFLOPS * 100, 2),
                        "M": M, "ms_per_pass": round(sec * 1e3, 2), "launches_per_pass": len(mats), "passes_timed": passes,
                        "how": f"full pass: each of the set's {len(mats)} distinct matrices once per pass, in layer order, "
                               f"{passes} passes timed after one of warm-up"}
    if M == 2048:
        res["accuracy"] = gemm_accuracy(next(m for m in mats if m[0] == "gate_up")[1], xs, ys, M)
        res["vendor_bf16_gemm"] = vendor_gemm({n: next(m for m in mats if m[0] == n)[1] for n in ("gate_up", "down")}, xs, M)
    return res


def vendor_gemm(shapes, xs, M):
    """For scale only: the vendor library's plain bf16 GEMM (torch.matmul) on the same shapes, with the weights
    already expanded to bf16 in HBM and a bf16 output, ten launches back to back."""
    import torch
    out = {"what": "torch.matmul, bf16 weights resident in HBM (3.5x the packed bytes), bf16 output; not part of the product"}
    for name, w in shapes.items():
        wb = torch.randn(w.N, w.K, device="cuda").to(torch.bfloat16)
        yb = torch.empty(M, w.N, device="cuda", dtype=torch.bfloat16)
        for _ in range(3):
            torch.matmul(xs[w.K], wb.t(), out=yb)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(10):
            torch.matmul(xs[w.K], wb.t(), out=yb)
        e1.record()
        torch.cuda.synchronize()
        sec = e0.elapsed_time(e1) * 1e-3 / 10
        out[name] = {"ms": round(sec * 1e3, 3), "TFLOPs": round(2.0 * M * w.N * w.K / sec / 1e12, 1)}
        del wb, yb
    return out


def gemm_accuracy(w, xs, ys, M):
    """Largest error of one bf16 GEMM launch on sampled weight rows, relative to the rms and to the largest |y| of
    the sample: against the exact weights (the error the bf16 rounding of W brings: unit roundoff 2^-9 per weight)
    and against the bf16-rounded weights (what the kernel itself adds: accumulation order only)."""
    import torch
    from backpack_amd import kquant
    x, y = xs[w.K], ys[w.N]
    kquant.matmul(x, w, out=y)
    rows = torch.randperm(w.N, device="cuda", generator=torch.Generator(device="cuda").manual_seed(3))[:256].to(torch.int32)
    deq = kquant.dequant_rows(w, rows)                    # fp32 [256, K], bit-exact weights
    got = y[:, rows.long()].double()
    x64 = x.double()
    exact = x64 @ deq.double().T
    rounded = x64 @ deq.to(torch.bfloat16).double().T
    rms, peak = float(exact.pow(2).mean().sqrt()), float(exact.abs().max())
    e1, e2 = float((got - exact).abs().max()), float((got - rounded).abs().max())
    return {"matrix": f"gate_up {w.N}x{w.K}, M={M}, 256 sampled weight rows",
            "max_err_over_rms": round(e1 / rms, 5), "max_err_over_peak": round(e1 / peak, 6),
            "frobenius_rel": round(float((got - exact).pow(2).sum().sqrt() / exact.pow(2).sum().sqrt()), 6),
            "vs_bf16_rounded_weights_over_peak": float(f"{e2 / peak:.3g}"),
            "note": "errors against the exact weights are the bf16 rounding of W that the workload prescribes "
                    "(tolerance 1e-2 of the largest |y|); against the rounded weights only the summation order is left"}


if __name__ == "__main__":
    main()
