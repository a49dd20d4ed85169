#!/usr/bin/env python3
"""Benchmark of the emitted gfx950 kernels on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--all]

A step is one launch of the workload's kernel over its full synthetic input,
already resident in HBM.  Prints ONE JSON line: throughput of the workload
(TFLOP/s for GEMM/FMHA, GB/s for LayerNorm/elementwise), the roofline of its
kernel (algorithmic work / HIP-event launch duration against the MI355X peak)
and the CPU baseline (the oracle's naive nest on one host core, bounded sample).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

# MI355X published dense peaks.
PEAK = {"hbm": (8000.0, "GB/s"), "bf16": (2500.0, "TFLOP/s"), "fp8": (5000.0, "TFLOP/s"),
        "f32": (157.3, "TFLOP/s")}

DEFAULT_WORKLOAD = "gemm_bf16_4096x11008x4096"

# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
# (summaries under profiles/), keyed by workload; absent = not measured.
MEASURED_TRAFFIC = {
    "add_bias_f32_16384x4096": 537022915,
    "bgemm_f32_16x1024": 586882804,
    "fmha_bf16_b8h32s2048d128": 537017109,
    "fmha_bf16_b8h32s2048d128_causal": 959612372,
    "gather_bf16_32000x4096_16384": 267689885,
    "gelu_16384x4096": 536870912,
    "gemm_bf16_4096x11008x4096": 820435393,
    "gemm_bf16_4096x11008x4096_bf16out": 736532757,
    "gemm_f32_1024": 29830782,
    "gemm_f32_4096": 469796778,
    "gemm_fp8_4096x11008x4096": 505749410,
    "gemm_fp8_nn_4096x11008x4096": 498713389,
    "layernorm_16384x4096": 537135035,
    "layernorm_gelu_16384x4096": 537152941,
    "softmax_f32_16384x4096": 536929445,
    "softmax_f32_65536x2048": 1073893382,
}


def make_inputs(torch, family, p):
    """Synthetic operands of the workload's shape, generated on the device."""
    g = torch.Generator(device="cuda")
    g.manual_seed(0x4B4347)
    dev = "cuda"
    if family == "layernorm":
        x = torch.randn(p["ROWS"], p["N"], device=dev, generator=g)
        gamma = torch.rand(p["NG"], device=dev, generator=g) + 0.5
        beta = torch.rand(p["NB"], device=dev, generator=g) * 0.2 - 0.1
        y = torch.empty_like(x)
        return [x, gamma, beta, y]
    if family == "elementwise":
        x = torch.randn(p["N"], device=dev, generator=g)
        return [x, torch.empty_like(x)]
    if family in ("gemm_f32", "gemm_bf16", "gemm_fp8"):
        b_, m, n, k = p.get("BATCH", 1), p["M"], p["N"], p["K"]
        if family == "gemm_f32":
            a = torch.rand(b_, m, k, device=dev, generator=g) * 2 - 1
            w = torch.rand(b_, k, n, device=dev, generator=g) * 2 - 1
            return [a, w, torch.empty(b_, m, n, device=dev)]
        a = torch.randn(b_, m, k, device=dev, generator=g)
        w = torch.randn(b_, k, n, device=dev, generator=g) * 0.02
        if p.get("TB", 0):
            w = w.transpose(-1, -2).contiguous()
        out_dt = torch.bfloat16 if p.get("OUT_BF16", 0) else torch.float32
        c = torch.empty(b_, m, n, device=dev, dtype=out_dt)
        if family == "gemm_bf16":
            return [a.bfloat16(), w.bfloat16(), c]
        sa = float(a.abs().max()) / 448.0
        sw = float(w.abs().max()) / 448.0
        return [(a / sa).to(torch.float8_e4m3fn), (w / sw).to(torch.float8_e4m3fn), c, sa, sw]
    if family == "fmha_bf16":
        shp = (p["B"], p["H"], p["S"], p["D"])
        q = torch.randn(shp, device=dev, generator=g).bfloat16()
        k = torch.randn(shp, device=dev, generator=g).bfloat16()
        v = torch.randn(shp, device=dev, generator=g).bfloat16()
        return [q, k, v, torch.empty_like(q)]
    if family == "softmax":
        x = torch.randn((p["ROWS"], p["N"]), device=dev, generator=g)
        return [x] if p.get("INPLACE", 1) else [x, torch.empty_like(x)]
    if family == "binary":
        dims = [int(t) for t in p["DIMS"].split(",")]
        def operand(strides):
            shape = [d if s else 1 for d, s in zip(dims, [int(t) for t in strides.split(",")])]
            return torch.randn(shape, device=dev, generator=g)
        return [operand(p["SA"]), operand(p["SB"]), torch.empty(dims, device=dev)]
    if family == "gather":
        esize = {2: torch.bfloat16, 4: torch.float32}[p["ESIZE"]]
        table = torch.randn((p["OUTER"], p["AXIS"], p["INNER"]), device=dev, generator=g).to(esize)
        idx = torch.randint(0, p["AXIS"], (p["NIDX"],), device=dev, generator=g, dtype=torch.int64)
        return [table, idx, torch.empty((p["OUTER"], p["NIDX"], p["INNER"]), device=dev, dtype=esize)]
    raise ValueError(family)


def family_roof(family):
    if family in ("layernorm", "elementwise", "binary", "softmax"):
        return "hbm", "hbm", "f32"
    if family == "gather":
        return "hbm", "hbm", "bf16"
    if family == "gemm_f32":
        return "mfma", "f32", "f32"
    if family == "gemm_fp8":
        return "mfma", "fp8", "fp8"
    return "mfma", "bf16", "bf16"


def cpu_baseline(family, p):
    """The oracle's naive nest on ONE host core over a bounded sample."""
    import numpy as np
    import oracle_lib as O
    if family in ("gemm_f32", "gemm_bf16", "gemm_fp8"):
        m, n, k = p["M"], p["N"], p["K"]
        rows = max(1, min(m, int(1.5e10 / (2.0 * n * k))))     # about ten seconds of one core
        a = O.uniform((rows, k), stream=1)
        b = O.uniform((k, n), stream=2)
        t0 = time.perf_counter()
        O.matmul(a, b, nest=True)
        dt = time.perf_counter() - t0
        return {"value": round(2.0 * rows * n * k / dt / 1e12, 6), "unit": "TFLOP/s", "cores": 1, "kind": "port",
                "sample": "%d of %d rows of C, naive i-j-k nest, fp32, %.1f s" % (rows, m, dt)}
    if family == "layernorm":
        n = p["N"]
        rows = p["ROWS"]
        x = O.normal((rows, n), stream=1)
        g = O.uniform((p["NG"],), stream=2, lo=0.5, hi=1.5)
        b = O.uniform((p["NB"],), stream=3, lo=-0.1, hi=0.1)
        t0 = time.perf_counter()
        y = O.layernorm(x, g, b, 1)
        if p.get("GELU"):
            O.elementwise(y, "Gelu")
        dt = time.perf_counter() - t0
        return {"value": round(2.0 * rows * n * 4 / dt / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": "%d of %d rows, 3-pass nest%s, %.2f s" % (rows, p["ROWS"], " + GELU nest" if p.get("GELU") else "", dt)}
    if family == "elementwise":
        n = min(p["N"], 1 << 24)
        x = O.normal((n,), stream=1)
        t0 = time.perf_counter()
        O.elementwise(x, "Gelu")
        dt = time.perf_counter() - t0
        return {"value": round(2.0 * n * 4 / dt / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": "%d of %d elements, %.2f s" % (n, p["N"], dt)}
    if family == "softmax":
        n = p["N"]
        rows = min(p["ROWS"], max(1, (1 << 28) // n))
        x = O.normal((rows, n), stream=1)
        t0 = time.perf_counter()
        O.softmax(x)
        dt = time.perf_counter() - t0
        return {"value": round(2.0 * rows * n * 4 / dt / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": "%d of %d rows, two-loop nest, %.2f s" % (rows, p["ROWS"], dt)}
    if family == "gather":
        rows = min(p["NIDX"], 4096)
        table = np.zeros((p["OUTER"], p["AXIS"], p["INNER"] * p["ESIZE"]), dtype=np.uint8)
        idx = np.random.RandomState(1).randint(0, p["AXIS"], size=(rows,))
        reps, t0 = 0, time.perf_counter()
        while reps < 1000 and time.perf_counter() - t0 < 10.0:
            O.gather(table, idx, 1)
            reps += 1
        dt = time.perf_counter() - t0
        return {"value": round(2.0 * reps * p["OUTER"] * rows * p["INNER"] * p["ESIZE"] / dt / 1e9, 4), "unit": "GB/s",
                "cores": 1, "kind": "port",
                "sample": "%d of %d indices, byte-wise nest, %d passes, %.1f s" % (rows, p["NIDX"], reps, dt)}
    if family == "fmha_bf16":
        s, d = p["S"], p["D"]
        rows = 64
        q = O.normal((1, s, d), stream=1)
        k = O.normal((1, s, d), stream=2)
        v = O.normal((1, s, d), stream=3)
        t0 = time.perf_counter()
        O.fmha(q[:, :rows].copy() if False else q, k, v, scale=float(p.get("SCALE", 1.0)), causal=bool(p.get("CAUSAL", 0)))
        dt = time.perf_counter() - t0
        fl = 4.0 * s * s * d * (0.5 if p.get("CAUSAL", 0) else 1.0)
        return {"value": round(fl / dt / 1e12, 6), "unit": "TFLOP/s", "cores": 1, "kind": "port",
                "sample": "1 of %d (batch,head) slabs, three naive nests, fp32, %.1f s" % (p["B"] * p["H"], dt)}
    return None


def run_workload(torch, name, steps, warmup, with_cpu, with_same=True):
    from kernelcodegen_amd import runtime as R
    from kernelcodegen_amd.configs import WORKLOADS
    family, params = WORKLOADS[name]
    text, info = R.emit_kernel(family, "kernel0", **params)
    mod = R.compile_source(R.prelude() + text, [info])
    kern = mod.kernel("kernel0")
    bound, peak_key, dtype = family_roof(family)
    # Every kernel is launched on three input/output sets in turn, so that a launch finds its operands in HBM
    # and not in the 256 MB last-level cache where the previous launch left them.  (On one set the streaming
    # kernels measure 10-25 % faster, the fp8 GEMM 14 % and the bf16 GEMM 4 %; that figure is reported as
    # roofline.same_buffers_frac and is not the throughput.)
    nsets = 3
    sets = [make_inputs(torch, family, params) for _ in range(nsets)]

    def timed_launches(count, rotate):
        """Per-launch duration from device events on the launch stream: the launches go in runs of at most 50,
        each between its own pair of events, and the median run counts (the HIP runtime stalls the enqueueing
        thread for some 30 ms once per process, around its 256th launch; a run that contains the stall is
        host time, not kernel time)."""
        runs = []
        done = 0
        while done < count:
            n = min(50, count - done)
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for i in range(done, done + n):
                kern.launch(*sets[i % nsets if rotate else 0])
            b.record()
            torch.cuda.synchronize()
            runs.append(a.elapsed_time(b) / n)
            done += n
        runs.sort()
        return runs[len(runs) // 2] if len(runs) % 2 else 0.5 * (runs[len(runs) // 2 - 1] + runs[len(runs) // 2])

    # Untimed priming past the runtime's one-time enqueue stall, then the W warm-up steps and the K timed steps.
    for i in range(320):
        kern.launch(*sets[i % nsets])
    torch.cuda.synchronize()
    for i in range(max(warmup, nsets)):
        kern.launch(*sets[i % nsets])
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        kern.launch(*sets[i % nsets])
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_step = wall * 1e3 / steps
    ms_kernel = timed_launches(max(steps, 6), True)
    ms_same = None
    if with_same:
        timed_launches(30, False)    # the first launches after the change of pattern are not representative
        ms_same = min(timed_launches(max(steps, 6), False) for _ in range(2))

    peak, unit = PEAK[peak_key]
    work = info["bytes"] / 1e9 if bound == "hbm" else info["flops"] / 1e12
    achieved = work / (ms_kernel * 1e-3)
    value = work / (ms_step * 1e-3)
    res = {
        "metric": ("%s throughput, %s" % (name, "GB/s + %HBM peak" if bound == "hbm" else "TFLOP/s + %MFMA peak")),
        "value": round(value, 3), "unit": unit, "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(ms_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dtype, "data": "synthetic",
        "config": {"workload": name, "family": family, "buffer_sets": nsets, **{k: v for k, v in params.items()}},
        "roofline": {"bound": bound, "achieved": round(achieved, 3), "peak": peak, "unit": unit,
                     "frac": round(achieved / peak, 4), "traffic": MEASURED_TRAFFIC.get(name),
                     "kernel_ms": round(ms_kernel, 5),
                     "algorithmic": info["bytes"] if bound == "hbm" else info["flops"]},
    }
    if ms_same is not None:
        res["roofline"]["same_buffers_frac"] = round(work / (ms_same * 1e-3) / peak, 4)
    if with_cpu:
        res["cpu_baseline"] = cpu_baseline(family, params)
    mod.destroy()
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default=DEFAULT_WORKLOAD)
    ap.add_argument("--all", action="store_true", help="also run every other workload (reported under 'others')")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-same-buffers", action="store_true",
                    help="leave out the launches on one buffer set (for a profiler run whose per-kernel average "
                         "should cover the rotating launches only)")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus %d is not supported (every workload is a "
                 "single-GPU kernel, nothing is sharded)" % a.gpus)
    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    from kernelcodegen_amd._lib import lib, check
    from kernelcodegen_amd.configs import WORKLOADS
    check(lib().kcg_hip_init(0), "kcg_hip_init")
    if a.workload not in WORKLOADS:
        sys.exit("unknown workload %s; choose from %s" % (a.workload, ", ".join(WORKLOADS)))
    res = run_workload(torch, a.workload, a.steps, a.warmup, not a.no_cpu_baseline, not a.no_same_buffers)
    if a.all:
        others = {}
        for name in WORKLOADS:
            if name == a.workload:
                continue
            r = run_workload(torch, name, a.steps, a.warmup, False, not a.no_same_buffers)
            # the side list reports the HIP-event figures (the wall clock of a short loop that follows
            # other workloads in the same process picks up their clean-up)
            others[name] = {"value": r["roofline"]["achieved"], "unit": r["unit"], "ms_per_step": r["ms_per_step"],
                            "frac": r["roofline"]["frac"], "kernel_ms": r["roofline"]["kernel_ms"],
                            "same_buffers_frac": r["roofline"].get("same_buffers_frac")}
            print("%-34s %10.3f %-8s %9.4f ms  %5.1f%% of peak" % (name, r["roofline"]["achieved"], r["unit"],
                                                                  r["roofline"]["kernel_ms"], 100 * r["roofline"]["frac"]),
                  file=sys.stderr, flush=True)
        res["others"] = others
    print(json.dumps(res))


if __name__ == "__main__":
    main()
