#!/usr/bin/env python3
"""Benchmark of the grouped_mm hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

A step is one forward call of ``grouped_mm`` on synthetic inputs that are already
resident in HBM.  The default workload is the Mixtral-style 2D x 3D MoE
up-projection (G = 8, 16384 routed rows, K = 4096, N = 14336, skewed group sizes
from the committed fixture).  Prints ONE JSON line: useful TFLOP/s
(2 * sum_g M_g * K * N per call), the roofline position of the kernel measured
with HIP events on the launch stream, and -- reported only -- the same per-group
fp32 matmul computed by the test oracle on the host CPU for a bounded sample of
the workload.
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

METRIC = "TFLOP/s + % bf16 MFMA peak, 2D×3D MoE G=8 K=4096 N=14336, 1 GPU"
PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E
SETTLE_S = 0.15            # seconds of untimed launches before warm-up, after the host-side parity check
# workload -> tag in the name of its rocprofv3 summary under profiles/ (`..__<tag>.md`)
PROFILE_TAG = {"readme": "readme_2d3d", "mixtral": "mixtral_2d3d", "mixtral_colmajor": "mixtral_colmajor_2d3d",
               "downproj": "downproj_2d3d", "fine": "fine_grained_2d3d", "batched": "batched_3d3d",
               "batched_colmajor": "batched_colmajor_3d3d", "kgrouped": "kgrouped_2d2d", "ngrouped": "ngrouped_3d2d"}


def measured_traffic(name):
    """HBM-side bytes per launch of the workload's kernel as its committed rocprofv3 summary states them
    (FETCH_SIZE + WRITE_SIZE, scaled by the copy-kernel calibration): the line
    `traffic_bytes_per_launch: N` of profiles/*__<tag>.md.  Returns (bytes or None, file or None)."""
    import glob
    import re
    tag = PROFILE_TAG.get(name)
    for path in sorted(glob.glob(os.path.join(ROOT, "profiles", f"*__{tag}.md"))) if tag else []:
        m = re.search(r"traffic_bytes_per_launch:\s*(\d+)", open(path).read())
        if m:
            return int(m.group(1)), os.path.relpath(path, ROOT)
    return None, None


def load_sizes(key):
    with open(os.path.join(ROOT, "tests", "golden", "group_sizes.json")) as f:
        return json.load(f)[key]


def make_workload(name, torch):
    """Returns dict(a, b, offs, out, launch, flops, bytes, bound, k, desc) with CPU tensors."""
    from grouped_mm_bf16_amd import kernels
    g1, g2 = torch.Generator().manual_seed(1), torch.Generator().manual_seed(2)
    bf = torch.bfloat16
    if name == "readme":
        sizes = [0, 7, 1, 13, 0, 11]
        g0 = torch.Generator().manual_seed(0)
        a = torch.randn(32, 64, generator=g0).to(bf)
        b = torch.randn(6, 64, 48, generator=g0).to(bf)
        w = dict(variant="2d3d", sizes=sizes, a=a, b=b, out_shape=(32, 48), out_dtype=bf,
                 flops=2.0 * 32 * 64 * 48, bound="latency", k=64,
                 bytes=a.numel() * 2 + 4 * 64 * 48 * 2 + 32 * 48 * 2,
                 desc="readme_2d3d_G6_M32_K64_N48_two_empty_groups")
    elif name in ("mixtral", "mixtral_colmajor"):
        # mixtral_colmajor: the weights as a linear layer stores them, [G, N, K] viewed transposed
        sizes = load_sizes("mixtral_top2_g8")
        a = torch.randn(16384, 4096, generator=g1).to(bf)
        b = (torch.randn(8, 4096, 14336, generator=g2) * 0.02).to(bf)
        w = dict(variant="2d3d", sizes=sizes, a=a, b=b, out_shape=(16384, 14336), out_dtype=bf,
                 flops=2.0 * 16384 * 4096 * 14336, bound="mfma", k=4096,
                 bytes=a.numel() * 2 + b.numel() * 2 + 16384 * 14336 * 2,
                 desc="mixtral_moe_up_proj_2d3d_G8_M16384_K4096_N14336_skewed_top2" + ("_Bcolmajor" if name.endswith("colmajor") else ""),
                 b_col=name.endswith("colmajor"))
    elif name == "downproj":
        # the down projection of the same layer (and the input gradient of the up projection): the same FLOPs
        # with a 3.5 times longer contraction and 4.25 rounds of tiles on 256 compute units
        sizes = load_sizes("mixtral_top2_g8")
        a = torch.randn(16384, 14336, generator=g1).to(bf)
        b = (torch.randn(8, 14336, 4096, generator=g2) * 0.02).to(bf)
        w = dict(variant="2d3d", sizes=sizes, a=a, b=b, out_shape=(16384, 4096), out_dtype=bf,
                 flops=2.0 * 16384 * 14336 * 4096, bound="mfma", k=14336,
                 bytes=a.numel() * 2 + b.numel() * 2 + 16384 * 4096 * 2,
                 desc="mixtral_moe_down_proj_2d3d_G8_M16384_K14336_N4096_skewed_top2")
    elif name == "fine":
        sizes = load_sizes("fine_grained_top8_g128")
        a = torch.randn(32768, 2048, generator=g1).to(bf)
        b = (torch.randn(128, 2048, 768, generator=g2) * 0.02).to(bf)
        nonempty = sum(1 for s in sizes if s > 0)
        w = dict(variant="2d3d", sizes=sizes, a=a, b=b, out_shape=(32768, 768), out_dtype=bf,
                 flops=2.0 * 32768 * 2048 * 768, bound="hbm", k=2048,
                 bytes=a.numel() * 2 + nonempty * 2048 * 768 * 2 + 32768 * 768 * 2,
                 desc="fine_grained_moe_2d3d_G128_M32768_K2048_N768_top8")
    elif name in ("batched", "batched_colmajor"):
        a = torch.randn(32, 1024, 1024, generator=g1).to(bf)
        b = (torch.randn(32, 1024, 4096, generator=g2) * 0.02).to(bf)
        w = dict(variant="3d3d", sizes=None, a=a, b=b, out_shape=(32, 1024, 4096), out_dtype=bf,
                 flops=2.0 * 32 * 1024 * 1024 * 4096, bound="mfma", k=1024,
                 bytes=a.numel() * 2 + b.numel() * 2 + 32 * 1024 * 4096 * 2,
                 desc="batched_3d3d_G32_M1024_K1024_N4096" + ("_Bcolmajor" if name.endswith("colmajor") else ""),
                 b_col=name.endswith("colmajor"))
    elif name == "kgrouped":
        sizes = load_sizes("mixtral_top2_g8")
        a = torch.randn(4096, 16384, generator=g1).to(bf)
        b = torch.randn(16384, 14336, generator=g2).to(bf)
        w = dict(variant="2d2d", sizes=sizes, a=a, b=b, out_shape=(8, 4096, 14336), out_dtype=torch.float32,
                 flops=2.0 * 4096 * 16384 * 14336, bound="mfma", k=16384,
                 bytes=a.numel() * 2 + b.numel() * 2 + 8 * 4096 * 14336 * 4,
                 desc="k_grouped_weight_grad_2d2d_G8_M4096_Ktotal16384_N14336_fp32out")
    elif name == "plain":
        # the Mixtral workload's FLOPs as ONE group: what the same tile does without any grouping
        a = torch.randn(1, 16384, 4096, generator=g1).to(bf)
        b = (torch.randn(1, 4096, 14336, generator=g2) * 0.02).to(bf)
        w = dict(variant="3d3d", sizes=None, a=a, b=b, out_shape=(1, 16384, 14336), out_dtype=bf,
                 flops=2.0 * 16384 * 4096 * 14336, bound="mfma", k=4096,
                 bytes=a.numel() * 2 + b.numel() * 2 + 16384 * 14336 * 2,
                 desc="plain_gemm_3d3d_G1_M16384_K4096_N14336")
    elif name == "ngrouped":
        sizes = load_sizes("mixtral_top2_g8")
        a = torch.randn(8, 4096, 4096, generator=g1).to(bf)
        b = (torch.randn(4096, 16384, generator=g2) * 0.02).to(bf)
        w = dict(variant="3d2d", sizes=sizes, a=a, b=b, out_shape=(4096, 16384), out_dtype=bf,
                 flops=2.0 * 4096 * 4096 * 16384, bound="mfma", k=4096,
                 bytes=a.numel() * 2 + b.numel() * 2 + 4096 * 16384 * 2,
                 desc="n_grouped_3d2d_G8_M4096_K4096_Ntotal16384_skewed_top2")
    else:
        raise SystemExit(f"unknown workload {name}")
    w["launch"] = {"2d3d": kernels.grouped_mm_2d3d, "3d3d": kernels.grouped_mm_3d3d,
                   "2d2d": kernels.grouped_mm_2d2d, "3d2d": kernels.grouped_mm_3d2d}[w["variant"]]
    return w


def cpu_baseline(w, torch, budget_s=15.0):
    """The oracle (per-group fp32 torch.matmul on the host) on a bounded sample."""
    from oracle import grouped_mm_oracle as oracle
    threads = os.cpu_count() or 1
    try:
        threads = min(threads, len(os.sched_getaffinity(0)))
    except AttributeError:
        pass
    env = os.environ.get("OMP_NUM_THREADS")
    if env and env.isdigit():
        threads = min(threads, int(env))
    torch.set_num_threads(threads)
    a, b, sizes = w["a"], w["b"], w["sizes"]
    if w["variant"] == "2d3d":
        ranges = oracle.group_ranges(torch.tensor(sizes).cumsum(0).tolist())
        order = sorted(range(len(sizes)), key=lambda g: sizes[g])  # small groups first
        order = [g for g in order if sizes[g] > 0]
        K, N = a.shape[1], b.shape[2]

        def run(groups):
            af = [a[ranges[g][0]:ranges[g][1]].float() for g in groups]
            bfl = [b[g].float() for g in groups]
            t0 = time.perf_counter()
            for x, y in zip(af, bfl):
                torch.matmul(x, y)
            return time.perf_counter() - t0, sum(2.0 * x.shape[0] * K * N for x in af)

        # probe with the median group, then take as many groups as fit the budget
        probe = [order[len(order) // 2]]
        run(probe)
        t, fl = run(probe)
        rate = fl / max(t, 1e-9)
        chosen, work = [], 0.0
        for g in order[::-1]:
            f = 2.0 * sizes[g] * K * N
            if chosen and (work + f) / rate > budget_s:
                continue
            chosen.append(g)
            work += f
        # the sample is sized for about a third of the budget per run: median of up to 3 timed runs
        runs = [run(chosen)]
        while len(runs) < 3 and sum(r[0] for r in runs) + runs[0][0] < 2 * budget_s:
            runs.append(run(chosen))
        t, fl = sorted(runs)[len(runs) // 2]
        sample = (f"groups {sorted(chosen)} of {len(sizes)} ({fl / w['flops'] * 100:.0f}% of the step's FLOPs), "
                  f"median of {len(runs)} timed run(s) after a probe")
    else:
        # batched / K-grouped / N-grouped: the groups' own products (3D x 3D: the first batches), as many
        # as fit about a third of the budget per run; 1 warm-up + 3 timed runs, median
        G = a.shape[0] if w["variant"] == "3d3d" else len(sizes)
        ranges = oracle.group_ranges(torch.tensor(sizes).cumsum(0).tolist()) if sizes else None

        def operands(g):
            if w["variant"] == "3d3d":
                return a[g].float(), b[g].float()
            s_, e_ = ranges[g]
            if w["variant"] == "3d2d":
                return a[g].float(), b[:, s_:e_].float()
            return a[:, s_:e_].float(), b[s_:e_].float()

        x, y = operands(0)
        torch.matmul(x[:64], y)                       # thread-pool start-up
        t0 = time.perf_counter()
        torch.matmul(x, y)                            # warm-up run = the probe
        rate = 2.0 * x.shape[0] * x.shape[1] * y.shape[1] / max(time.perf_counter() - t0, 1e-9)
        chosen, ops, work = [], [], 0.0
        for g in range(G):
            x, y = operands(g)
            f = 2.0 * x.shape[0] * x.shape[1] * y.shape[1]
            if f == 0 or (chosen and (work + f) / rate > budget_s / 3):
                continue
            chosen.append(g)
            ops.append((x, y))
            work += f
        times = []
        for _ in range(3):
            t0 = time.perf_counter()
            for x, y in ops:
                torch.matmul(x, y)
            times.append(time.perf_counter() - t0)
        t, fl = sorted(times)[1], work
        sample = (f"groups {chosen} of {G} ({fl / w['flops'] * 100:.0f}% of the step's FLOPs), "
                  f"median of 3 timed runs after a warm-up")
    return {"value": round(fl / t / 1e12, 4), "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "sample": sample, "seconds": round(t, 3)}


def load_diag():
    """The bench-only diagnostics library (register-only MFMA loop), built beside the product library."""
    import ctypes
    from grouped_mm_bf16_amd import build
    if not os.path.exists(build.DIAG_LIB_PATH):
        raise SystemExit(f"{build.DIAG_LIB_PATH} is missing: build it with `python -m grouped_mm_bf16_amd.build`")
    lib = ctypes.CDLL(build.DIAG_LIB_PATH)
    i32, i64, vp = ctypes.c_int32, ctypes.c_int64, ctypes.c_void_p
    lib.gmm_diag_mfma_rate.restype = ctypes.c_int
    lib.gmm_diag_mfma_rate.argtypes = [vp, i64, vp, i64, i32, i32, i32, vp, vp]
    return lib


def mfma_only(args, torch, dev):
    """Rate of the matrix pipe alone (register-only loops of v_mfma_f32_16x16x32_bf16, which the assembly tile
    uses, and of v_mfma_f32_32x32x16_bf16), with operand values drawn like the workload's (N(0,1) for A
    fragments, 0.02 N(0,1) for B fragments) and with zeros."""
    import ctypes
    lib = load_diag()
    gen = torch.Generator().manual_seed(3)
    iters = 4000
    out = torch.empty(512 * 256 * 2, dtype=torch.float32, device=dev)
    res = {}
    for label, scale in (("random", 1.0), ("zeros", 0.0)):
        # 16 fragments per thread: the first 8 feed A operands (unit scale), the last 8 B operands (0.02)
        vals = torch.randn(4096 * 16, 8, generator=gen) * scale
        vals[(torch.arange(4096 * 16) % 16) >= 8] *= 0.02
        frags = vals.to(torch.bfloat16).to(dev)
        for shape, shape_name in ((0, "16x16x32"), (1, "32x32x16")):
            for waves in (1, 2):
                blocks = ctypes.c_int32(0)

                def launch():
                    rc = lib.gmm_diag_mfma_rate(frags.data_ptr(), frags.numel() * 2, out.data_ptr(), out.numel() * 4,
                                                waves, iters, shape, ctypes.addressof(blocks),
                                                torch.cuda.current_stream().cuda_stream)
                    if rc != 0:
                        raise SystemExit(f"gmm_diag_mfma_rate failed with status {rc}")
                for _ in range(args.warmup):
                    launch()
                torch.cuda.synchronize()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for _ in range(args.steps):
                    launch()
                e1.record()
                torch.cuda.synchronize()
                ms = e0.elapsed_time(e1) / args.steps
                flops = blocks.value * 4 * iters * (1048576.0 if shape == 0 else 524288.0)
                res[f"{shape_name}_{label}_{waves}_waves_per_simd"] = round(flops / ms / 1e9, 1)
    print(json.dumps({"metric": "v_mfma_f32_16x16x32_bf16 alone, register operands (context for the MFMA roofline)",
                      "value": res["16x16x32_random_1_waves_per_simd"], "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
                      "warmup": args.warmup, "peak": PEAK_BF16_TFLOPS, "detail": res}))


def library_comparator(w, a, b, offs, torch, steps):
    """PyTorch-ROCm's own grouped GEMM on the same device tensors: context for `value`, never an oracle."""
    import torch.nn.functional as F
    if not hasattr(F, "grouped_mm") or w["out_dtype"] != a.dtype:
        return {"name": "torch.nn.functional.grouped_mm", "value": None, "note": "not applicable to this workload"}
    run = (lambda: F.grouped_mm(a, b)) if offs is None else (lambda: F.grouped_mm(a, b, offs=offs))
    try:
        for _ in range(3):
            run()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            run()
        e1.record()
        torch.cuda.synchronize()
    except Exception as ex:  # the library rejects some layouts; that is a result too
        return {"name": "torch.nn.functional.grouped_mm", "value": None, "note": repr(ex)[:200]}
    ms = e0.elapsed_time(e1) / steps
    return {"name": "torch.nn.functional.grouped_mm", "value": round(w["flops"] / (ms * 1e-3) / 1e12, 2),
            "unit": "TFLOP/s", "ms_per_step": round(ms, 4)}


def parity_check(w, out, offs, torch, oracle):
    """Oracle comparison on the tensors that are about to be timed: the whole output of the small README
    case, otherwise a sample of rows of the first, a middle and the last group (K per element's own group)."""
    got = out.cpu()
    a, b = w["a"], w["b"]
    if w["desc"].startswith("readme"):
        oracle.assert_close(got, oracle.grouped_mm(a, b, offs.cpu()), w["k"], what="bench parity")
        return
    ranges = oracle.group_ranges(offs.cpu().tolist()) if offs is not None else None
    G = a.shape[0] if w["variant"] == "3d3d" else len(ranges)
    for g in sorted({0, G // 2, G - 1}):
        if w["variant"] == "2d3d":
            s_, e_ = ranges[g]
            if e_ == s_:
                continue
            rows = sorted({s_, (s_ + e_) // 2, e_ - 1})
            want = (a[rows].float() @ b[g].float()).to(got.dtype)
            oracle.assert_close(got[rows], want, w["k"], what=f"bench parity rows {rows} group {g}")
        elif w["variant"] == "3d3d":
            rows = [0, a.shape[1] // 2, a.shape[1] - 1]
            want = (a[g][rows].float() @ b[g].float()).to(got.dtype)
            oracle.assert_close(got[g][rows], want, w["k"], what=f"bench parity batch {g}")
        elif w["variant"] == "2d2d":
            s_, e_ = ranges[g]
            rows = [0, a.shape[0] // 2, a.shape[0] - 1]
            want = (a[rows][:, s_:e_].float() @ b[s_:e_].float()).to(got.dtype)
            oracle.assert_close(got[g][rows], want, e_ - s_, what=f"bench parity group {g}")
        else:
            s_, e_ = ranges[g]
            rows = [0, a.shape[1] // 2, a.shape[1] - 1]
            want = (a[g][rows].float() @ b[:, s_:e_].float()).to(got.dtype)
            oracle.assert_close(got[rows][:, s_:e_], want, w["k"], what=f"bench parity group {g}")


def run_workload(name, steps, warmup, torch, dev, path="auto", wall=True, settle_s=0.0):
    """Times one workload on tensors resident in HBM.  Returns (w, record): `record` has the wall-clock time
    over exactly `steps` steps (when `wall`), the per-launch kernel times from HIP events on the launch
    stream, the roofline position and a parity flag.  settle_s > 0 (the short runs of the `configs` object):
    warm up for at least that long and time at least that long, whatever `steps` says -- a kernel of 0.15 ms
    measured for a few milliseconds after the host-side set-up reads the clock ramp, not the kernel."""
    from grouped_mm_bf16_amd import kernels
    from oracle import grouped_mm_oracle as oracle
    w = make_workload(name, torch)
    a, b = w["a"].to(dev), w["b"].to(dev)
    if w.get("b_col"):
        b = b.transpose(-2, -1).contiguous().transpose(-2, -1)
    offs = None
    if w["sizes"] is not None:
        offs = torch.tensor(w["sizes"], dtype=torch.int64).cumsum(0).to(torch.int32).to(dev)
    out = torch.empty(w["out_shape"], device=dev, dtype=w["out_dtype"])

    def step():
        if offs is None:
            w["launch"](a, b, out)
        else:
            w["launch"](a, b, offs, out)

    with kernels.forced_path(path):
        step()
        torch.cuda.synchronize()
        parity_check(w, out, offs, torch, oracle)        # raises on a mismatch: nothing wrong gets timed
        family = kernels.last_path()
        # The parity check above keeps the host busy for seconds while the GPU idles and its clocks fall; the
        # first tens of milliseconds of work after that run 5-15 % slow.  Keep the GPU busy for SETTLE_S
        # first (same launches, untimed), then do the `warmup` steps and time exactly `steps` steps.
        t0 = time.perf_counter()
        n_done = 0
        while time.perf_counter() - t0 < max(settle_s, SETTLE_S):
            for _ in range(10):
                step()
            torch.cuda.synchronize()
            n_done += 10
        if settle_s > 0:
            steps = max(steps, n_done)      # short config runs: as many timed steps as fitted into that interval
        for _ in range(warmup):
            step()
        torch.cuda.synchronize()
        ms_per_step = None
        if wall:
            # whole-job wall clock over exactly `steps` steps
            t0 = time.perf_counter()
            for _ in range(steps):
                step()
            torch.cuda.synchronize()
            ms_per_step = (time.perf_counter() - t0) / steps * 1e3
        # kernel time per launch: one pair of HIP events on the launch stream around the timed region (back-to-back
        # launches, as in the wall-clock loop); a second pass with a pair per step gives the spread (each of
        # those readings also holds the gap that the event markers themselves put between two launches)
        r0, r1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        r0.record()
        for _ in range(steps):
            step()
        r1.record()
        torch.cuda.synchronize()
        k_avg = r0.elapsed_time(r1) / steps
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
        for e0, e1 in evs:
            e0.record()
            step()
            e1.record()
        torch.cuda.synchronize()
        k_ms = [e0.elapsed_time(e1) for e0, e1 in evs]
    if w["bound"] == "hbm":
        achieved, peak, unit = w["bytes"] / (k_avg * 1e-3) / 1e9, PEAK_HBM_GBS, "GB/s"
    else:
        achieved, peak, unit = w["flops"] / (k_avg * 1e-3) / 1e12, PEAK_BF16_TFLOPS, "TFLOP/s"
    traffic, source = measured_traffic(name)
    roof = {"bound": w["bound"], "achieved": round(achieved, 2), "peak": peak, "unit": unit,
            "frac": round(achieved / peak, 4), "traffic": traffic, "traffic_source": source,
            "kernel_ms_avg": round(k_avg, 4), "kernel_ms_min_single": round(min(k_ms), 4),
            "kernel_ms_median_single": round(statistics.median(k_ms), 4),
            "algorithmic_flops": w["flops"], "algorithmic_bytes": w["bytes"]}
    del a, b, out
    return w, {"ms_per_step": ms_per_step, "family": family, "roofline": roof, "parity": "ok", "steps": steps}


MOE_LAYERS = {   # tokens, hidden, inner, experts, top_k
    "moe_mixtral": (8192, 4096, 14336, 8, 2),
    "moe_fine": (4096, 2048, 768, 128, 8),
}


def run_moe(name, steps, warmup, torch, dev):
    """One mixture-of-experts feed-forward layer (routing, gathered up projection with the SwiGLU activation in
    its epilogue, down projection, weighted un-permute), all on the device; kernel time of the whole layer from
    HIP events.  Parity: the first 256 tokens against the oracle (tokens are independent of each other)."""
    from grouped_mm_bf16_amd import moe
    from oracle import grouped_mm_oracle as oracle
    from oracle import moe_oracle
    T, H, I, E, k = MOE_LAYERS[name]
    g = torch.Generator(device=dev).manual_seed(7)
    bf = torch.bfloat16
    x = torch.randn(T, H, generator=g, device=dev).to(bf)
    logits = torch.randn(T, E, generator=g, device=dev)
    if name == "moe_fine":
        logits += 1.5 * torch.randn(E, generator=g, device=dev)      # skewed popularity: empty and tiny experts
    else:
        logits[:, 0] += 1.0
    w_up = (torch.randn(E, H, 2 * I, generator=g, device=dev) * 0.02).to(bf)
    w_down = (torch.randn(E, I, H, generator=g, device=dev) * 0.02).to(bf)
    w_il = moe.interleave_gate_up(w_up)      # done once when weights are loaded: not part of a step
    out = moe.moe_forward(x, logits, w_il, w_down, k, interleaved=True)
    torch.cuda.synchronize()
    n = 256
    want = moe_oracle.moe_forward(x[:n].cpu(), logits[:n].cpu(), w_up.cpu(), w_down.cpu(), k, fused=True)
    del w_up
    oracle.assert_close(out[:n].cpu(), want, I, what=f"bench parity {name}")
    for _ in range(warmup):
        moe.moe_forward(x, logits, w_il, w_down, k, interleaved=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < 0.15:          # let the clocks settle after the host-side parity check
        moe.moe_forward(x, logits, w_il, w_down, k, interleaved=True)
        torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        moe.moe_forward(x, logits, w_il, w_down, k, interleaved=True)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / steps
    flops = 2 * T * k * H * 2 * I + 2 * T * k * I * H
    # algorithmic bytes of the layer: its inputs once (tokens, logits, both weight slabs of every expert that
    # has a token) and its output once; what the stages hand to each other is the implementation's own traffic
    offs = moe.moe_route(logits, k).offs.cpu()
    used = int((torch.diff(offs, prepend=torch.zeros(1, dtype=offs.dtype)) > 0).sum())
    nbytes = T * H * 2 + T * E * 4 + used * (H * 2 * I + I * H) * 2 + T * H * 2
    tflops, gbs = flops / (ms * 1e-3) / 1e12, nbytes / (ms * 1e-3) / 1e9
    hbm_bound = nbytes / PEAK_HBM_GBS > flops / (PEAK_BF16_TFLOPS * 1e3)     # which floor is the higher one
    return {"workload": f"MoE layer: {T} tokens, hidden {H}, inner {I} (SwiGLU in the up projection's epilogue), {E} experts, top {k}, bf16",
            "ms": round(ms, 4), "tflops": round(tflops, 2), "gbs": round(gbs, 1), "bound": "hbm" if hbm_bound else "mfma",
            "frac": round(gbs / PEAK_HBM_GBS if hbm_bound else tflops / PEAK_BF16_TFLOPS, 4),
            "algorithmic_flops": flops, "algorithmic_bytes": nbytes, "experts_with_tokens": used,
            "parity": "ok", "steps": steps}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", default="mixtral",
                    choices=["mixtral", "mixtral_colmajor", "downproj", "readme", "fine", "batched", "batched_colmajor", "kgrouped", "ngrouped", "plain",
                             "copy", "mfma_only", "moe_mixtral", "moe_fine"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-configs", action="store_true",
                    help="skip the short runs of the other benchmark configurations (the `configs` object)")
    ap.add_argument("--library-comparator", action="store_true",
                    help="also time PyTorch-ROCm's own torch.nn.functional.grouped_mm on the same tensors (context only)")
    ap.add_argument("--path", default="auto", choices=["auto", "mfma", "generic"])
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py measures one GPU: grouped_mm has no multi-GPU path in this build "
                         "(run with --gpus 1)")

    import torch
    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a GPU (torch.cuda.is_available() is False)")

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.workload == "copy":
        # plain 1 GiB device copy: the known-size kernel that calibrates rocprof's FETCH_SIZE / WRITE_SIZE
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(args.warmup):
            dst.copy_(src)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            dst.copy_(src)
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) / args.steps * 1e3
        print(json.dumps({"metric": "device copy of 1 GiB (calibration)", "value": round(2 * (1 << 30) / ms / 1e6, 1),
                          "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
                          "ms_per_step": round(ms, 4), "bytes_read": 1 << 30, "bytes_written": 1 << 30}))
        return
    if args.workload == "mfma_only":
        mfma_only(args, torch, dev)
        return
    if args.workload in MOE_LAYERS:
        rec = run_moe(args.workload, args.steps, args.warmup, torch, dev)
        print(json.dumps({"metric": "MoE feed-forward layer, useful TFLOP/s of the two projections", "value": rec["tflops"],
                          "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": rec["ms"],
                          "higher_is_better": True, "dtype": "bf16", "data": "synthetic", "config": rec}))
        return

    w, r = run_workload(args.workload, args.steps, args.warmup, torch, dev, args.path)
    tflops = w["flops"] / (r["ms_per_step"] * 1e-3) / 1e12
    rec = {
        "metric": METRIC, "value": round(tflops, 2), "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(r["ms_per_step"], 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": w["desc"], "kernel_family": r["family"],
                   "pct_bf16_mfma_peak": round(tflops / PEAK_BF16_TFLOPS * 100, 2),
                   "untimed_settle_s_before_warmup": SETTLE_S},
        "roofline": r["roofline"],
    }
    if args.library_comparator:
        # same tensors again (the workload's own were freed with its run)
        a, b = w["a"].to(dev), w["b"].to(dev)
        offs = None if w["sizes"] is None else torch.tensor(w["sizes"]).cumsum(0).to(torch.int32).to(dev)
        rec["library_comparator"] = library_comparator(w, a, b, offs, torch, args.steps)
        del a, b
    if not args.no_cpu_baseline:
        rec["cpu_baseline"] = cpu_baseline(w, torch)
    del w
    if args.workload == "mixtral" and not args.no_configs:
        # The other benchmark configurations, a few steps each (kernel time from HIP events; the headline
        # fields above are the Mixtral workload's alone).
        rec["configs"] = {}
        for name in ("readme", "mixtral_colmajor", "downproj", "batched", "batched_colmajor", "fine", "kgrouped", "ngrouped"):
            try:
                wi, ri = run_workload(name, 30, 10, torch, dev, args.path, wall=False, settle_s=0.15)
                k_avg = ri["roofline"]["kernel_ms_avg"]
                rec["configs"][name] = {
                    "workload": wi["desc"], "kernel_family": ri["family"], "ms": k_avg,
                    "tflops": round(wi["flops"] / (k_avg * 1e-3) / 1e12, 2),
                    "gbs": round(wi["bytes"] / (k_avg * 1e-3) / 1e9, 1),
                    "bound": wi["bound"], "frac": ri["roofline"]["frac"] if wi["bound"] != "latency" else None,
                    "traffic": ri["roofline"]["traffic"], "parity": ri["parity"], "steps": ri["steps"]}
                del wi
            except Exception as ex:   # a config that fails must not take the headline down with it
                rec["configs"][name] = {"parity": "FAILED", "error": repr(ex)[:300]}
        # the layer around the product (routing, gather, activation, un-permute)
        for name in MOE_LAYERS:
            try:
                rec["configs"][name] = run_moe(name, 10, 3, torch, dev)
            except Exception as ex:
                rec["configs"][name] = {"parity": "FAILED", "error": repr(ex)[:300]}
    print(json.dumps(rec))


if __name__ == "__main__":
    main()
