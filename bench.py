#!/usr/bin/env python3
"""Benchmark of the per-device sliced GEMM on one MI355X.

Workload (the headline configuration): GPT-3-like FFN up-projection, one device of a 4x4 mesh, output-stationary:
X[4096,12288] bf16 ~N(0,1), W[12288,12288] bf16 ~N(0,0.02), S=4 block-cyclic slices along K (3072 each,
materialised contiguous in HBM as an all-gather would deliver them), fp32 accumulate -> C[4096,12288] bf16.
One "step" = one ms_gemm_os call over all four slices.  Inputs are resident in HBM before timing starts.

Prints ONE JSON line: whole-job TFLOP/s (`value`), the kernel's roofline fraction measured with HIP events
per launch (`roofline`), and the CPU restatement of the same device body timed on the host cores
(`cpu_baseline`).  Extra keys report the S=1 baseline, the slicing overhead and the LS / RS configurations.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2516.6     # MI355X dense bf16 MFMA: 256 CU x 2.4 GHz x 4096 FLOP/clk/CU
PEAK_FP32_TFLOPS = 157.3      # MI355X dense fp32 MFMA
# Bytes per launch of the config-2 kernel that cross the L2 <-> fabric boundary (Infinity Cache or HBM).  This is an
# OFFLINE figure: two rocprofv3 --pmc runs of this program (FETCH_SIZE and WRITE_SIZE, each scaled by what the same counter
# reads for a 1 GiB device copy in the same run: 2 KiB and 1 KiB per count), valid for the kernel variant named beside it.  It is reported only when the launch this run timed used that variant (ms_query tells).
# HBM-side traffic per config-2 launch from rocprofv3 (FETCH_SIZE x the factor a 1 GiB copy gives in the same run + WRITE_SIZE),
# per kernel variant: a figure measured offline on that kernel, reported only when the run used it
TRAFFIC_PROFILES = {
    12: {"bytes": int(round(688301.0 * 1024 * 1048576 / 524314.0 + 98447.1 * 1024)),
         "source": "profiles/gemm_bf16_x16_256x384x64_os_cfg2.md @ variant 12 (gemm_bf16_x16_kernel, 256x384x64 tile)"},
    10: {"bytes": int(round(698639.1 * 1024 * 1048576 / 524313.19 + 114688 * 1024)),
         "source": "profiles/gemm_bf16_big_256x384x64_os_cfg2.md @ variant 10 (gemm_bf16_big_kernel<4,6>, 256x384x64 tile)"},
}
X16_VARIANTS = (12, 13)         # bf16 kernel variants that issue v_mfma_f32_16x16x32_bf16 (the others: 32x32x16)
SETTLE_LAUNCHES = 60          # untimed launches before the warm-up: the package power controller's start-up transient


def sel_index(L, S, B, k):
    g = np.arange(L)
    return g[(g // B) % S == k]


def make_config2(torch, S):
    g = torch.Generator(device="cuda").manual_seed(0)
    X = torch.randn((4096, 12288), generator=g, device="cuda").to(torch.bfloat16)
    W = (torch.randn((12288, 12288), generator=g, device="cuda") * 0.02).to(torch.bfloat16)
    idx = [torch.from_numpy(sel_index(12288, S, 8, k)).cuda() for k in range(S)]
    A = [X[:, i].contiguous() for i in idx]
    B = [W[i, :].contiguous() for i in idx]
    return X, W, A, B


def median(xs):
    return float(np.median(np.asarray(xs, dtype=np.float64)))


def cpu_baseline(A_host, B_host, flops_full):
    """Time the oracle's CPU device body (per-slice fp32 BLAS loop) on a bounded sample."""
    from oracle import meshslice_oracle as orc
    try:
        from threadpoolctl import threadpool_info, threadpool_limits
    except Exception:  # pragma: no cover
        threadpool_info = threadpool_limits = None
    want = min(16, os.cpu_count() or 1)
    ctx = threadpool_limits(limits=want) if threadpool_limits else None
    try:
        cores = want
        if threadpool_info:
            blas = [p for p in threadpool_info() if p.get("user_api") == "blas"]
            if blas:
                cores = int(blas[0].get("num_threads", want))
        t0 = time.perf_counter()
        orc.cpu_device_body_os(A_host[:1], B_host[:1])          # warm-up on one slice
        t_one = time.perf_counter() - t0
        S = len(A_host)
        if t_one * S > 8.0:      # slow host: time a single slice, three times
            reps, sample_slices = 3, 1
        else:
            reps, sample_slices = 3, S
        ts = []
        for _ in range(reps):
            t0 = time.perf_counter()
            orc.cpu_device_body_os(A_host[:sample_slices], B_host[:sample_slices])
            ts.append(time.perf_counter() - t0)
        sec = median(ts)
        flops = flops_full * sample_slices / S
        return {
            "value": round(flops / sec / 1e12, 4), "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "sample": f"{sample_slices} of {S} slices of the same workload ([4096,3072]x[3072,12288] each), fp32 BLAS on "
                      f"bf16-rounded inputs, 1 warm-up + {reps} reps, median {sec:.3f} s; CPU restatement of the "
                      f"reference device body (JAX is not installable offline)",
            "seconds": round(sec, 4), "os_cpu_count": os.cpu_count(),
        }
    finally:
        if ctx is not None:
            ctx.__exit__(None, None, None)


def power_run(torch, run, flops, seconds, what, variant):
    """Runs `run` back to back for `seconds` while a thread samples `amd-smi metric -p -c`; returns the sustained rate and
    the mean / max of the socket power and of the first graphics clock it printed."""
    import re
    import subprocess
    import threading
    samples, stop = [], threading.Event()

    def sampler():
        while not stop.is_set():
            try:
                samples.append(subprocess.run(["amd-smi", "metric", "-p", "-c"], capture_output=True, text=True, timeout=10).stdout)
            except Exception as e:      # no amd-smi, or no permission: reported as zero samples
                samples.append("")
            time.sleep(0.1)

    th = threading.Thread(target=sampler)
    torch.cuda.synchronize()
    th.start()
    t0, n = time.perf_counter(), 0
    while time.perf_counter() - t0 < seconds:
        for _ in range(50):
            run()
        torch.cuda.synchronize()
        n += 50
    dt = time.perf_counter() - t0
    stop.set()
    th.join()
    watts = [float(m.group(1)) for o in samples[1:] for m in [re.search(r"SOCKET_POWER:\s*([0-9.]+)", o)] if m]
    mhz = [float(m.group(1)) for o in samples[1:] for m in [re.search(r"GFX_0:\s*\n\s*CLK:\s*([0-9.]+)", o)] if m]
    stat = lambda v: {"n": len(v), "mean": round(sum(v) / len(v), 1), "max": max(v)} if v else {"n": 0}
    return {"power_run": what, "kernel_variant": variant, "seconds": round(dt, 2), "launches": n, "tflops": round(flops * n / dt / 1e12, 1),
            "socket_power_w": stat(watts), "gfx_clk_mhz": stat(mhz)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=300)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the CPU leg (profiling runs)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also launch one 1 GiB device copy (scales rocprofv3 FETCH_SIZE / WRITE_SIZE)")
    ap.add_argument("--only-main", action="store_true", help="skip the S=1 / LS / RS side measurements")
    ap.add_argument("--kernel-only", choices=("os", "ls", "rs", "fp32"), default=None,
                    help="profiling runs: launch only the kernel of configuration 2 (os), 3 (ls) or 4 (rs), or the fp32 kernel "
                         "on 4096^3, and print its time")
    ap.add_argument("--power", type=float, default=0.0, metavar="SECONDS",
                    help="with --kernel-only: run the kernel back to back for SECONDS while sampling `amd-smi metric -p -c` "
                         "(socket power, graphics clock) and print their mean / max")
    ap.add_argument("--ones", action="store_true", help="with --kernel-only os: all-ones operands (the reference's timing operands)")
    ap.add_argument("--variant", type=int, default=0, help="profiling runs: force a bf16 kernel variant (ms_set_variant), 0 = library's choice")
    ap.add_argument("--shape", default=None, metavar="M,N,K",
                    help="with --kernel-only os: one unsliced bf16 product of this shape instead of configuration 2")
    ap.add_argument("--reserve", type=int, default=0, help="profiling runs: compute units the kernels leave free (ms_set_reserved_cus)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures ONE mesh device's local GEMM on ONE GPU; --gpus > 1 is not part of this build "
              "(the mesh is emulated on the host, no collectives are built).", file=sys.stderr)
        sys.exit(2)

    import torch
    import meshslice_amd as ms
    from meshslice_amd import _lib
    from oracle import meshslice_oracle as orc

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    lib = _lib.load()
    torch.cuda.set_device(0)
    S = 4
    M, N, K = 4096, 12288, 12288
    flops = 2.0 * M * N * K
    X, W, A, B = make_config2(torch, S)
    C = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")

    if args.copy_calibration:
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    if args.variant:
        _lib.check(lib.ms_set_variant(args.variant))
    if args.reserve:
        _lib.check(lib.ms_set_reserved_cus(args.reserve))

    if args.kernel_only:
        # one configuration's kernel alone, for the profiler: settle + warm-up + steps back-to-back launches
        if args.kernel_only == "os" and args.shape:
            m_, n_, k_ = (int(v) for v in args.shape.split(","))
            g = torch.Generator(device="cuda").manual_seed(6)
            Ax = [torch.randn((m_, k_), generator=g, device="cuda").to(torch.bfloat16)]
            Bx = [(torch.randn((k_, n_), generator=g, device="cuda") * 0.02).to(torch.bfloat16)]
            Cx = torch.empty((m_, n_), dtype=torch.bfloat16, device="cuda")
            run, fl = (lambda: ms.gemm_os(Ax, Bx, out=Cx)), 2.0 * m_ * n_ * k_
        elif args.kernel_only == "os":
            run, fl = (lambda: ms.gemm_os(A, B, out=C)), flops
        elif args.kernel_only == "ls":
            Ws = [W[torch.from_numpy(sel_index(12288, 8, 8, k)).cuda(), :].contiguous() for k in range(8)]
            Y = [torch.empty((4096, 1536), dtype=torch.float32, device="cuda") for _ in range(8)]
            run, fl = (lambda: ms.gemm_ls(X, Ws, out=Y)), flops
        elif args.kernel_only == "fp32":
            g = torch.Generator(device="cuda").manual_seed(5)
            A32 = torch.randn((4096, 4096), generator=g, device="cuda")
            B32 = torch.randn((4096, 4096), generator=g, device="cuda") * 0.02
            C32 = torch.empty((4096, 4096), dtype=torch.float32, device="cuda")
            run, fl = (lambda: ms.gemm_os([A32], [B32], out=C32)), 2.0 * 4096 ** 3
        else:
            g = torch.Generator(device="cuda").manual_seed(4)
            X4 = torch.randn((4096, 3072), generator=g, device="cuda").to(torch.bfloat16)
            dY = (torch.randn((4096, 12288), generator=g, device="cuda") * 1e-3).to(torch.bfloat16)
            Xs = [X4[:, torch.from_numpy(sel_index(3072, 4, 8, k)).cuda()].contiguous() for k in range(4)]
            Y = [torch.empty((768, 12288), dtype=torch.float32, device="cuda") for _ in range(4)]
            run, fl = (lambda: ms.gemm_rs(Xs, dY, out=Y)), 2.0 * 3072 * 12288 * 4096
        if args.ones and args.kernel_only == "os":
            A = [torch.ones_like(a) for a in A]
            B = [torch.ones_like(b) for b in B]
            run = lambda: ms.gemm_os(A, B, out=C)
        for _ in range(SETTLE_LAUNCHES + args.warmup):
            run()
        if args.power > 0:
            print(json.dumps(power_run(torch, run, fl, args.power, args.kernel_only, int(lib.ms_query(_lib.MS_QUERY_LAST_VARIANT)))), flush=True)
            return
        e0 = torch.cuda.Event(enable_timing=True); e1 = torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(args.steps):
            run()
        e1.record()
        torch.cuda.synchronize()
        t = e0.elapsed_time(e1) / args.steps
        print(json.dumps({"kernel_only": args.kernel_only, "kernel_variant": int(lib.ms_query(_lib.MS_QUERY_LAST_VARIANT)),
                          "splits": int(lib.ms_query(_lib.MS_QUERY_LAST_SPLITS)), "steps": args.steps, "kernel_ms_mean": round(t, 4),
                          "tflops": round(fl / t / 1e9, 1),
                          "frac_of_peak": round(fl / t / 1e9 / (PEAK_FP32_TFLOPS if args.kernel_only == "fp32" else PEAK_BF16_TFLOPS), 4)}), flush=True)
        return

    # ---- settle phase (always, whatever --warmup says): the first launches after an idle period run up to 30 % slow
    for _ in range(SETTLE_LAUNCHES):
        ms.gemm_os(A, B, out=C)
    torch.cuda.synchronize()
    variant = int(lib.ms_query(_lib.MS_QUERY_LAST_VARIANT))
    launches = int(lib.ms_query(_lib.MS_QUERY_LAST_LAUNCHES))

    # ---- timed region: W warm-up steps, then exactly K steps between two synchronisations; two HIP events on the
    # launch stream bracket the same K launches, so their mean is the kernel's duration in THIS region
    for _ in range(args.warmup):
        ms.gemm_os(A, B, out=C)
    e0 = torch.cuda.Event(enable_timing=True); e1 = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        ms.gemm_os(A, B, out=C)
    e1.record()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    value = flops / (ms_per_step * 1e-3) / 1e12
    k_ms = e0.elapsed_time(e1) / args.steps

    # the same launches bracketed one by one (each followed by a host wait, which lets the device idle between
    # launches: these read a little differently from back-to-back launches and are reported for information)
    per_launch = ms.time_call("os", (A, B), C, warmup=2, reps=min(max(args.steps, 10), 100))
    achieved = flops / (k_ms * 1e-3) / 1e12
    traffic_ok = variant in TRAFFIC_PROFILES and launches == 1
    TRAFFIC_PROFILE = TRAFFIC_PROFILES.get(variant, {})
    roofline = {"bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                "frac": round(achieved / PEAK_BF16_TFLOPS, 4),
                "traffic": TRAFFIC_PROFILE["bytes"] if traffic_ok else None,
                "traffic_source": TRAFFIC_PROFILE["source"] if traffic_ok else
                f"none: this run launched variant {variant} ({launches} launch(es)), the profiles cover variants {sorted(TRAFFIC_PROFILES)} as one launch",
                "kernel_variant": variant,
                "kernel_ms_mean": round(k_ms, 4), "kernel_ms_how": f"two HIP events on the launch stream around the {args.steps} timed launches",
                "kernel_ms_single_launch_mean": round(float(np.mean(per_launch)), 4),
                "kernel_ms_single_launch_min": round(float(np.min(per_launch)), 4),
                "algorithmic_flops_per_launch": flops,
                "algorithmic_hbm_bytes_per_launch": 2 * (M * K + K * N + M * N)}

    extra = {}
    # parity spot check of the benchmarked output against the float64 oracle on sampled rows
    rows = np.random.default_rng(0).choice(M, 16, replace=False)
    want = X[rows].float().cpu().numpy().astype(np.float64) @ W.float().cpu().numpy().astype(np.float64)
    extra["parity_rel_frobenius_sampled_rows"] = float(f"{orc.rel_frobenius(C[rows].float().cpu().numpy(), want):.3e}")

    def _sustained(f, n, warm=10):
        """mean ms per launch of n back-to-back launches between two HIP events on the launch stream"""
        for _ in range(warm):
            f()
        a = torch.cuda.Event(enable_timing=True); b = torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(n):
            f()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / n

    # Every side leg is measured like the main one, whatever --steps and --warmup say: SETTLE_LAUNCHES launches of THAT
    # kernel first (fresh allocations, another kernel's power state and a cold instruction cache cost the first launches
    # up to 30 %), then SIDE_TIMED back-to-back launches between two HIP events; the legs are gone through twice
    # (A B C A B C) and each reports its better round.  With a leg length that followed --steps, a 20-step run timed
    # configuration 4 on 40 launches right after its buffers were made and read 0.270 ms where the sustained figure is
    # 0.227 ms.
    SIDE_TIMED = 200

    def _legs(fs):
        best = [float("inf")] * len(fs)
        for _ in range(2):
            for i, f in enumerate(fs):
                best[i] = min(best[i], _sustained(f, SIDE_TIMED, warm=SETTLE_LAUNCHES))
        return best

    out_extra = {}
    if not args.only_main:
        # S = 1 against S = 4, measured the same way and interleaved (A B A B), best of each
        C1 = torch.empty_like(C)
        t_s4, t_s1 = _legs([lambda: ms.gemm_os(A, B, out=C), lambda: ms.gemm_os([X], [W], out=C1)])
        extra["os_s1_ms"] = round(t_s1, 4)
        extra["os_s4_ms"] = round(t_s4, 4)
        extra["os_s1_tflops"] = round(flops / t_s1 / 1e9, 1)
        extra["slicing_overhead_s4_vs_s1"] = round(t_s4 / t_s1 - 1.0, 4)
        del C1
        # config 3: LS, S=8 -> 8 fp32 chunks [4096,1536]; config 4: RS, S=4 -> 4 fp32 chunks [768,12288]; fp32 4096^3
        idx8 = [torch.from_numpy(sel_index(12288, 8, 8, k)).cuda() for k in range(8)]
        Ws = [W[i, :].contiguous() for i in idx8]
        Yl = [torch.empty((4096, 1536), dtype=torch.float32, device="cuda") for _ in range(8)]
        g = torch.Generator(device="cuda").manual_seed(4)
        X4 = torch.randn((4096, 3072), generator=g, device="cuda").to(torch.bfloat16)
        dY = (torch.randn((4096, 12288), generator=g, device="cuda") * 1e-3).to(torch.bfloat16)
        idx4 = [torch.from_numpy(sel_index(3072, 4, 8, k)).cuda() for k in range(4)]
        Xs = [X4[:, i].contiguous() for i in idx4]
        Yr = [torch.empty((768, 12288), dtype=torch.float32, device="cuda") for _ in range(4)]
        Yr16 = [torch.empty((768, 12288), dtype=torch.bfloat16, device="cuda") for _ in range(4)]
        fl4 = 2.0 * 3072 * 12288 * 4096
        g = torch.Generator(device="cuda").manual_seed(1)
        A32 = torch.randn((4096, 4096), generator=g, device="cuda"); B32 = torch.randn((4096, 4096), generator=g, device="cuda")
        C32 = torch.empty((4096, 4096), device="cuda")
        variants = {}

        def _named(name, f):
            def run():
                f()
                variants[name] = int(lib.ms_query(_lib.MS_QUERY_LAST_VARIANT))
            return run
        t_ls, t_rs, t_rs16, t_f32, t_f32_vendor = _legs([
            _named("ls", lambda: ms.gemm_ls(X, Ws, out=Yl)), _named("rs", lambda: ms.gemm_rs(Xs, dY, out=Yr)),
            _named("rs16", lambda: ms.gemm_rs(Xs, dY, out=Yr16)),
            lambda: ms.gemm_os([A32], [B32], out=C32), lambda: torch.matmul(A32, B32, out=C32)])
        extra["ls_s8_ms"] = round(t_ls, 4); extra["ls_s8_tflops"] = round(flops / t_ls / 1e9, 1)
        out_extra["roofline_ls"] = {"workload": "config 3: LS, A[4096,12288] x 8 slices W_s[1536,12288]^T -> 8 fp32 chunks", "bound": "mfma",
                                    "achieved": round(flops / t_ls / 1e9, 2), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                                    "frac": round(flops / t_ls / 1e9 / PEAK_BF16_TFLOPS, 4), "kernel_ms_mean": round(t_ls, 4),
                                    "kernel_variant": variants["ls"], "launches_timed": SIDE_TIMED}
        extra["rs_s4_ms"] = round(t_rs, 4); extra["rs_s4_tflops"] = round(fl4 / t_rs / 1e9, 1)
        out_extra["roofline_rs"] = {"workload": "config 4: RS, 4 slices X_s[4096,768]^T x dY[4096,12288] -> 4 fp32 chunks", "bound": "mfma",
                                    "achieved": round(fl4 / t_rs / 1e9, 2), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                                    "frac": round(fl4 / t_rs / 1e9 / PEAK_BF16_TFLOPS, 4), "kernel_ms_mean": round(t_rs, 4),
                                    "kernel_variant": variants["rs"], "launches_timed": SIDE_TIMED,
                                    # the reference's own chunk dtype (its einsum returns the operands' dtype, TensorParallel.py:200-212)
                                    "bf16_chunks": {"kernel_ms_mean": round(t_rs16, 4), "achieved": round(fl4 / t_rs16 / 1e9, 2),
                                                    "frac": round(fl4 / t_rs16 / 1e9 / PEAK_BF16_TFLOPS, 4), "kernel_variant": variants["rs16"]}}
        extra["vendor_library_fp32_4096_ms"] = round(t_f32_vendor, 4)
        out_extra["roofline_fp32"] = {"workload": "fp32 4096 x 4096 x 4096, one slice", "bound": "mfma",
                                      "achieved": round(2.0 * 4096 ** 3 / t_f32 / 1e9, 2), "peak": PEAK_FP32_TFLOPS, "unit": "TFLOP/s",
                                      "frac": round(2.0 * 4096 ** 3 / t_f32 / 1e9 / PEAK_FP32_TFLOPS, 4), "kernel_ms_mean": round(t_f32, 4),
                                      "launches_timed": SIDE_TIMED}
        del Ws, Yl, Xs, Yr, Yr16, X4, dY, A32, B32, C32
        # the fp32 path on config 1 (device block 512x512x1024 in four K slices)
        g = torch.Generator(device="cuda").manual_seed(1)
        A1 = [torch.randn((512, 256), generator=g, device="cuda") for _ in range(4)]
        B1 = [torch.randn((256, 512), generator=g, device="cuda") for _ in range(4)]
        C32 = torch.empty((512, 512), device="cuda")
        # (launches this short are bound by the host's call rate, and one stall of the host thread inside a loop reads as
        # a many times slower kernel: best of three loops)
        t = min(_sustained(lambda: ms.gemm_os(A1, B1, out=C32), 200) for _ in range(3))
        extra["fp32_config1_ms"] = round(t, 5); extra["fp32_config1_tflops"] = round(2.0 * 512 * 512 * 1024 / t / 1e9, 2)
        del A1, B1, C32
        # fused epilogue: GELU folded into the config-2 product vs the product followed by a separate GELU kernel; the vendor
        # library's GEMM (hipBLASLt through torch.matmul) on the same un-sliced operands, same box, for scale; and one device's
        # whole output-stationary step on a 4x4 mesh: cut its own X shard [4096, 3072] and W shard [3072, 12288] into the S
        # slices it sends to its peers (the peers' slices arrive by all-gather), then the sliced GEMM.  All measured like the
        # other legs: launches back to back between two HIP events after a settle phase (a launch timed alone, the device
        # idling before it, reads 3-15 % longer and says little about a training step).
        from meshslice_amd.slice_layout import measure_rates, pack_slices
        Xown, Wown = X[:, :K // 4].contiguous(), W[:K // 4, :].contiguous()
        xs = pack_slices(Xown, S, 8, 1); ws = pack_slices(Wown, S, 8, 0)

        def _device_step():
            pack_slices(Xown, S, 8, 1, out=xs)
            pack_slices(Wown, S, 8, 0, out=ws)
            ms.gemm_os(A, B, out=C)
        torch.matmul(X, W)
        # the same product behind its input gate with every slice already flagged: what the gate itself costs
        flags = torch.ones(S + 1, dtype=torch.int32, device=C.device); flags[S] = 0
        t_plain, t_gelu, t_sep, t_vendor, t_step, t_gated = _legs([
            lambda: ms.gemm_os(A, B, out=C), lambda: ms.gemm_os(A, B, out=C, activation="gelu"),
            lambda: torch.nn.functional.gelu(ms.gemm_os(A, B, out=C), approximate="tanh"),
            lambda: torch.matmul(X, W), _device_step, lambda: ms.gemm_os_gated(A, B, flags, out=C)])
        extra["os_s4_gated_all_slices_flagged_ms"] = round(t_gated, 4)
        extra["os_s4_fused_gelu_ms"] = round(t_gelu, 4)
        extra["os_s4_then_separate_gelu_ms"] = round(t_sep, 4)
        extra["vendor_library_matmul_s1_ms"] = round(t_vendor, 4)
        extra["os_s4_device_step_ms"] = round(t_step, 4)
        extra["os_s4_gemm_alone_same_method_ms"] = round(t_plain, 4)
        # the layout kernels either side of the GEMM on the same [4096, 12288] bf16 shard: algorithmic GB/s (HBM roofline 8000)
        for label, t, nbytes in measure_rates(dtypes=(torch.bfloat16,), reduce_case=False, reps=24):
            key = "layout_" + label.replace("bfloat16 ", "").replace(" of the shard", "").replace("=", "").replace(" ", "_").lower() + "_gbps"
            extra[key] = round(nbytes / t / 1e9, 0)
        # what this device sustains on a bare stream of one MFMA instruction (no memory traffic) for operands drawn
        # like X: the practical, power-limited ceiling beside the data-sheet peak.  Both bf16 shapes are measured; the
        # ceiling the timed kernel is held against is that of the instruction it issues (variant 12: 16x16x32).
        from meshslice_amd.local_gemm import mfma_stream_rate
        probe_ops = X[:16, :512].contiguous().reshape(-1)
        stream_tf = {shape: mfma_stream_rate(probe_ops, shape=shape) / 1e12 for shape in ("32x32x16", "16x16x32")}
        used = "16x16x32" if variant in X16_VARIANTS else "32x32x16"
        extra["mfma_stream_tflops_32x32x16"] = round(stream_tf["32x32x16"], 1)
        extra["mfma_stream_tflops_16x16x32"] = round(stream_tf["16x16x32"], 1)
        extra["mfma_stream_ceiling_instruction"] = used
        extra["mfma_stream_ceiling_tflops"] = round(stream_tf[used], 1)
        extra["achieved_over_mfma_stream_ceiling"] = round(value / stream_tf[used], 4)

    out = {
        "metric": "per-device sliced GEMM throughput (GPT-3 FFN up-proj, output-stationary, S=4)",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "GPT-3-like FFN up-projection: one device of a 4x4 mesh, OS, X[4096,12288] x W[12288,12288] bf16, "
                               "S=4 block-cyclic K slices of 3072, fp32 accumulate, C[4096,12288] bf16",
                   "S": S, "m": M, "n": N, "k_slice": K // S, "blocksize": 8},
        "pct_of_bf16_mfma_peak": round(100.0 * value / PEAK_BF16_TFLOPS, 2),
        "settle_launches": SETTLE_LAUNCHES,
        "roofline": roofline,
    }
    out.update(out_extra)
    if not args.no_cpu_baseline:
        A_host = [a.float().cpu().numpy() for a in A]
        B_host = [b.float().cpu().numpy() for b in B]
        out["cpu_baseline"] = cpu_baseline(A_host, B_host, flops)
    else:
        out["cpu_baseline"] = None
    out["extra"] = extra
    out["device"] = {"cus": int(lib.ms_query(_lib.MS_QUERY_CU_COUNT)), "clock_khz": int(lib.ms_query(_lib.MS_QUERY_CLOCK_KHZ))}
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
