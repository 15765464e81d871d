"""Yardsticks for the tile choosers and the kernels behind them, on products outside the GPT-3 family.

``python3 -m meshslice_amd.compare vendor [--small]``
    this build's one-slice bf16 product (bf16 in and out) beside the vendor library's (``torch.matmul``) for the three
    operand layouts nn / nt / tn, i.e. the OS / LS / RS entry points with one slice, on cubes and a few tall, wide and
    long shapes (``--small``: ten products from 1024^3 to 3072^3).

``python3 -m meshslice_amd.compare chooser [--cases N] [--slices S] [--seed K]``
    how far the default tile choice is from the best of ten forced tile variants, on N shapes drawn at random per
    dataflow (dimensions 512..16384, 0.02..3 TFLOP per product), S slices each.

``python3 -m meshslice_amd.compare fp32``
    the fp32 kernel's default choice (tile and split count), each of its five tiles forced (ids 21..25, each with the
    split count the library would take for it) and the vendor library's product, output-stationary, on ten products
    from 512 x 512 x 1024 to 4096^3.

Every time is the mean of back-to-back launches between two HIP events after warm-up launches (a launch timed alone,
the device idling before it, reads 3-15 % longer); one line per case, then a JSON summary.  The measurement protocol
of the reference's cost model (CostModel.py:74-98) times one call at a time instead."""
import argparse
import json
import random
import statistics
import sys

import torch

from . import _lib
from .local_gemm import gemm_ls, gemm_os, gemm_rs

LARGE = [(1024,) * 3, (2048,) * 3, (3072,) * 3, (4096,) * 3, (5120,) * 3, (6144,) * 3, (8192,) * 3, (4096, 14336, 4096), (4096, 4096, 14336),
         (8192, 8192, 2048), (2048, 8192, 8192), (4096, 11008, 4096), (16384, 4096, 4096)]
SMALL = [(1024,) * 3, (1536,) * 3, (2048,) * 3, (2560,) * 3, (3072,) * 3, (2048, 4096, 2048), (2048, 2048, 8192), (1024, 4096, 4096),
         (2048, 1536, 3072), (4096, 1536, 1536)]
FORCED = (3, 5, 6, 7, 8, 9, 11, 12, 13, 14)
SIZES = [512, 768, 1024, 1536, 2048, 2560, 3072, 4096, 5120, 6144, 7168, 8192, 10240, 12288, 16384]


def _normal(shape, scale, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return (torch.randn(shape, generator=g, device="cuda") * scale).to(torch.bfloat16)


def _sustained_us(f, warm, steps):
    for _ in range(warm):
        f()
    a = torch.cuda.Event(enable_timing=True); b = torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(steps):
        f()
    b.record(); torch.cuda.synchronize()
    return a.elapsed_time(b) / steps * 1e3


def _call(flow, m, n, k, S, with_vendor=False):
    """(this build's call, the vendor library's call or None) for C[m, n] over contraction k in S slices, bf16 outputs."""
    if flow == "os":
        A = [_normal((m, k // S), 1.0, s) for s in range(S)]; B = [_normal((k // S, n), 0.02, 10 + s) for s in range(S)]
        C = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
        return (lambda: gemm_os(A, B, out=C)), ((lambda: torch.matmul(A[0], B[0], out=C)) if with_vendor else None)
    if flow == "ls":
        A = _normal((m, k), 1.0, 1); W = [_normal((n // S, k), 0.02, 10 + s) for s in range(S)]
        Y = [torch.empty((m, n // S), dtype=torch.bfloat16, device="cuda") for _ in range(S)]
        return (lambda: gemm_ls(A, W, out=Y)), ((lambda: torch.matmul(A, W[0].T, out=Y[0])) if with_vendor else None)
    X = [_normal((k, m // S), 1.0, s) for s in range(S)]; W = _normal((k, n), 0.02, 9)
    Y = [torch.empty((m // S, n), dtype=torch.bfloat16, device="cuda") for _ in range(S)]
    return (lambda: gemm_rs(X, W, out=Y)), ((lambda: torch.matmul(X[0].T, W, out=Y[0])) if with_vendor else None)


def _settle():
    """Half a second of work before the first case: both libraries' one-time set-up and the device's ramp from idle."""
    ours, theirs = _call("os", 4096, 4096, 4096, 1, with_vendor=True)
    for _ in range(3):
        _sustained_us(ours, 10, 200)
        _sustained_us(theirs, 10, 200)


def vendor(shapes):
    lib = _lib.load()
    _settle()
    ratios = {}
    for lay, flow in (("nn", "os"), ("nt", "ls"), ("tn", "rs")):
        for (m, n, k) in shapes:
            ours, theirs = _call(flow, m, n, k, 1, with_vendor=True)
            # the two take turns, and each reports its better turn: after a product of a few microseconds the device has
            # clocked down, and whichever is timed first pays for that
            t = tv = float("inf")
            for _ in range(2):
                t = min(t, _sustained_us(ours, 40, 100))
                v, s = lib.ms_query(_lib.MS_QUERY_LAST_VARIANT), lib.ms_query(_lib.MS_QUERY_LAST_SPLITS)
                tv = min(tv, _sustained_us(theirs, 40, 100))
            fl = 2.0 * m * n * k
            ratios.setdefault(lay, []).append(tv / t)
            print(f"{lay} {m}x{n}x{k}: this build {t:.0f} us {fl / t / 1e6:.0f} TFLOP/s (variant {v}, {s} split) | vendor {tv:.0f} us "
                  f"{fl / tv / 1e6:.0f} TFLOP/s | vendor time / this build's {tv / t:.3f}", flush=True)
    return {lay: {"cases": len(r), "geometric_mean": round(statistics.geometric_mean(r), 3), "min": round(min(r), 3), "max": round(max(r), 3),
                  "slower_than_vendor": sum(x < 1.0 for x in r)} for lay, r in ratios.items()}


def chooser(cases, S, seed):
    lib = _lib.load()
    rnd = random.Random(seed)
    shapes = []
    while len(shapes) < cases:
        m, n, k = (rnd.choice(SIZES) for _ in range(3))
        if 2.0 * m * n * k < 2e10 or 2.0 * m * n * k > 3e12 or (m * k + k * n + m * n) * 2 > 2e9:
            continue
        shapes.append((m, n, k))
    out = {}
    _settle()
    for flow in ("os", "ls", "rs"):
        ratios = []
        for (m, n, k) in shapes:
            if (n if flow == "ls" else m if flow == "rs" else k) % (S * 64):
                continue
            f, _ = _call(flow, m, n, k, S)
            try:
                lib.ms_set_variant(0)
                t0 = _sustained_us(f, 25, 40)
                v0, s0 = lib.ms_query(_lib.MS_QUERY_LAST_VARIANT), lib.ms_query(_lib.MS_QUERY_LAST_SPLITS)
                forced = {}
                for v in FORCED:
                    lib.ms_set_variant(v)
                    forced[v] = _sustained_us(f, 8, 20)
                lib.ms_set_variant(0)
                t0 = min(t0, _sustained_us(f, 25, 40))
            finally:
                lib.ms_set_variant(0)
            best = min(forced, key=forced.get)
            ratios.append(t0 / forced[best])
            print(f"{flow} {m}x{n}x{k} S={S}: default variant {v0} ({s0} split) {t0:.0f} us | best forced {best}: {forced[best]:.0f} us | "
                  f"ratio {t0 / forced[best]:.3f} | " + " ".join(f"{v}:{t:.0f}" for v, t in forced.items()), flush=True)
        out[flow] = {"cases": len(ratios), "mean": round(statistics.mean(ratios), 3), "max": round(max(ratios), 3),
                     "beyond_3_percent": sum(r > 1.03 for r in ratios), "beyond_6_percent": sum(r > 1.06 for r in ratios)}
    return out


FP32_SHAPES = [(4096, 4096, 4096), (8192, 2048, 2048), (3072, 3072, 4096), (2048, 3072, 4096), (2048, 6144, 2048), (2048, 2048, 8192),
               (1536, 1536, 4096), (1024, 2048, 4096), (1024, 1024, 1024), (512, 512, 1024)]
FP32_TILES = (21, 22, 23, 24, 25)      # 256x128, 128x192 (eight waves), 128x128, 64x64, 192x192 (four waves)


def fp32(shapes=FP32_SHAPES):
    lib = _lib.load()
    _settle()
    ratios, off = [], []
    for (m, n, k) in shapes:
        g = torch.Generator(device="cuda").manual_seed(m + n + k)
        A = torch.randn((m, k), generator=g, device="cuda"); B = torch.randn((k, n), generator=g, device="cuda") * 0.02
        C = torch.empty((m, n), device="cuda")
        ours = lambda: gemm_os([A], [B], out=C)
        theirs = lambda: torch.matmul(A, B, out=C)
        times, what = {}, {}
        try:
            for _ in range(2):
                for v in (0,) + FP32_TILES:
                    lib.ms_set_variant(v)
                    t = _sustained_us(ours, 15, 40)
                    times[v] = min(times.get(v, t), t)
                    what[v] = (int(lib.ms_query(_lib.MS_QUERY_LAST_VARIANT)), int(lib.ms_query(_lib.MS_QUERY_LAST_SPLITS)))
                lib.ms_set_variant(0)
                tv = _sustained_us(theirs, 15, 40)
                times["vendor"] = min(times.get("vendor", tv), tv)
        finally:
            lib.ms_set_variant(0)
        best = min(FP32_TILES, key=lambda v: times[v])
        fl = 2.0 * m * n * k
        ratios.append(times["vendor"] / times[0]); off.append(times[0] / times[best])
        print(f"fp32 {m}x{n}x{k}: default tile {what[0][0]} x{what[0][1]} {times[0]:.0f} us {fl / times[0] / 1e6:.1f} TFLOP/s | forced "
              + " ".join(f"{v}(x{what[v][1]}):{times[v]:.0f}" for v in FP32_TILES) + f" | vendor {times['vendor']:.0f} us | vendor time / this build's "
              f"{times['vendor'] / times[0]:.3f}", flush=True)
    return {"cases": len(ratios), "vendor_over_ours_geometric_mean": round(statistics.geometric_mean(ratios), 3), "min": round(min(ratios), 3),
            "max": round(max(ratios), 3), "default_over_best_tile_max": round(max(off), 3)}


def main(argv=None) -> None:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    sub = ap.add_subparsers(dest="what", required=True)
    pv = sub.add_parser("vendor"); pv.add_argument("--small", action="store_true")
    pc = sub.add_parser("chooser")
    sub.add_parser("fp32")
    pc.add_argument("--cases", type=int, default=60); pc.add_argument("--slices", type=int, default=2); pc.add_argument("--seed", type=int, default=5)
    args = ap.parse_args(argv)
    torch.cuda.set_device(0)
    res = vendor(SMALL if args.small else LARGE) if args.what == "vendor" else fp32() if args.what == "fp32" else chooser(args.cases, args.slices, args.seed)
    print(json.dumps({args.what: res}), flush=True)


if __name__ == "__main__":
    main(sys.argv[1:])
