"""Measurement aids of libmeshslice_hip.so on the current GPU: what bounds the output-stationary bf16 kernel.

Three probes, each a thin wrapper over one C entry point, and a command line that prints them as one JSON object:

* ``os_parts``: BASELINE's configuration 2 (or any output-stationary bf16 product) on the 256x384x64 kernel of the
  16x16x32 MFMA with parts of its K loop left out (``ms_probe_os_parts``): the whole kernel, without its global -> LDS
  loads, without its fragment reads, the MFMAs alone, the operand stream alone, without the wait / the barrier of a
  K step;
* ``l2_lds_stream``: a bare L2 -> LDS stream of direct-to-LDS loads whose data sits in the L2s
  (``ms_probe_l2_lds_stream``);
* ``mfma_stream``: a bare stream of one bf16 MFMA instruction on register-resident operands
  (``ms_probe_mfma_stream_ex``, see local_gemm.mfma_stream_rate).

``python -m meshslice_amd.probes [--ones] [--resident] [--power SECONDS]`` runs all three; ``--ones`` uses all-ones
operands (the reference's timing operands, CostModel.py:78-79: the device then stays below its power limit),
``--resident`` adds the first probe on a product whose operands stay in the L2s, ``--power`` samples
``amd-smi metric -p -c`` while each kernel runs back to back (and once with the device idle).
"""
from __future__ import annotations

import argparse
import ctypes
import json
import re
import subprocess
import threading
import time
from typing import Dict, List, Optional, Sequence

import torch

from . import _lib
from .local_gemm import _prepare_os, _stream, mfma_stream_rate

PEAK_BF16_FLOPS = 2.5166e15      # MI355X dense bf16 MFMA: 256 CU x 2.4 GHz x 4096 FLOP/clk/CU
SKIP_LOADS, SKIP_FRAGS, SKIP_MFMA, SKIP_VMWAIT, SKIP_BARRIER = 1, 2, 4, 8, 16
PARTS = (
    (0, "whole kernel"),
    (SKIP_VMWAIT, "no wait for the loads before a step's barrier"),
    (SKIP_BARRIER, "no barrier in the K loop"),
    (SKIP_VMWAIT | SKIP_BARRIER, "neither wait nor barrier"),
    (SKIP_FRAGS, "no fragment reads (LDS -> registers)"),
    (SKIP_LOADS, "no global -> LDS loads"),
    (SKIP_LOADS | SKIP_FRAGS, "MFMAs alone (tile loop, prologue and write-out kept)"),
    (SKIP_MFMA, "operand stream alone (no MFMAs, no fragment reads)"),
)


def os_parts_ms(skip: int, A_slices: Sequence[torch.Tensor], B_slices: Sequence[torch.Tensor], out: torch.Tensor,
                warmup: int = 60, reps: int = 200) -> float:
    """Mean milliseconds per launch of the output-stationary 16x16x32 kernel with the parts in ``skip`` left out
    (``ms_probe_os_parts``); operands and ``out`` as for gemm_os, all bf16.  ``out`` is scratch when ``skip != 0``."""
    call = _prepare_os(A_slices, B_slices, out, None)
    if A_slices[0].dtype != torch.bfloat16 or out.dtype != torch.bfloat16:
        raise ValueError("the probe runs the bf16-in / bf16-out kernel")
    ms = ctypes.c_float(0.0)
    with torch.cuda.device(call.device):
        rc = _lib.load().ms_probe_os_parts(int(skip), *call.args[:10], int(warmup), int(reps), ctypes.byref(ms), _stream())
    _lib.check(rc)
    return float(ms.value)


def l2_lds_stream_rate(region_steps: int = 24, in_flight_steps: int = 2, steps: int = 2000, warmup: int = 3, reps: int = 10) -> Dict[str, float]:
    """Bytes per second of a bare L2 -> LDS stream on the current GPU (``ms_probe_l2_lds_stream``): ``region_steps`` x 80 KB
    per XCD, read round and round by all of its compute units (24 steps = 1.9 MB: L2 hits)."""
    dev = torch.device("cuda", torch.cuda.current_device())
    nbytes = 8 * int(region_steps) * 81920
    buf = torch.ones(nbytes // 2, dtype=torch.bfloat16, device=dev)
    sink = torch.zeros(1, dtype=torch.float32, device=dev)
    ms, moved = ctypes.c_float(0.0), ctypes.c_double(0.0)
    rc = _lib.load().ms_probe_l2_lds_stream(ctypes.c_void_p(buf.data_ptr()), nbytes, int(region_steps), int(in_flight_steps), int(steps),
                                            int(warmup), int(reps), ctypes.c_void_p(sink.data_ptr()), ctypes.byref(ms), ctypes.byref(moved), _stream())
    _lib.check(rc)
    cus = int(_lib.load().ms_query(_lib.MS_QUERY_CU_COUNT))
    sec = ms.value * 1e-3
    return {"bytes_per_s": moved.value / sec, "bytes_per_s_per_cu": moved.value / sec / cus, "us_per_80KB_step": ms.value * 1e3 / steps,
            "region_bytes_per_xcd": region_steps * 81920, "in_flight_steps": in_flight_steps}


class _PowerSampler:
    """Samples ``amd-smi metric -p -c`` (socket power, first graphics clock) ten times a second in a thread."""

    def __init__(self):
        self.samples: List[str] = []
        self._stop = threading.Event()
        self._th = threading.Thread(target=self._run)

    def _run(self):
        while not self._stop.is_set():
            try:
                self.samples.append(subprocess.run(["amd-smi", "metric", "-p", "-c"], capture_output=True, text=True, timeout=10).stdout)
            except Exception:      # no amd-smi, or no permission: reported as zero samples
                self.samples.append("")
            time.sleep(0.1)

    def __enter__(self):
        self._th.start()
        return self

    def __exit__(self, *exc):
        self._stop.set()
        self._th.join()

    def summary(self) -> Dict[str, object]:
        watts = [float(m.group(1)) for o in self.samples[1:] for m in [re.search(r"SOCKET_POWER:\s*([0-9.]+)", o)] if m]
        mhz = [float(m.group(1)) for o in self.samples[1:] for m in [re.search(r"GFX_0:\s*\n\s*CLK:\s*([0-9.]+)", o)] if m]
        stat = lambda v: {"n": len(v), "mean": round(sum(v) / len(v), 1), "max": max(v)} if v else {"n": 0}
        return {"socket_power_w": stat(watts), "gfx_clk_mhz": stat(mhz)}


def config2_operands(ones: bool = False, S: int = 4, seed: int = 0):
    """A_s[4096, 12288/S] ~ N(0,1), B_s[12288/S, 12288] ~ N(0,0.02), bf16 (all ones with ``ones``), and C[4096,12288]."""
    g = torch.Generator(device="cuda").manual_seed(seed)
    ks = 12288 // S
    if ones:
        A = [torch.ones((4096, ks), dtype=torch.bfloat16, device="cuda") for _ in range(S)]
        B = [torch.ones((ks, 12288), dtype=torch.bfloat16, device="cuda") for _ in range(S)]
    else:
        A = [torch.randn((4096, ks), generator=g, device="cuda").to(torch.bfloat16) for _ in range(S)]
        B = [(torch.randn((ks, 12288), generator=g, device="cuda") * 0.02).to(torch.bfloat16) for _ in range(S)]
    return A, B, torch.empty((4096, 12288), dtype=torch.bfloat16, device="cuda")


def resident_operands(resident: bool, seed: int = 1):
    """A 4096 x 12288 x 4096 product whose operands the L2s can keep (``resident``: 64 slices that are all the SAME
    [4096, 64] and [64, 12288] buffers, so every K step re-reads the panels of the first) or cannot (one slice with
    K = 4096): the same launches, tiles and FLOPs, with and without the traffic between the L2s and memory."""
    g = torch.Generator(device="cuda").manual_seed(seed)
    k = 64 if resident else 4096
    A = torch.randn((4096, k), generator=g, device="cuda").to(torch.bfloat16)
    B = (torch.randn((k, 12288), generator=g, device="cuda") * 0.02).to(torch.bfloat16)
    reps = 64 if resident else 1
    return [A] * reps, [B] * reps, torch.empty((4096, 12288), dtype=torch.bfloat16, device="cuda")


def os_parts_table(ones: bool = False, power_seconds: float = 0.0, rounds: int = 2, only: Optional[Sequence[int]] = None,
                   operands=None, flops: float = 2.0 * 4096 * 12288 * 12288) -> List[Dict[str, object]]:
    """The parts of ``PARTS`` on configuration 2 (or on ``operands = (A_slices, B_slices, C)`` of ``flops``), each timed
    ``rounds`` times in turn (the better time is kept): skip code, label, ms per launch, FLOP/s the product's algorithmic
    FLOPs would make at that time, and its share of the bf16 peak."""
    A, B, C = operands if operands is not None else config2_operands(ones)
    best: Dict[int, float] = {}
    parts = [p for p in PARTS if only is None or p[0] in only]
    for _ in range(rounds):
        for skip, _label in parts:
            t = os_parts_ms(skip, A, B, C)
            best[skip] = min(best.get(skip, t), t)
    rows = []
    for skip, label in parts:
        row: Dict[str, object] = {"skip": skip, "what": label, "ms": round(best[skip], 4), "tflops_equiv": round(flops / best[skip] / 1e9, 1),
                                  "frac_of_peak": round(flops / (best[skip] * 1e-3) / PEAK_BF16_FLOPS, 4)}
        if power_seconds > 0:
            os_parts_ms(skip, A, B, C, warmup=60, reps=1)
            with _PowerSampler() as ps:
                t0 = time.perf_counter()
                while time.perf_counter() - t0 < power_seconds:
                    os_parts_ms(skip, A, B, C, warmup=0, reps=200)
            row.update(ps.summary())
        rows.append(row)
    return rows


def main(argv=None) -> None:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--ones", action="store_true", help="all-ones operands for the kernel-parts probe (the device stays below its power limit)")
    ap.add_argument("--power", type=float, default=0.0, metavar="SECONDS", help="sample socket power and clock for SECONDS per kernel of the parts probe")
    ap.add_argument("--only", default=None, help="comma-separated skip codes of the parts probe to run (default: all)")
    ap.add_argument("--resident", action="store_true", help="also time a 4096 x 12288 x 4096 product on operands the L2s keep and on distinct ones")
    ap.add_argument("--no-streams", action="store_true", help="skip the L2 -> LDS and MFMA stream probes (profiler runs of the parts probe)")
    args = ap.parse_args(argv)
    torch.cuda.set_device(0)
    only = None if args.only is None else [int(v) for v in args.only.split(",")]
    out: Dict[str, object] = {"operands": "ones" if args.ones else "N(0,1) x N(0,0.02)",
                              "os_parts_config2": os_parts_table(args.ones, args.power, only=only)}
    if args.resident:
        fl = 2.0 * 4096 * 12288 * 4096
        for name, res in (("os_parts_l2_resident_operands", True), ("os_parts_same_product_distinct_operands", False)):
            out[name] = os_parts_table(False, args.power, only=only if only is not None else (0, SKIP_LOADS, SKIP_MFMA),
                                       operands=resident_operands(res), flops=fl)
    if not args.no_streams:
        out["l2_lds_stream"] = [l2_lds_stream_rate(in_flight_steps=f) for f in (1, 2, 3)] + [l2_lds_stream_rate(region_steps=1)]
        if args.power > 0:
            with _PowerSampler() as ps:
                t0 = time.perf_counter()
                while time.perf_counter() - t0 < args.power:
                    l2_lds_stream_rate(steps=4000, warmup=0, reps=50)
            out["l2_lds_stream_power"] = ps.summary()
            time.sleep(1.0)
            with _PowerSampler() as ps:
                time.sleep(args.power)
            out["idle_power"] = ps.summary()
        X = torch.randn(16 * 512, generator=torch.Generator(device="cpu").manual_seed(0)).to(torch.bfloat16).cuda()
        ops = torch.ones_like(X) if args.ones else X
        out["mfma_stream_tflops"] = {f"{shape}_{w}_wave_per_simd": round(mfma_stream_rate(ops, shape=shape, waves_per_simd=w) / 1e12, 1)
                                     for shape in ("32x32x16", "16x16x32") for w in (1, 2)}
        if args.power > 0:
            out["mfma_stream_power"] = {}
            for shape in ("32x32x16", "16x16x32"):
                with _PowerSampler() as ps:
                    t0 = time.perf_counter()
                    while time.perf_counter() - t0 < args.power:
                        mfma_stream_rate(ops, shape=shape, warmup=0, reps=200)
                out["mfma_stream_power"][shape] = ps.summary()
    print(json.dumps(out, indent=1), flush=True)


if __name__ == "__main__":
    main()
