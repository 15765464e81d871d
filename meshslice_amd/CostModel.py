"""Time model of the 2-D GEMM algorithms: analytical communication terms plus a MEASURED compute term.

Follows reference CostModel.py: ``DeviceMesh`` (:8-29), the ring all-gather / reduce-scatter
estimates (:47-63, :120-134), ``estimateMatmul`` (:74-98), the unsliced ``GSPMD_OS/LS/RS`` (:220-247)
and the sliced ``MeshFlow_OS/LS/RS`` (:249-285) models, each returning ``(prologue, steady_state)``
seconds.  The SUMMA / Cannon / logical-ring models of the reference are comparison baselines and are
not built.

The compute term is what this build changes: ``estimateMatmul`` times the gfx950 kernel of the same
layout on the MI355X (HIP events, warm-up + ``repeat`` launches, mean; operands N(0, 0.02) by default, all ones
as in the reference on request), or — when a fitted
``ComputeTerm`` has been installed with ``use_compute_term`` — evaluates ``t0 + 2MNK / (eta * peak)``
without touching the GPU.  There is no CPU timing path.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Iterable, Optional, Tuple

import numpy as np

BF16_PEAK_FLOPS = 2.5166e15   # MI355X dense bf16 MFMA peak: 256 CU x 2.4 GHz x 4096 FLOP/clk/CU


class DeviceMesh:
    """Mesh shape + link parameters (reference CostModel.py:8-29).  One of the two extents may itself
    be a pair ``(r, c)``: that mesh dimension is then a 2-D sub-mesh of r*c devices."""

    def __init__(self, device_shape: tuple, flops_per_chip: float, bws_per_direction, link_latencies, base_overheads):
        self.reshape(device_shape)
        self.flops = flops_per_chip
        self.bws = bws_per_direction
        self.link_latencies = link_latencies
        self.base_overheads = base_overheads

    def reshape(self, newshape):
        self.meshdim = None
        self.submesh = None
        dims = []
        for d, ext in enumerate(newshape):
            if isinstance(ext, tuple):
                self.meshdim, self.submesh = d, ext
                dims.append(ext[0] * ext[1])
            else:
                dims.append(ext)
        self.shape = tuple(dims)


def bytesize(shape) -> int:
    return shape[0] * shape[1] * 2


def _ring_collective(mesh: DeviceMesh, kind: str, data_shape, dim: int, precision: int) -> float:
    """Ring all-gather / reduce-scatter along mesh dimension ``dim``: ``size-1`` steps, each moving one
    shard and paying one link latency, plus a fixed launch overhead.  On a sub-meshed dimension the
    two halves of the data travel row-first and column-first at once (reference :55-62, :127-133)."""
    nbytes = data_shape[0] * data_shape[1] * precision // 8
    lat = mesh.link_latencies[kind]
    base = mesh.base_overheads[kind]
    bw = mesh.bws[kind][dim]
    if mesh.meshdim is not None and dim == mesh.meshdim:
        r, c = mesh.submesh
        half = nbytes // 2
        row_first = (half / bw) * (r - 1) + (half * r / bw) * (c - 1)
        col_first = (half / bw) * (c - 1) + (half * c / bw) * (r - 1)
        return base + max(row_first, col_first) + lat * (r + c - 2)
    steps = mesh.shape[dim] - 1
    return base + steps * (nbytes / bw) + lat * steps


def estimateAllgather(mesh: DeviceMesh, data_shape: tuple, dim: int, precision: int) -> float:
    return _ring_collective(mesh, "allgather", data_shape, dim, precision)


def estimateReduceScatter(mesh: DeviceMesh, data_shape: tuple, dim: int, precision: int) -> float:
    return _ring_collective(mesh, "reducescatter", data_shape, dim, precision)


# ------------------------------------------------------------------------------------------------
# compute term
# ------------------------------------------------------------------------------------------------

@dataclass
class ComputeTerm:
    """Fitted model of one kernel launch: ``t = t0 + 2*M*N*K / (eta * peak)`` per layout, with the
    measured points kept for exact look-up."""
    t0: Dict[str, float] = field(default_factory=dict)
    eta: Dict[str, float] = field(default_factory=dict)
    table: Dict[Tuple[int, int, int, str], float] = field(default_factory=dict)
    peak: float = BF16_PEAK_FLOPS

    def seconds(self, M: int, N: int, K: int, layout: str) -> float:
        hit = self.table.get((int(M), int(N), int(K), layout))
        if hit is not None:
            return hit
        if layout not in self.eta:
            raise KeyError(f"no fitted compute term for layout {layout!r}")
        return self.t0[layout] + 2.0 * M * N * K / (self.eta[layout] * self.peak)

    def to_dict(self):
        return {"peak": self.peak, "t0": self.t0, "eta": self.eta,
                "table": [[m, n, k, lay, t] for (m, n, k, lay), t in sorted(self.table.items())]}

    @classmethod
    def from_dict(cls, d):
        ct = cls(t0=dict(d["t0"]), eta=dict(d["eta"]), peak=float(d.get("peak", BF16_PEAK_FLOPS)))
        for m, n, k, lay, t in d.get("table", []):
            ct.table[(int(m), int(n), int(k), lay)] = float(t)
        return ct


def fit_compute_term(samples: Iterable[Tuple[int, int, int, str, float]], peak: float = BF16_PEAK_FLOPS) -> ComputeTerm:
    """Least-squares fit of ``t = t0 + flops / (eta*peak)`` per layout from measured
    ``(M, N, K, layout, seconds)`` samples."""
    ct = ComputeTerm(peak=peak)
    by_layout: Dict[str, list] = {}
    for m, n, k, lay, t in samples:
        ct.table[(int(m), int(n), int(k), lay)] = float(t)
        by_layout.setdefault(lay, []).append((2.0 * m * n * k, float(t)))
    for lay, pts in by_layout.items():
        f = np.array([p[0] for p in pts]); t = np.array([p[1] for p in pts])
        if len(pts) >= 2 and np.ptp(f) > 0:
            slope, icpt = np.polyfit(f, t, 1)
        else:
            slope, icpt = t[0] / f[0], 0.0
        if slope <= 0:   # degenerate sample set: fall back to the mean rate
            slope, icpt = float(np.sum(t) / np.sum(f)), 0.0
        ct.t0[lay] = float(max(icpt, 0.0))
        ct.eta[lay] = float(1.0 / (slope * peak))
    return ct


_installed: Optional[ComputeTerm] = None
_measured: Dict[tuple, float] = {}


def use_compute_term(term: Optional[ComputeTerm]) -> None:
    """Install (or, with None, remove) a fitted compute term used by ``estimateMatmul``."""
    global _installed
    _installed = term


OPERAND_KINDS = ("normal", "ones")
# What the timing operands hold when a call does not say: N(0, 0.02) values rounded to bf16.  The reference times
# its matmul on all-ones operands (CostModel.py:78-79); on this power-limited device constant operands run
# 20-25 % faster than real tensors, which would bias the compute term low against every communication term.
DEFAULT_OPERANDS = "normal"
# untimed launches before the timed ones: one for 'ones' (the reference's protocol, :90); for 'normal' enough to
# pass the start-up transient of the package power controller, during which launches run up to 30 % slow
_WARMUP = {"ones": 1, "normal": 10}


def _term_path(operands: str) -> str:
    import os
    name = "compute_term_mi355x.json" if operands == "normal" else "compute_term_mi355x_ones.json"
    return os.path.join(os.path.dirname(os.path.abspath(__file__)), "data", name)


def load_compute_term(path: Optional[str] = None, operands: Optional[str] = None) -> ComputeTerm:
    """Install a compute term measured on MI355X that ships with the package and return it: by default the
    one fitted on N(0, 0.02) operands, with ``operands='ones'`` the one fitted on the reference's all-ones
    timing operands.  ``path`` names another JSON as written by ``python -m meshslice_amd.Autotuner --out``."""
    import json
    if path is None:
        path = _term_path(_operand_kind(operands))
    with open(path) as f:
        d = json.load(f)
    term = ComputeTerm.from_dict(d["term"] if "term" in d else d)
    use_compute_term(term)
    return term


def _operand_kind(operands: Optional[str]) -> str:
    kind = DEFAULT_OPERANDS if operands is None else operands
    if kind not in OPERAND_KINDS:
        raise ValueError(f"unknown operand kind {kind!r} (one of {OPERAND_KINDS})")
    return kind


def _timing_operand(shape, dtype, kind: str, seed: int):
    """A [rows, cols] GPU tensor of ones, or of seeded N(0, 0.02) samples rounded to ``dtype``."""
    import torch
    if kind == "ones":
        return torch.ones(shape, dtype=dtype, device="cuda")
    g = torch.Generator(device="cuda").manual_seed(seed)
    return (torch.randn(shape, generator=g, device="cuda") * 0.02).to(dtype)


def _time_layout(M, N, K, S, layout, dtype, kind, repeat):
    """Mean seconds per launch of the fused S-slice call of ``layout`` on per-slice shape [M,K] x [K,N]."""
    import torch
    from . import local_gemm
    mk = lambda shape, i: _timing_operand(shape, dtype, kind, 1 + i)
    warm = _WARMUP[kind]
    if layout == "nn":
        A = [mk((M, K), 2 * s) for s in range(S)]; B = [mk((K, N), 2 * s + 1) for s in range(S)]
        ms = local_gemm.time_call("os", (A, B), torch.empty((M, N), dtype=dtype, device="cuda"), warmup=warm, reps=repeat)
    elif layout == "nt":
        out = [torch.empty((M, N), dtype=torch.float32, device="cuda") for _ in range(S)]
        ms = local_gemm.time_call("ls", (mk((M, K), 0), [mk((N, K), 1 + s) for s in range(S)]), out, warmup=warm, reps=repeat)
    else:
        out = [torch.empty((M, N), dtype=torch.float32, device="cuda") for _ in range(S)]
        ms = local_gemm.time_call("rs", ([mk((K, M), 1 + s) for s in range(S)], mk((K, N), 0)), out, warmup=warm, reps=repeat)
    return float(np.mean(ms)) * 1e-3


def measureVendorUnsliced(M, N, K, S, layout: str = "nn", input_precision=None, repeat: int = 5,
                          operands: Optional[str] = None) -> float:
    """Seconds of the vendor library's ONE unsliced product that does the work of the fused S-slice call
    (``torch.matmul``, i.e. hipBLASLt / rocBLAS, on contiguous operands in the layout's own storage; bf16 in and out):
    'nn' [M, S K] x [S K, N], 'nt' [M, K] x [S N, K]^T, 'tn' [K, S M]^T x [K, N].  A yardstick for the sweep's tables,
    not a dependency: nothing else in the package calls the library.  Timed like ``measureFused`` (same operand kinds,
    warm-up counts and HIP events around each launch)."""
    import torch
    from . import local_gemm
    if layout not in ("nn", "nt", "tn"):
        raise ValueError(f"unknown layout {layout!r}")
    kind = _operand_kind(operands)
    if not torch.cuda.is_available():
        raise local_gemm._lib.MeshSliceError("measureVendorUnsliced needs the GPU")
    dtype = input_precision or torch.bfloat16
    M, N, K, S = int(M), int(N), int(K), int(S)
    mk = lambda shape, i: _timing_operand(shape, dtype, kind, 1 + i)
    if layout == "nn":
        a, b = mk((M, S * K), 0), mk((S * K, N), 1)
        run = lambda out: torch.matmul(a, b, out=out)
        out = torch.empty((M, N), dtype=dtype, device="cuda")
    elif layout == "nt":
        a, b = mk((M, K), 0), mk((S * N, K), 1)
        run = lambda out: torch.matmul(a, b.t(), out=out)
        out = torch.empty((M, S * N), dtype=dtype, device="cuda")
    else:
        a, b = mk((K, S * M), 0), mk((K, N), 1)
        run = lambda out: torch.matmul(a.t(), b, out=out)
        out = torch.empty((S * M, N), dtype=dtype, device="cuda")
    for _ in range(_WARMUP[kind]):
        run(out)
    times = []
    for _ in range(int(repeat)):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        run(out)
        e1.record()
        e1.synchronize()
        times.append(e0.elapsed_time(e1))
    return float(np.mean(times)) * 1e-3


def estimateMatmul(mesh, M, N, K, input_precision=None, layout: str = "nn", repeat: int = 5,
                   operands: Optional[str] = None) -> float:
    """Seconds of one local ``[M,K] x [K,N]`` contraction (reference CostModel.py:74-98).

    ``layout``: 'nn' (OS slice), 'nt' (LS: B stored [N,K]), 'tn' (RS: A stored [K,M]).  ``mesh`` is
    unused, as in the reference.  Measures on the GPU unless a fitted term is installed: ``operands='ones'``
    is the reference's protocol (all-ones operands, one warm-up launch), ``'normal'`` (the default, see
    DEFAULT_OPERANDS) times N(0, 0.02) operands after ten warm-up launches."""
    if layout not in ("nn", "nt", "tn"):
        raise ValueError(f"unknown layout {layout!r}")
    kind = _operand_kind(operands)
    M, N, K = int(M), int(N), int(K)
    if _installed is not None:
        return _installed.seconds(M, N, K, layout)
    import torch
    from . import local_gemm
    dtype = input_precision or torch.bfloat16
    key = (M, N, K, layout, dtype, repeat, kind)
    if key in _measured:
        return _measured[key]
    if not torch.cuda.is_available():
        raise local_gemm._lib.MeshSliceError(
            "estimateMatmul needs the GPU (or a fitted ComputeTerm installed with use_compute_term)")
    sec = _time_layout(M, N, K, 1, layout, dtype, kind, repeat)
    _measured[key] = sec
    return sec


def measureFused(M, N, K, S, layout: str = "nn", input_precision=None, repeat: int = 5,
                 operands: Optional[str] = None) -> float:
    """Seconds of ONE fused call that does the work of ``S`` per-slice contractions of shape
    ``[M,K] x [K,N]`` (the per-slice shape ``estimateMatmul`` is asked about): 'nn' = ms_gemm_os over S
    k-slices, 'nt' = ms_gemm_ls emitting S chunks, 'tn' = ms_gemm_rs emitting S chunks.  GPU only;
    ``operands`` as in ``estimateMatmul``."""
    import torch
    from . import local_gemm
    if layout not in ("nn", "nt", "tn"):
        raise ValueError(f"unknown layout {layout!r}")
    kind = _operand_kind(operands)
    if not torch.cuda.is_available():
        raise local_gemm._lib.MeshSliceError("measureFused needs the GPU")
    return _time_layout(int(M), int(N), int(K), int(S), layout, input_precision or torch.bfloat16, kind, repeat)


# ------------------------------------------------------------------------------------------------
# algorithm models: (prologue, steady state)
# ------------------------------------------------------------------------------------------------

def GSPMD_OS(mesh, M, N, K, steps=8, precisions=(16, 16, 16)):
    """Unsliced output-stationary (reference :220-227)."""
    R, C = mesh.shape
    ag_i = estimateAllgather(mesh, (M // R, K // C), 1, precisions[0])
    ag_w = estimateAllgather(mesh, (K // R, N // C), 0, precisions[1])
    compute = estimateMatmul(mesh, M // R, N // C, K)
    return (ag_i, max(compute, ag_w))


def GSPMD_LS(mesh, M, N, K, steps=8, precisions=(16, 16, 16)):
    """Unsliced LHS-stationary (reference :229-237)."""
    R, C = mesh.shape
    ag_w = estimateAllgather(mesh, (N // R, K // C), 0, precisions[1])
    compute = estimateMatmul(mesh, M // R, N, K // C, layout="nt")
    rs_o = estimateReduceScatter(mesh, (M // R, N // C), 1, precisions[2])
    return (rs_o, max(ag_w, compute))


def GSPMD_RS(mesh, M, N, K, steps=8, precisions=(16, 16, 16)):
    """Unsliced RHS-stationary (reference :239-247)."""
    R, C = mesh.shape
    ag_i = estimateAllgather(mesh, (K // R, M // C), 1, precisions[0])
    compute = estimateMatmul(mesh, M, N // C, K // R, layout="tn")
    rs_o = estimateReduceScatter(mesh, (M // R, N // C), 0, precisions[2])
    return (rs_o, max(ag_i, compute))


def MeshFlow_OS(mesh, M, N, K, steps=32, precisions=(16, 16, 16)):
    """Sliced output-stationary: per slice, gather both operands' slices while the previous slice
    multiplies (reference :249-258)."""
    R, C = mesh.shape
    ag_i = estimateAllgather(mesh, (M // R, K // C // steps), 1, precisions[0])
    ag_w = estimateAllgather(mesh, (K // R // steps, N // C), 0, precisions[1])
    compute = estimateMatmul(mesh, M // R, N // C, K // steps)
    return (max(ag_i, ag_w), max(ag_i, ag_w, compute) * (steps - 1) + compute)


def MeshFlow_LS(mesh, M, N, K, steps=32, precisions=(16, 16, 16)):
    """Sliced LHS-stationary: gather a weight slice, multiply, reduce-scatter the chunk (reference :260-272)."""
    R, C = mesh.shape
    ag_w = estimateAllgather(mesh, (N // R // steps, K // C), 0, precisions[1])
    rs_o = estimateReduceScatter(mesh, (M // R, N // C // steps), 1, precisions[2])
    compute = estimateMatmul(mesh, M // R, N // steps, K // C, layout="nt")
    return (ag_w + rs_o, compute + max(ag_w, rs_o, compute) * (steps - 1))


def MeshFlow_RS(mesh, M, N, K, steps=32, precisions=(16, 16, 16)):
    """Sliced RHS-stationary (reference :273-285)."""
    R, C = mesh.shape
    ag_i = estimateAllgather(mesh, (K // R, M // C // steps), 1, precisions[0])
    rs_o = estimateReduceScatter(mesh, (M // R // steps, N // C), 0, precisions[2])
    compute = estimateMatmul(mesh, M // steps, N // C, K // R, layout="tn")
    return (ag_i + rs_o, compute + max(ag_i, rs_o, compute) * (steps - 1))


def tup2ms(t):
    return (str(t[0] * 1000) + "ms", str(t[1] * 1000) + "ms", str((t[0] + t[1]) * 1000) + "ms")
