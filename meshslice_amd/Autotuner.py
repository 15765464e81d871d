"""The parts of the reference's autotuner that consume the measured compute term.

* ``FFLayerModel`` with its dataflow rule and ``emulate`` (reference Autotuner.py:21-35, :141-169):
  forward + backward-data + backward-weight model time of one feed-forward layer for a slice count;
* ``possibleK`` (:242-273): admissible slice counts from the divisibility of the sliced extent;
* ``emulateFFTime`` (:391-426): per layer, scan the candidate slice counts and keep the best — as the method
  of ``class Autotuner(graph, shapes)`` like the reference's (same name, arguments and return value), and as
  a free function over a plain layer list;
* the interconnect constants the reference measured on TPUv4 (:17-19), kept as data;
* ``sweep_compute_term``: time the per-slice kernels of one GPT-3-like layer on the MI355X for
  several meshes and slice counts and refit ``CostModel.estimateMatmul``'s compute term.

The graph builder, transposition pass and analytical mesh search of the reference are host
bookkeeping with no device work and are not built.  Two slips of the reference are not reproduced:
``emulateFFTime`` records the loop variable of the scan as the best slice count (the reference
stores the module-level ``K``, :418), and an unknown dataflow name is an error.
"""
from __future__ import annotations

import math
from typing import Dict, Iterable, List, Sequence, Tuple

from . import CostModel
from .CostModel import DeviceMesh

# TPUv4 interconnect calibration shipped with the reference (Autotuner.py:17-19)
latencies = {"allgather": 5e-6, "reducescatter": 5e-6, "sendrecv": 5e-5}
bws = {"allgather": (27.472e9, 79.751e9), "reducescatter": (37.506e9, 63.167e9), "sendrecv": (38.801e9, 35.224e9)}
base_overheads = {"allgather": 13e-6, "reducescatter": 26e-6, "sendrecv": 13e-6}


def default_mesh(shape, flops: float = CostModel.BF16_PEAK_FLOPS) -> DeviceMesh:
    return DeviceMesh(shape, flops, bws_per_direction=bws, link_latencies=latencies, base_overheads=base_overheads)


def pick_dataflow(B: int, I: int, O: int) -> str:
    """Keep the largest of (tokens x in, tokens x out, in x out) stationary (reference :29-34, :297-302)."""
    if O > I and B >= I:
        return "os"
    if I >= O and B >= O:
        return "ls"
    return "rs"


class FFLayerModel:
    def __init__(self, B, I, O, dataflow=None, transpose=False):
        self.bsize, self.in_dim, self.out_dim = B, I, O
        if dataflow is None:
            dataflow = pick_dataflow(B, I, O)
        if dataflow not in ("os", "ls", "rs"):
            raise ValueError(f"unknown dataflow {dataflow!r}")
        self.dataflow = dataflow
        self.transpose = transpose

    def passes(self) -> List[Tuple[str, int, int, int]]:
        """(model, M, N, K) of the forward, backward-data and backward-weight GEMMs (reference :142-167)."""
        B, I, O = self.bsize, self.in_dim, self.out_dim
        plain = {
            "os": [("os", B, O, I), ("ls", B, I, O), ("rs", I, O, B)],
            "ls": [("ls", B, O, I), ("os", B, I, O), ("rs", O, I, B)],
            "rs": [("rs", B, O, I), ("ls", I, B, O), ("os", I, O, B)],
        }
        transposed = {
            "os": [("os", O, B, I), ("rs", I, B, O), ("ls", O, I, B)],
            "ls": [("rs", O, B, I), ("os", I, B, O), ("ls", I, O, B)],
            "rs": [("ls", O, B, I), ("rs", B, I, O), ("os", O, I, B)],
        }
        return (transposed if self.transpose else plain)[self.dataflow]

    def emulate(self, mesh: DeviceMesh, K: int) -> float:
        model = {"os": CostModel.MeshFlow_OS, "ls": CostModel.MeshFlow_LS, "rs": CostModel.MeshFlow_RS}
        total = 0.0
        for name, M, N, Kd in self.passes():
            pro, steady = model[name](mesh, M, N, Kd, K)
            total += pro + steady
        return total


def possibleK(B, I, O, meshshape, dataflow) -> List[int]:
    """Candidate slice counts (reference :242-273): the sliced extent, divided by lcm(R, C) and by the
    block size 8, picks a list by its divisibility."""
    mlcm = meshshape[0] * meshshape[1] // math.gcd(meshshape[0], meshshape[1])
    kdim = {"os": I, "ls": O}.get(dataflow, B) // mlcm // 8
    ladder = [(48, [3, 4, 6, 8, 12, 16, 24]), (40, [4, 5, 8, 10, 20]), (24, [3, 4, 6, 8, 12, 24]),
              (20, [4, 5, 10, 20]), (16, [4, 8, 16]), (12, [3, 4, 12]), (10, [5, 10]), (8, [4, 8]),
              (6, [3, 6]), (4, [4]), (5, [5])]
    for div, ks in ladder:
        if kdim % div == 0:
            return list(ks)
    return [kdim]


def emulateFFTime(layers: Sequence[Tuple[int, int, int, str]], meshshape, sweep: bool = False,
                  candidates=None, verbose: bool = False):
    """Model time of the feed-forward layers ``(B, I, O, dataflow)`` on ``meshshape`` with the best slice
    count per layer (reference :391-426).  Without ``sweep`` the scan stops at the first slice count
    that does not improve.  Returns ``(seconds, [best K per layer])``."""
    mesh = default_mesh(meshshape)
    total, best = 0.0, []
    for (B, I, O, dataflow) in layers:
        model = FFLayerModel(B, I, O, dataflow)
        klist = list(candidates) if candidates is not None else possibleK(B, I, O, meshshape, dataflow)
        bestK, bestT = klist[0], model.emulate(mesh, klist[0])
        for k in klist[1:]:
            t = model.emulate(mesh, k)
            if verbose:
                print(f"FFtime at k={k} is {t}")
            if t < bestT:
                bestK, bestT = k, t
            elif not sweep:
                break
        total += bestT
        best.append(bestK)
    return total, best


class LayerGraph:
    """The two attributes of the reference's ``ComputeGraph`` that its ``Autotuner`` reads (``nodenames`` and
    ``nodes``, reference :171-223), built from a list of feed-forward layers ``(name, B, I, O)``: each layer
    becomes an 'Input' node of shape [B, I] feeding a 'FeedForward' node of shape [B, O]."""

    def __init__(self, layers: Iterable[Tuple[str, int, int, int]]):
        self.nodenames: List[str] = []
        self.nodes: Dict[str, dict] = {}
        for (name, B, I, O) in layers:
            src = f"Input:{name}"
            for nm, op, inputs, shape in ((src, "Input", (), [B, I]), (name, "FeedForward", (src,), [B, O])):
                self.nodenames.append(nm)
                self.nodes[nm] = {"op_name": nm, "op_type": op, "inputs": inputs, "shape": shape}


class Autotuner:
    """The slice-count / mesh-shape search of the reference's ``Autotuner`` that runs on the measured compute
    term (reference Autotuner.py:278-483): ``emulateFFTime(meshshape, sweep)`` and ``emulatedFinetune(sweep)``.

    ``graph`` is anything with the reference ``ComputeGraph``'s ``nodenames`` / ``nodes`` (a ``LayerGraph``
    built from a layer list will do); ``shapes`` the candidate mesh shapes, all with the same device count.
    Per feed-forward node the dataflow follows the reference's rule (:291-302) and an 'rs' layer flips the
    transposition of what follows it (:303-313).  Not built: the analytical first guess (``analyticalAutotune``,
    host arithmetic on link constants) — the search starts from ``bestshape`` (default ``shapes[0]``) — and the
    insertion of 'Transpose' nodes where the two inputs of an 'Add' disagree (the 'Add' is taken as not
    transposed).  ``emulateFFTime`` records the loop variable as a layer's best slice count where the
    reference stores its module-level ``K`` (:418); ``emulatedFinetune(sweep=True)`` keeps the best shape where
    the reference assigns a misspelt attribute and returns nothing (:440)."""

    def __init__(self, graph, shapes, bestshape=None, verbose: bool = False):
        self.graph = graph
        self.shapes = list(shapes)
        self.layers = list(graph.nodenames)
        self.verbose = verbose
        self.dataflows: Dict[str, str] = {}
        self.transposition: Dict[str, bool] = {}
        self.ksplits: Dict[str, int] = {}
        for lname in self.layers:
            node = graph.nodes[lname]
            if node["op_type"] == "FeedForward":
                self.dataflows[lname] = pick_dataflow(*self._dims(lname))
        for lname in self.layers:
            node = graph.nodes[lname]
            if node["op_type"] == "Input":
                self.transposition[lname] = False
            elif node["op_type"] == "Add":
                a, b = (self.transposition[i] for i in node["inputs"][:2])
                self.transposition[lname] = a and b
            else:
                t = self.transposition[node["inputs"][0]]
                self.transposition[lname] = (not t) if self.dataflows.get(lname) == "rs" else t
        self.bestshape = tuple(bestshape) if bestshape is not None else tuple(self.shapes[0])
        if self.bestshape not in [tuple(s) for s in self.shapes]:
            raise ValueError(f"bestshape {self.bestshape} is not one of the candidate shapes")

    def _dims(self, lname) -> Tuple[int, int, int]:
        """(B, I, O) of feed-forward node ``lname``: B = product of the leading output dimensions, I = last
        dimension of its input, O = last dimension of its output (reference :292-297)."""
        node = self.graph.nodes[lname]
        B = 1
        for d in node["shape"][:-1]:
            B *= d
        return B, self.graph.nodes[node["inputs"][0]]["shape"][-1], node["shape"][-1]

    def _say(self, msg: str) -> None:
        if self.verbose:
            print(msg)

    def emulateFFTime(self, meshshape, sweep: bool = False):
        """Model seconds of all feed-forward nodes on ``meshshape`` with each node's best slice count, and those
        counts by node name (reference :391-426).  Without ``sweep`` a node's scan over ``possibleK`` stops at
        the first count that does not improve."""
        mesh = default_mesh(tuple(meshshape), flops=242 * 1024 ** 4)
        total, ksplits = 0.0, {}
        for lname in self.graph.nodenames:
            if self.graph.nodes[lname]["op_type"] != "FeedForward":
                continue
            B, I, O = self._dims(lname)
            model = FFLayerModel(B, I, O, self.dataflows[lname], self.transposition[lname])
            klist = possibleK(B, I, O, meshshape, self.dataflows[lname])
            bestK, bestT = klist[0], model.emulate(mesh, klist[0])
            self._say(f"{lname}: candidates {klist}; FFtime at k={bestK} is {bestT}")
            for k in klist[1:]:
                t = model.emulate(mesh, k)
                self._say(f"FFtime at k={k} is {t}")
                if t < bestT:
                    bestK, bestT = k, t
                elif not sweep:
                    break
            total += bestT
            ksplits[lname] = bestK
        self._say(f"FFtime: {total * 1000}ms")
        return total, ksplits

    def emulatedFinetune(self, sweep: bool = False):
        """Walk from ``bestshape`` to a neighbouring mesh shape while the model time drops (reference :427-483);
        with ``sweep`` try every shape.  Sets and returns ``(bestshape, ksplits)``."""
        times = {}

        def at(idx):
            if idx not in times:
                self._say(f"Trying shape of {self.shapes[idx]}")
                times[idx] = self.emulateFFTime(self.shapes[idx], sweep=sweep)
            return times[idx]

        shapes = [tuple(s) for s in self.shapes]
        cur = shapes.index(self.bestshape)
        if sweep:
            best = min(range(len(shapes)), key=lambda i: (at(i)[0], i != cur))
        else:
            def walk(idx, step):
                while 0 <= idx + step < len(shapes) and at(idx + step)[0] < at(idx)[0]:
                    idx += step
                return idx
            if cur > 0 and at(cur - 1)[0] < at(cur)[0]:          # the previous shape first, as the reference
                best = walk(cur - 1, -1)
            elif cur + 1 < len(shapes) and at(cur + 1)[0] < at(cur)[0]:
                best = walk(cur + 1, +1)
            else:
                best = cur
        self.bestshape, self.ksplits = shapes[best], at(best)[1]
        self._say(f"Best mesh shape is : {self.bestshape}")
        return self.bestshape, self.ksplits


# ------------------------------------------------------------------------------------------------
# compute-term sweep on the MI355X
# ------------------------------------------------------------------------------------------------

def gpt3_layers(tokens: int = 16384, hidden: int = 12288, ffn: int = 49152) -> List[Tuple[str, int, int, int, str]]:
    """(name, B, I, O, dataflow) of the four feed-forward GEMMs of one GPT-3-like layer, with the
    dataflows the reference's benchmark assigns (BenchTransformer.py:80-93)."""
    return [("in_proj", tokens, hidden, 3 * hidden, "os"), ("out_proj", tokens, hidden, hidden, "ls"),
            ("ff1", tokens, hidden, ffn, "os"), ("ff2", tokens, ffn, hidden, "ls")]


def per_slice_shapes(B, I, O, dataflow, meshshape, S, passes=("fwd", "bwd_data", "bwd_weight")):
    """Per-slice kernel shapes ``(pass, M, N, K, layout)`` a device runs, by the rules of
    CostModel.MeshFlow_OS/LS/RS: OS (M/R, N/C, K/S) nn; LS (M/R, N/S, K/C) nt; RS (M/S, N/C, K/R) tn."""
    R, C = meshshape
    out = []
    names = ("fwd", "bwd_data", "bwd_weight")
    for pname, (model, M, N, K) in zip(names, FFLayerModel(B, I, O, dataflow).passes()):
        if pname not in passes:
            continue
        if model == "os":
            out.append((pname, M // R, N // C, K // S, "nn"))
        elif model == "ls":
            out.append((pname, M // R, N // S, K // C, "nt"))
        else:
            out.append((pname, M // S, N // C, K // R, "tn"))
    return out


def sweep_compute_term(meshes=((2, 8), (4, 4), (8, 8)), slice_counts=(1, 2, 4, 8, 16),
                       passes=("fwd",), layers=None, repeat: int = 5, verbose: bool = True, fused: bool = False,
                       operands=None, vendor: bool = False):
    """Measure every per-slice kernel of the sweep on the GPU and fit the compute term.  ``operands`` ('normal' or
    'ones', default CostModel.DEFAULT_OPERANDS) says what the timing operands hold, see CostModel.estimateMatmul.

    Returns ``(ComputeTerm, rows)`` where each row is
    ``(mesh, layer, pass, S, M, N, K, layout, seconds_per_slice)``; with ``fused`` a tenth entry holds the
    seconds of the one fused S-slice call a device really issues, and with ``vendor`` (needs ``fused``) an eleventh the
    seconds of the vendor library's unsliced product of the same work (CostModel.measureVendorUnsliced)."""
    if vendor and not fused:
        raise ValueError("vendor=True compares with the fused call: pass fused=True too")
    layers = layers or gpt3_layers()
    rows, samples, seen, seen_fused, seen_vendor = [], [], {}, {}, {}
    for mesh in meshes:
        for (lname, B, I, O, dataflow) in layers:
            for S in slice_counts:
                for (pname, M, N, K, layout) in per_slice_shapes(B, I, O, dataflow, mesh, S, passes):
                    key = (M, N, K, layout)
                    if key not in seen:
                        seen[key] = CostModel.estimateMatmul(None, M, N, K, layout=layout, repeat=repeat, operands=operands)
                        samples.append((M, N, K, layout, seen[key]))
                    row = (mesh, lname, pname, S, M, N, K, layout, seen[key])
                    extra = ""
                    if fused:
                        fk = key + (S,)
                        if fk not in seen_fused:
                            seen_fused[fk] = CostModel.measureFused(M, N, K, S, layout=layout, repeat=repeat, operands=operands)
                        row = row + (seen_fused[fk],)
                        ftf = 2.0 * M * N * K * S / seen_fused[fk] / 1e12
                        extra = f" | S x slice {S*seen[key]*1e3:.4f} ms, fused {seen_fused[fk]*1e3:.4f} ms {ftf:.0f} TFLOP/s"
                        if vendor:
                            if fk not in seen_vendor:
                                seen_vendor[fk] = CostModel.measureVendorUnsliced(M, N, K, S, layout=layout, repeat=repeat, operands=operands)
                            row = row + (seen_vendor[fk],)
                            extra += f", vendor unsliced {seen_vendor[fk]*1e3:.4f} ms"
                    rows.append(row)
                    if verbose:
                        tf = 2.0 * M * N * K / seen[key] / 1e12
                        print(f"mesh {mesh[0]}x{mesh[1]} {lname:8s} {pname:10s} S={S:2d} {layout} "
                              f"[{M}x{N}x{K}] {seen[key]*1e3:.4f} ms/slice {tf:.0f} TFLOP/s{extra}", flush=True)
    return CostModel.fit_compute_term(samples), rows


def _main(argv=None):
    """``python -m meshslice_amd.Autotuner``: run the compute-term sweep on the GPU, print the table,
    the fitted ``(t0, eta)`` per layout and the model's slice-count choice with the measured term."""
    import argparse
    import json
    ap = argparse.ArgumentParser(description="refit the cost model's compute term from MI355X kernel times")
    ap.add_argument("--passes", default="fwd", help="comma list of fwd,bwd_data,bwd_weight")
    ap.add_argument("--slices", default="1,2,4,8,16")
    ap.add_argument("--meshes", default="2x8,4x4,8x8")
    ap.add_argument("--repeat", type=int, default=5)
    ap.add_argument("--fused", action="store_true", help="also time the fused S-slice call of every row")
    ap.add_argument("--operands", default=CostModel.DEFAULT_OPERANDS, choices=CostModel.OPERAND_KINDS,
                    help="timing operands: N(0, 0.02) samples, or all ones as in the reference")
    ap.add_argument("--vendor", action="store_true", help="with --fused: also time the vendor library's unsliced product of every row")
    ap.add_argument("--out", default=None, help="write the fitted term and the rows as JSON")
    a = ap.parse_args(argv)
    meshes = [tuple(int(v) for v in m.split("x")) for m in a.meshes.split(",")]
    slices = [int(v) for v in a.slices.split(",")]
    term, rows = sweep_compute_term(meshes, slices, tuple(a.passes.split(",")), repeat=a.repeat, fused=a.fused, operands=a.operands, vendor=a.vendor)
    for lay in sorted(term.eta):
        print(f"fit {lay}: t0 = {term.t0[lay]*1e6:.1f} us, eta = {term.eta[lay]:.3f} of {term.peak/1e12:.1f} TFLOP/s")
    CostModel.use_compute_term(term)
    try:
        layers = [(B, I, O, df) for (_n, B, I, O, df) in gpt3_layers()]
        for mesh in meshes:
            total, best = emulateFFTime(layers, mesh, sweep=True, candidates=[s for s in slices if s > 1])
            print(f"mesh {mesh[0]}x{mesh[1]}: model FF time {total*1e3:.3f} ms with slice counts {best} "
                  f"(TPUv4 link constants of the reference, MI355X compute term)")
    finally:
        CostModel.use_compute_term(None)
    if a.out:
        with open(a.out, "w") as f:
            what = "N(0, 0.02) samples" if a.operands == "normal" else "ones as in the reference's estimateMatmul"
            json.dump({"device": f"MI355X (gfx950), bf16, operands filled with {what}", "operands": a.operands,
                       "term": term.to_dict(),
                       "rows": [[f"{r[0][0]}x{r[0][1]}"] + list(r[1:]) for r in rows]}, f, indent=1)


if __name__ == "__main__":
    _main()
