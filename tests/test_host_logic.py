"""Host-side logic that needs no GPU: the C ABI loads and exports what the header declares, the mesh
plumbing of TensorParallel.py agrees with the oracle's closed forms, the cost model's formulas match
hand-computed values, and the golden fixtures agree with the oracle."""
import json
import os
import re

import numpy as np
import pytest
import torch

from oracle import meshslice_oracle as orc
import meshslice_amd
from meshslice_amd import _lib, CostModel, Autotuner
from meshslice_amd import TensorParallel as TP
from meshslice_amd.mesh import Mesh, create_device_mesh

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ---------------------------------------------------------------- C ABI
def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "meshslice_hip.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(ms_[a-z_0-9]+)\s*\(", header))
    assert {"ms_gemm_os", "ms_gemm_ls", "ms_gemm_rs", "ms_version", "ms_last_error", "ms_query"} <= declared
    lib = _lib.load()
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
    assert set(_lib.EXPORTS) == declared
    assert lib.ms_version() >= 100
    assert lib.ms_query(_lib.MS_QUERY_MAX_SLICES) == 64


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libmeshslice_hip.so")
    with pytest.raises(_lib.MeshSliceError, match="no CPU fallback"):
        _lib.load()


def test_cpu_tensors_are_rejected_not_computed():
    a = torch.zeros(8, 8); b = torch.zeros(8, 8)
    with pytest.raises(_lib.MeshSliceError):
        meshslice_amd.gemm_os([a], [b])
    mesh = Mesh(create_device_mesh((2, 2)), ("row", "col"))
    with pytest.raises(_lib.MeshSliceError):
        TP.SPMD(mesh, "collective").OS()(torch.zeros(16, 16), torch.zeros(16, 16))


# ---------------------------------------------------------------- mesh plumbing has no CPU path either
def test_slicing_gathering_and_chunk_assembly_reject_cpu_tensors():
    """The block-cyclic slicing, the gather placement and the reduce + interleave of the chunks run in HIP
    kernels; on CPU tensors they raise instead of computing (their parity tests are GPU tests)."""
    G = torch.arange(24 * 64, dtype=torch.float32).reshape(24, 64)
    Xs = TP._shards(G, 4, 2)
    assert Xs[1][1].shape == (6, 32) and Xs[1][1].data_ptr() == G[6:12, 32:].data_ptr()      # views, no copies
    with pytest.raises(_lib.MeshSliceError):
        TP._gather_col_slices([Xs[1][0], Xs[1][1]], 2, 8)
    with pytest.raises(_lib.MeshSliceError):
        TP._gather_row_slices([G[:16], G[:16]], 2, 8)
    with pytest.raises(_lib.MeshSliceError):
        TP._finish([[G, G], [G, G]], 0, 1, 8, torch.float32)
    with pytest.raises(ValueError):
        TP._gather_col_slices([Xs[1][0]], 3, 8)          # 32 columns are not a multiple of 3 * 8


def test_spmd_surface_and_shape_errors():
    mesh = Mesh(create_device_mesh((4, 2)), ("row", "col"))
    assert mesh.axis_names == ("row", "col") and mesh.devices.shape == (4, 2)
    s = TP.SPMD(mesh, "meshflow")
    assert s.blocksize == 8 and s.rowaxis == "row" and s.colaxis == "col"
    for name in ("systolic", "noff", "meshflow"):      # any other name selects the sliced bodies
        assert TP.SPMD(mesh, name).funcs["os"] is TP.MeshFlow_OS
    assert TP.SPMD(mesh, "collective").funcs["ls"] is TP.Collective_LS
    assert TP.SPMD(mesh, "wang").funcs["rs"] is TP.Wang_RS
    with pytest.raises(AssertionError):                 # the reference asserts a square mesh (TensorParallel.py:359)
        TP.SPMD(mesh, "cannon")
    sq = Mesh(create_device_mesh((2, 2)), ("row", "col"))
    assert TP.SPMD(sq, "cannon").funcs["os"] is TP.Cannon_OS and not TP.SPMD(sq, "cannon").sliced
    f = s.OS()                                          # default K = 8
    assert f.K == 8
    with pytest.raises(ValueError):                     # 256/2 = 128 per shard, needs multiple of 8*8
        f(torch.zeros(512, 96), torch.zeros(96, 1024))
    with pytest.raises(ValueError):
        s.LS(0)
    with pytest.raises(ValueError):
        f.device(4, 0)
    with pytest.raises(ValueError, match="K == 1"):
        TP.MeshFlow_OS(None, None, 0, 0, 4, 2, 1, 8)


@pytest.mark.parametrize("algorithm,R,C", [("wang", 2, 4), ("wang", 4, 2), ("wang", 1, 3), ("cannon", 2, 2), ("cannon", 4, 4), ("cannon", 3, 3)])
def test_ring_order_of_the_device_bodies_matches_the_oracle(algorithm, R, C):
    for dataflow in ("os", "ls", "rs"):
        for i in range(R):
            for j in range(C):
                order = TP._ring_order(algorithm, dataflow, R, C, i, j)
                assert order == orc.ring_order(algorithm, dataflow, R, C, i, j)
                assert sorted(order) == [(b, h) for b in range(C) for h in (0, 1)]      # every half-block exactly once


# ---------------------------------------------------------------- cost model
def _mesh(shape):
    return Autotuner.default_mesh(shape)


def test_ring_collective_estimates_by_hand():
    m = _mesh((4, 4))
    # all-gather of a [1024, 96] bf16 shard along dim 1: 3 steps of 196608 B at 79.751 GB/s + 3*5us + 13us
    want = 13e-6 + 3 * (1024 * 96 * 2 / 79.751e9) + 3 * 5e-6
    assert CostModel.estimateAllgather(m, (1024, 96), 1, 16) == pytest.approx(want, rel=1e-12)
    want = 26e-6 + 3 * (512 * 64 * 2 / 37.506e9) + 3 * 5e-6
    assert CostModel.estimateReduceScatter(m, (512, 64), 0, 16) == pytest.approx(want, rel=1e-12)
    sub = _mesh(((2, 2), 4))
    assert sub.shape == (4, 4) and sub.meshdim == 0 and sub.submesh == (2, 2)
    half = (512 * 64 * 2) // 2
    bw = 27.472e9
    want = 13e-6 + max(half / bw + half * 2 / bw, half / bw + half * 2 / bw) + 5e-6 * 2
    assert CostModel.estimateAllgather(sub, (512, 64), 0, 16) == pytest.approx(want, rel=1e-12)


def test_meshflow_models_use_per_slice_shapes_and_compose_by_hand():
    calls = []
    term = CostModel.ComputeTerm()

    class Spy(CostModel.ComputeTerm):
        def seconds(self, M, N, K, layout):
            calls.append((M, N, K, layout))
            return 1e-4
    CostModel.use_compute_term(Spy())
    try:
        m = _mesh((4, 4))
        M, N, K, S = 16384, 49152, 12288, 4
        pro, steady = CostModel.MeshFlow_OS(m, M, N, K, S)
        assert calls[-1] == (4096, 12288, 3072, "nn")
        ag_i = CostModel.estimateAllgather(m, (4096, 768), 1, 16)
        ag_w = CostModel.estimateAllgather(m, (768, 12288), 0, 16)
        assert pro == pytest.approx(max(ag_i, ag_w))
        assert steady == pytest.approx(max(ag_i, ag_w, 1e-4) * 3 + 1e-4)
        pro, steady = CostModel.MeshFlow_LS(m, 16384, 12288, 49152, 8)
        assert calls[-1] == (4096, 1536, 12288, "nt")
        ag = CostModel.estimateAllgather(m, (384, 12288), 0, 16)
        rs = CostModel.estimateReduceScatter(m, (4096, 384), 1, 16)
        assert pro == pytest.approx(ag + rs) and steady == pytest.approx(1e-4 + max(ag, rs, 1e-4) * 7)
        pro, steady = CostModel.MeshFlow_RS(m, 12288, 49152, 16384, 4)
        assert calls[-1] == (3072, 12288, 4096, "tn")
        CostModel.GSPMD_OS(m, M, N, K)
        assert calls[-1] == (4096, 12288, 12288, "nn")
        CostModel.GSPMD_LS(m, 16384, 12288, 49152)
        assert calls[-1] == (4096, 12288, 12288, "nt")
        CostModel.GSPMD_RS(m, 12288, 49152, 16384)
        assert calls[-1] == (12288, 12288, 4096, "tn")
    finally:
        CostModel.use_compute_term(None)
    assert term.table == {}


def test_compute_term_fit_recovers_a_planted_model():
    peak = CostModel.BF16_PEAK_FLOPS
    t0, eta = 7e-6, 0.6
    shapes = [(4096, 12288, 768), (4096, 12288, 3072), (2048, 6144, 1536), (8192, 6144, 12288)]
    samples = [(m, n, k, "nn", t0 + 2.0 * m * n * k / (eta * peak)) for m, n, k in shapes]
    ct = CostModel.fit_compute_term(samples)
    assert ct.t0["nn"] == pytest.approx(t0, rel=1e-6) and ct.eta["nn"] == pytest.approx(eta, rel=1e-6)
    assert ct.seconds(4096, 12288, 768, "nn") == samples[0][4]           # table hit
    assert ct.seconds(1024, 1024, 1024, "nn") == pytest.approx(t0 + 2.0 * 1024**3 / (eta * peak))
    back = CostModel.ComputeTerm.from_dict(json.loads(json.dumps(ct.to_dict())))
    assert back.seconds(4096, 12288, 3072, "nn") == samples[1][4]
    with pytest.raises(KeyError):
        ct.seconds(8, 8, 8, "tn")


def test_estimate_matmul_without_gpu_or_term_raises():
    CostModel.use_compute_term(None)
    if torch.cuda.is_available():
        pytest.skip("GPU present")
    with pytest.raises(_lib.MeshSliceError):
        CostModel.estimateMatmul(None, 256, 256, 256)
    with pytest.raises(ValueError):
        CostModel.estimateMatmul(None, 8, 8, 8, layout="tt")


def test_possible_k_and_layer_passes():
    # reference Autotuner.py:242-273 on the GPT-3 layer: 12288 / lcm(4,4) / 8 = 384 = 48*8
    assert Autotuner.possibleK(16384, 12288, 49152, (4, 4), "os") == [3, 4, 6, 8, 12, 16, 24]
    assert Autotuner.possibleK(16384, 12288, 49152, (8, 8), "os") == [3, 4, 6, 8, 12, 16, 24]  # 192
    assert Autotuner.possibleK(16384, 49152, 12288, (2, 8), "ls") == [3, 4, 6, 8, 12, 16, 24]
    assert Autotuner.possibleK(4096, 1280, 5120, (4, 4), "os") == [4, 5, 8, 10, 20]            # 40
    assert Autotuner.possibleK(7 * 2 * 8, 8, 8, (2, 2), "rs") == [7]                                 # fallback
    assert Autotuner.pick_dataflow(16384, 12288, 49152) == "os"
    assert Autotuner.pick_dataflow(16384, 49152, 12288) == "ls"
    assert Autotuner.pick_dataflow(64, 4096, 4096) == "rs"
    f = Autotuner.FFLayerModel(16384, 12288, 49152, "os")
    assert f.passes() == [("os", 16384, 49152, 12288), ("ls", 16384, 12288, 49152), ("rs", 12288, 49152, 16384)]
    shapes = Autotuner.per_slice_shapes(16384, 12288, 49152, "os", (4, 4), 4)
    assert shapes == [("fwd", 4096, 12288, 3072, "nn"), ("bwd_data", 4096, 3072, 12288, "nt"),
                      ("bwd_weight", 3072, 12288, 4096, "tn")]
    ls = Autotuner.per_slice_shapes(16384, 49152, 12288, "ls", (4, 4), 8, passes=("fwd",))
    assert ls == [("fwd", 4096, 1536, 12288, "nt")]


def test_emulate_ff_time_scans_slice_counts():
    class Flat(CostModel.ComputeTerm):
        def seconds(self, M, N, K, layout):
            return 2.0 * M * N * K / 1.5e15 + 5e-6      # fixed launch cost favours fewer slices
    CostModel.use_compute_term(Flat())
    try:
        layers = [(16384, 12288, 49152, "os"), (16384, 49152, 12288, "ls")]
        total, best = Autotuner.emulateFFTime(layers, (4, 4), sweep=True)
        by_hand = []
        for (B, I, O, df) in layers:
            model = Autotuner.FFLayerModel(B, I, O, df)
            times = {k: model.emulate(Autotuner.default_mesh((4, 4)), k) for k in Autotuner.possibleK(B, I, O, (4, 4), df)}
            by_hand.append(min(times, key=times.get))
            assert times[by_hand[-1]] <= min(times.values())
        assert best == by_hand
        t2, b2 = Autotuner.emulateFFTime(layers, (4, 4), sweep=False)
        assert t2 >= total
    finally:
        CostModel.use_compute_term(None)


# ---------------------------------------------------------------- golden fixtures vs oracle
def test_golden_notebook_blocks_match_oracle():
    g = json.load(open(os.path.join(ROOT, "tests", "golden", "notebook_blocks.json")))
    d = orc.notebook_inputs(np.float64)
    R, C = g["mesh"]
    full = {"os": orc.dense("os", d["X"], d["W"]), "ls": orc.dense("ls", d["dY"], d["W"]),
            "rs": orc.dense("rs", d["X"], d["dY"])}
    for flow, Y in full.items():
        for key, st in g[flow].items():
            i, j = map(int, key.split(","))
            blk = orc.shard(Y, R, C, i, j)
            assert blk.sum() == pytest.approx(st["sum"], rel=1e-13)
            assert (blk * blk).sum() == pytest.approx(st["sumsq"], rel=1e-13)
            assert [blk[0, 0], blk[0, -1], blk[-1, 0], blk[-1, -1]] == st["corners"]


def test_shipped_compute_term_loads_and_feeds_the_models():
    term = CostModel.load_compute_term()
    try:
        assert set(term.eta) == {"nn", "nt", "tn"}
        assert all(0.2 < e < 1.0 for e in term.eta.values())
        # a measured point of the sweep: ff1 forward slice on the 4x4 mesh at S=4
        t = CostModel.estimateMatmul(None, 4096, 12288, 3072, layout="nn")
        assert 0.1e-3 < t < 0.5e-3
        pro, steady = CostModel.MeshFlow_OS(_mesh((4, 4)), 16384, 49152, 12288, 4)
        assert steady >= 4 * t
    finally:
        CostModel.use_compute_term(None)


def test_autotuner_class_mirrors_the_reference_surface():
    """``Autotuner(graph, shapes).emulateFFTime(meshshape, sweep)`` -> (seconds, {node name: slice count}), the
    dataflow rule and the transposition flip of 'rs' layers (reference Autotuner.py:278-313, :391-426)."""
    class Flat(CostModel.ComputeTerm):
        def seconds(self, M, N, K, layout):
            return 2.0 * M * N * K / 1.5e15 + 5e-6
    layers = [("in_proj", 16384, 12288, 36864), ("out_proj", 16384, 12288, 12288),
              ("ff1", 16384, 12288, 49152), ("ff2", 16384, 49152, 12288)]
    graph = Autotuner.LayerGraph(layers)
    assert graph.nodenames[:2] == ["Input:in_proj", "in_proj"] and graph.nodes["ff1"]["op_type"] == "FeedForward"
    shapes = [(2, 8), (4, 4), (8, 2)]
    CostModel.use_compute_term(Flat())
    try:
        tuner = Autotuner.Autotuner(graph, shapes, bestshape=(4, 4))
        assert tuner.dataflows == {"in_proj": "os", "out_proj": "ls", "ff1": "os", "ff2": "ls"}
        assert not any(tuner.transposition.values())
        total, ks = tuner.emulateFFTime((4, 4), sweep=True)
        flat_total, flat_best = Autotuner.emulateFFTime([(B, I, O, tuner.dataflows[n]) for n, B, I, O in layers], (4, 4), sweep=True)
        assert list(ks) == [n for n, *_ in layers] and list(ks.values()) == flat_best
        # the class prices the mesh with the reference's 242 * 1024**4 FLOP/s figure, the free function with the MI355X peak;
        # neither enters the model times, which come from the installed compute term
        assert total == pytest.approx(flat_total, rel=1e-12)
        # neighbour search: ends on a shape that none of its neighbours beats, and sweep finds the global best
        best, ksplits = tuner.emulatedFinetune()
        times = {s: tuner.emulateFFTime(s)[0] for s in shapes}
        i = shapes.index(best)
        assert all(times[best] <= times[shapes[j]] for j in (i - 1, i + 1) if 0 <= j < len(shapes))
        assert ksplits == tuner.emulateFFTime(best)[1]
        tuner2 = Autotuner.Autotuner(graph, shapes)
        assert tuner2.bestshape == (2, 8)
        best2, _ = tuner2.emulatedFinetune(sweep=True)
        swept = {s: tuner2.emulateFFTime(s, sweep=True)[0] for s in shapes}
        assert swept[best2] == min(swept.values())
    finally:
        CostModel.use_compute_term(None)
    # an 'rs' layer (weight largest) flips the transposition of what follows it
    chain = Autotuner.LayerGraph([("small", 64, 4096, 4096)])
    chain.nodenames.append("next")
    chain.nodes["next"] = {"op_name": "next", "op_type": "Gelu", "inputs": ("small",), "shape": [64, 4096]}
    t = Autotuner.Autotuner(chain, [(2, 2)])
    assert t.dataflows["small"] == "rs" and t.transposition == {"Input:small": False, "small": True, "next": True}
    with pytest.raises(ValueError):
        Autotuner.Autotuner(graph, shapes, bestshape=(3, 3))


def test_both_shipped_compute_terms_load_and_the_ones_term_is_the_faster():
    """The default term is fitted on N(0, 0.02) operands; the reference's all-ones protocol stays selectable and, on
    this power-limited device, reads faster for every layout."""
    try:
        normal = CostModel.load_compute_term()
        ones = CostModel.load_compute_term(operands="ones")
        assert set(normal.eta) == set(ones.eta) == {"nn", "nt", "tn"}
        for lay in normal.eta:
            assert 0.2 < normal.eta[lay] < ones.eta[lay] < 1.0
        with pytest.raises(ValueError):
            CostModel.load_compute_term(operands="zeros")
        with pytest.raises(ValueError):
            CostModel.estimateMatmul(None, 8, 8, 8, operands="zeros")
    finally:
        CostModel.use_compute_term(None)


def test_both_shipped_compute_terms_lead_to_the_same_slice_counts():
    """The reference times its compute term on all-ones operands (CostModel.py:78-79); the default here is N(0, 0.02).  With
    the reference's link constants the two shipped tables lead ``emulateFFTime`` to the same slice counts for the
    GPT-3-like layers on every mesh of the sweep, or to neighbours whose modelled times tie: the slice count one table
    picks costs at most 0.5 % more than the best under the other table.  The modelled totals differ (ones is the faster)."""
    layers = [(B, I, O, df) for (_name, B, I, O, df) in Autotuner.gpt3_layers()]
    meshes = ((2, 8), (4, 4), (8, 8))
    picks, totals, times = {}, {}, {}
    try:
        for kind in ("normal", "ones"):
            CostModel.use_compute_term(CostModel.load_compute_term(operands=kind))
            for mesh in meshes:
                totals[kind, mesh], picks[kind, mesh] = Autotuner.emulateFFTime(layers, mesh, sweep=True)
                times[kind, mesh] = [{k: Autotuner.FFLayerModel(B, I, O, df).emulate(Autotuner.default_mesh(mesh), k)
                                      for k in Autotuner.possibleK(B, I, O, mesh, df)} for (B, I, O, df) in layers]
    finally:
        CostModel.use_compute_term(None)
    same = 0
    for mesh in meshes:
        assert totals["ones", mesh] < totals["normal", mesh]
        for kind, other in (("normal", "ones"), ("ones", "normal")):
            for layer, k in enumerate(picks[kind, mesh]):
                t = times[other, mesh][layer]
                assert t[k] <= 1.005 * min(t.values()), (mesh, layer, kind, k, t)
        same += picks["normal", mesh] == picks["ones", mesh]
    assert same >= 2      # (at the time of writing the 8x8 mesh's two feed-forward layers pick 4 against 3: 14.412 against 14.419 ms)
