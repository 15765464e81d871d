"""The autotuner sweep's per-device shapes on the GPU: the fused S-slice call of every layout on the 2x8, 4x4 and
8x8 meshes against the float64 oracle, and the cost model's measuring path (``estimateMatmul``, ``measureFused``,
``sweep_compute_term``; reference CostModel.py:74-98, :249-285 and Autotuner.py:141-169).

Operands are bf16 N(0, 0.02), seeded by the case; tolerance rel-Frobenius <= 1e-2 (bf16 in, fp32 accumulate)
against float64 numpy products of the same bf16 values on sampled rows of the output.
"""
import zlib

import numpy as np
import pytest
import torch

from oracle import meshslice_oracle as orc
import meshslice_amd as ms
from meshslice_amd import Autotuner, CostModel, _lib

pytestmark = pytest.mark.gpu
TOL_BF16 = 1e-2
LAYERS = {name: (B, I, O, df) for (name, B, I, O, df) in Autotuner.gpt3_layers()}

# (mesh, layer, pass) whose per-slice shape has the wanted layout; one per mesh and layout
PICKS = [
    ((2, 8), "ff1", "fwd", "nn"),            # 8192 x 6144 x 12288/S
    ((4, 4), "in_proj", "fwd", "nn"),        # 4096 x 9216 x 12288/S: two launches (fractional last round)
    ((8, 8), "out_proj", "bwd_data", "nn"),  # 2048 x 1536 x 12288/S: 64 tiles for 256 compute units
    ((2, 8), "ff2", "fwd", "nt"),            # 8192 x 12288/S x 6144
    ((4, 4), "in_proj", "bwd_data", "nt"),   # 4096 x 12288/S x 9216
    ((8, 8), "out_proj", "fwd", "nt"),       # 2048 x 12288/S x 1536
    ((2, 8), "ff1", "bwd_weight", "tn"),     # 12288/S x 6144 x 8192
    ((4, 4), "out_proj", "bwd_weight", "tn"),  # 12288/S x 3072 x 4096
    ((8, 8), "out_proj", "bwd_weight", "tn"),  # 12288/S x 1536 x 2048: 768-row chunks at S = 16
]


def _shape(mesh, layer, pname, S):
    B, I, O, df = LAYERS[layer]
    (got,) = Autotuner.per_slice_shapes(B, I, O, df, mesh, S, passes=(pname,))
    return got[1:]   # (M, N, K, layout)


def _operand(shape, *key):
    g = torch.Generator(device="cuda").manual_seed(zlib.crc32(repr(key).encode()))
    return (torch.randn(shape, generator=g, device="cuda") * 0.02).to(torch.bfloat16)


def _f64(t):
    return t.float().cpu().numpy().astype(np.float64)


def test_the_picks_cover_the_shapes_the_sweep_is_known_for():
    assert _shape((4, 4), "in_proj", "fwd", 1) == (4096, 9216, 12288, "nn")
    assert _shape((8, 8), "out_proj", "bwd_data", 4) == (2048, 1536, 3072, "nn")
    assert _shape((8, 8), "out_proj", "bwd_weight", 16) == (768, 1536, 2048, "tn")
    for mesh, layer, pname, layout in PICKS:
        assert _shape(mesh, layer, pname, 4)[3] == layout


def _check_fused_call(mesh, layer, pname, S, nrows=12, ncols=192):
    """The one fused S-slice call a device issues for (mesh, layer, pass) against float64 numpy products of the same
    bf16 values on ``nrows`` sampled rows x ``ncols`` sampled columns of the output (of three chunks for LS / RS)."""
    M, N, K, layout = _shape(mesh, layer, pname, S)
    key = (mesh, layer, pname, S)
    rng = np.random.default_rng(zlib.crc32(repr(key).encode()))
    rows = torch.from_numpy(np.sort(rng.choice(M, min(M, nrows), replace=False))).cuda()
    cols = torch.from_numpy(np.sort(rng.choice(N, min(N, ncols), replace=False))).cuda()
    if layout == "nn":      # C = sum_s A_s @ B_s
        A = [_operand((M, K), key, "a", s) for s in range(S)]
        Bm = [_operand((K, N), key, "b", s) for s in range(S)]
        C = ms.gemm_os(A, Bm)
        want = sum(_f64(a[rows]) @ _f64(b[:, cols]) for a, b in zip(A, Bm))
        assert orc.rel_frobenius(_f64(C[rows][:, cols]), want) <= TOL_BF16
    elif layout == "nt":    # Y_s = A @ W_s^T
        A = _operand((M, K), key, "a")
        W = [_operand((N, K), key, "w", s) for s in range(S)]
        Y = ms.gemm_ls(A, W)
        for s in sorted({0, S // 2, S - 1}):
            assert orc.rel_frobenius(_f64(Y[s][rows][:, cols]), _f64(A[rows]) @ _f64(W[s][cols]).T) <= TOL_BF16
    else:                   # Y_s = X_s^T @ W
        X = [_operand((K, M), key, "x", s) for s in range(S)]
        W = _operand((K, N), key, "w")
        Y = ms.gemm_rs(X, W)
        Wd = _f64(W[:, cols])
        for s in sorted({0, S // 2, S - 1}):
            assert orc.rel_frobenius(_f64(Y[s][rows][:, cols]), _f64(X[s][:, rows]).T @ Wd) <= TOL_BF16
    return M, N, K, layout


@pytest.mark.parametrize("S", [1, 4, 16])
@pytest.mark.parametrize("mesh,layer,pname,layout", PICKS, ids=[f"{m[0]}x{m[1]}-{l}-{p}" for m, l, p, _ in PICKS])
def test_fused_call_of_a_sweep_shape_matches_the_oracle(mesh, layer, pname, layout, S):
    M, N, K, lay = _check_fused_call(mesh, layer, pname, S, ncols=1 << 30)      # whole sampled rows
    assert lay == layout
    if (M, N, K * S) == (4096, 9216, 12288):
        assert _lib.load().ms_query(_lib.MS_QUERY_LAST_LAUNCHES) == 2


# The sweep of BASELINE's configuration 5 row by row: the four forward GEMMs of one GPT-3-like layer (reference
# BenchTransformer.py:80-93) on the 2x8, 4x4 and 8x8 meshes at every slice count of the sweep (per-slice shapes by
# reference CostModel.py:249-285): 60 rows; and one backward-data and one backward-weight row per mesh at S = 2 and 8.
MESHES = [(2, 8), (4, 4), (8, 8)]
SLICE_COUNTS = [1, 2, 4, 8, 16]
FORWARD_ROWS = [(mesh, layer, "fwd", S) for mesh in MESHES for layer in ("in_proj", "out_proj", "ff1", "ff2") for S in SLICE_COUNTS]
BACKWARD_ROWS = [(mesh, layer, pname, S) for mesh, layer, pname in
                 [((2, 8), "ff1", "bwd_data"), ((2, 8), "ff2", "bwd_weight"), ((4, 4), "ff2", "bwd_data"), ((4, 4), "ff1", "bwd_weight"),
                  ((8, 8), "in_proj", "bwd_data"), ((8, 8), "ff2", "bwd_weight")] for S in (2, 8)]


def test_the_forward_rows_are_the_sixty_of_the_sweep():
    assert len(FORWARD_ROWS) == 60 and len(set(FORWARD_ROWS)) == 60
    assert {_shape(m, l, p, S)[3] for m, l, p, S in FORWARD_ROWS} == {"nn", "nt"}
    assert {_shape(m, l, p, S)[3] for m, l, p, S in BACKWARD_ROWS} == {"nn", "nt", "tn"}
    assert _shape((4, 4), "ff1", "fwd", 4) == (4096, 12288, 3072, "nn")           # configuration 2
    assert _shape((4, 4), "ff2", "fwd", 8) == (4096, 1536, 12288, "nt")           # configuration 3
    assert _shape((4, 4), "ff1", "bwd_weight", 4) == (3072, 12288, 4096, "tn")    # configuration 4's product, all four slices


@pytest.mark.parametrize("mesh,layer,pname,S", FORWARD_ROWS + BACKWARD_ROWS,
                         ids=[f"{m[0]}x{m[1]}-{l}-{p}-S{S}" for m, l, p, S in FORWARD_ROWS + BACKWARD_ROWS])
def test_every_row_of_the_sweep_matches_the_oracle(mesh, layer, pname, S):
    _check_fused_call(mesh, layer, pname, S)


@pytest.mark.parametrize("layout,shape", [("nn", (4096, 12288, 3072)), ("nt", (4096, 3072, 9216)), ("tn", (3072, 12288, 8192))])
@pytest.mark.parametrize("operands", ["normal", "ones"])
def test_estimate_matmul_measures_on_the_gpu_and_caches(layout, shape, operands):
    CostModel.use_compute_term(None)
    CostModel._measured.clear()
    M, N, K = shape
    t = CostModel.estimateMatmul(None, M, N, K, layout=layout, operands=operands)
    ideal = 2.0 * M * N * K / CostModel.BF16_PEAK_FLOPS
    assert ideal < t < 3.0 * ideal
    assert len(CostModel._measured) == 1
    assert CostModel.estimateMatmul(None, M, N, K, layout=layout, operands=operands) == t      # served from the cache
    assert len(CostModel._measured) == 1
    # the fused call that does S = 4 such slices costs about four of them (and never less than their ideal time)
    tf = CostModel.measureFused(M, N, K, 4, layout=layout, operands=operands)
    assert 4 * ideal < tf < 4 * 3.0 * ideal


def test_sweep_compute_term_fits_a_term_that_reproduces_its_table():
    CostModel.use_compute_term(None)
    CostModel._measured.clear()
    layers = [l for l in Autotuner.gpt3_layers() if l[0] == "out_proj"]
    term, rows = Autotuner.sweep_compute_term(meshes=((8, 8),), slice_counts=(4, 16), passes=("fwd", "bwd_data"),
                                              layers=layers, repeat=3, verbose=False, fused=True)
    assert len(rows) == 4 and set(term.eta) == {"nt", "nn"}
    for (mesh, lname, pname, S, M, N, K, layout, sec, fused_sec) in rows:
        assert term.seconds(M, N, K, layout) == sec                     # table look-up
        assert 2.0 * M * N * K / CostModel.BF16_PEAK_FLOPS < sec < 1e-3
        assert fused_sec > 2.0 * M * N * K * S / CostModel.BF16_PEAK_FLOPS
    # off the table the fitted line answers
    for lay in term.eta:
        assert 0.05 < term.eta[lay] < 2.0 and term.t0[lay] >= 0.0
        want = term.t0[lay] + 2.0 * 1000 * 2000 * 3000 / (term.eta[lay] * term.peak)
        assert term.seconds(1000, 2000, 3000, lay) == pytest.approx(want, rel=1e-12)
    # installed, the term feeds the models without touching the GPU again
    CostModel.use_compute_term(term)
    try:
        n = len(CostModel._measured)
        M, N, K, layout = rows[0][4:8]
        assert CostModel.estimateMatmul(None, M, N, K, layout=layout) == rows[0][8]
        assert len(CostModel._measured) == n
    finally:
        CostModel.use_compute_term(None)
