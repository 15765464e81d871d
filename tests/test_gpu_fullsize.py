"""The three GPT-3-sized configurations (output-, LHS- and RHS-stationary) at their full sizes, checked through size-independent properties: sampled
rows / columns against the float64 oracle, slice-count invariance (S slices give the unsliced product),
linearity in one operand, and chunk independence."""
import numpy as np
import pytest
import torch

from oracle import meshslice_oracle as orc
import meshslice_amd as ms

pytestmark = pytest.mark.gpu
TOL_BF16 = 1e-2


def _randn_bf16(shape, scale, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return (torch.randn(shape, generator=g, device="cuda") * scale).to(torch.bfloat16)


def _f64(t):
    return t.float().cpu().numpy().astype(np.float64)


def _slices_cols(X, S, B=8):
    L = X.shape[1]
    return [X[:, torch.from_numpy(orc.sel(L, S, B, k)).cuda()].contiguous() for k in range(S)]


def _slices_rows(W, S, B=8):
    L = W.shape[0]
    return [W[torch.from_numpy(orc.sel(L, S, B, k)).cuda(), :].contiguous() for k in range(S)]


def test_config2_os_s4_full_size():
    """X[4096,12288] N(0,1), W[12288,12288] N(0,0.02), S=4 block-cyclic K slices -> C bf16."""
    X = _randn_bf16((4096, 12288), 1.0, 0); W = _randn_bf16((12288, 12288), 0.02, 1)
    A4, B4 = _slices_cols(X, 4), _slices_rows(W, 4)
    assert tuple(A4[0].shape) == (4096, 3072) and tuple(B4[0].shape) == (3072, 12288)
    C4 = ms.gemm_os(A4, B4)
    C1 = ms.gemm_os([X], [W])
    rows = np.random.default_rng(0).choice(4096, 48, replace=False)
    want = _f64(X[rows]) @ _f64(W)
    assert orc.rel_frobenius(_f64(C4[rows]), want) <= TOL_BF16
    assert orc.rel_frobenius(_f64(C1[rows]), want) <= TOL_BF16
    # S=4 and S=1 sum the same products in a different order: equal up to bf16 output rounding
    assert orc.rel_frobenius(_f64(C4), _f64(C1)) <= 4e-3
    cols = np.random.default_rng(1).choice(12288, 32, replace=False)
    want = _f64(X) @ _f64(W[:, cols])
    assert orc.rel_frobenius(_f64(C4[:, cols]), want) <= TOL_BF16
    # linearity: doubling one operand's slices doubles the output exactly (power-of-two scaling)
    C2 = ms.gemm_os([a * 2 for a in A4], B4)
    assert torch.equal(C2.float(), C4.float() * 2)


def test_config3_ls_s8_full_size():
    """A[4096,12288], gathered W[12288,12288] stored [out,in], S=8 -> 8 fp32 chunks [4096,1536]."""
    A = _randn_bf16((4096, 12288), 1.0, 2); W = _randn_bf16((12288, 12288), 0.02, 3)
    Ws = _slices_rows(W, 8)
    assert tuple(Ws[0].shape) == (1536, 12288)
    Y = ms.gemm_ls(A, Ws)
    assert len(Y) == 8 and tuple(Y[0].shape) == (4096, 1536) and Y[0].dtype == torch.float32
    rows = np.random.default_rng(2).choice(4096, 32, replace=False)
    for k in (0, 3, 7):
        want = _f64(A[rows]) @ _f64(Ws[k]).T
        assert orc.rel_frobenius(_f64(Y[k][rows]), want) <= TOL_BF16
    # chunk independence: chunk k alone (S=1 call on its slice) is bit-identical
    alone = ms.gemm_ls(A, [Ws[5]])[0]
    assert torch.equal(alone, Y[5])
    # scattering the chunks back by sel_k reproduces the unsliced product
    full = ms.gemm_ls(A, [W])[0]
    for k in (1, 6):
        idx = torch.from_numpy(orc.sel(12288, 8, 8, k)).cuda()
        assert torch.equal(full[:, idx], Y[k])


def test_config4_rs_s4_full_size():
    """X[4096,3072] (used transposed), dY[4096,12288] N(0,1e-3), S=4 -> 4 fp32 chunks [768,12288]."""
    X = _randn_bf16((4096, 3072), 1.0, 4); dY = _randn_bf16((4096, 12288), 1e-3, 5)
    Xs = _slices_cols(X, 4)
    assert tuple(Xs[0].shape) == (4096, 768)
    Y = ms.gemm_rs(Xs, dY)
    assert len(Y) == 4 and tuple(Y[0].shape) == (768, 12288)
    cols = np.random.default_rng(3).choice(12288, 64, replace=False)
    for k in range(4):
        want = _f64(Xs[k]).T @ _f64(dY[:, cols])
        assert orc.rel_frobenius(_f64(Y[k][:, cols]), want) <= TOL_BF16
    full = ms.gemm_rs([X], dY)[0]
    for k in (0, 2):
        idx = torch.from_numpy(orc.sel(3072, 4, 8, k)).cuda()
        assert torch.equal(full[idx, :], Y[k])


def test_os_with_a_fractional_last_round_is_split_into_two_launches():
    """X[4096,12288] x W[12288,9216], S=4: no single tile shape fills its last round of compute units, so the call
    runs the 256x384 tile on the first 6144 columns and the best shape for the rest on the other 3072.  The result
    is the single-launch one (same products summed in the same order per element), with and without the fused
    epilogue, for bf16 and fp32 outputs; the residual and the row moments follow the split."""
    from meshslice_amd import _lib
    L = _lib.load()
    X = _randn_bf16((4096, 12288), 1.0, 40); W = _randn_bf16((12288, 9216), 0.02, 41)
    A4, B4 = _slices_cols(X, 4), _slices_rows(W, 4)
    for out_dtype in (torch.bfloat16, torch.float32):
        L.ms_set_variant(0)
        got = ms.gemm_os(A4, B4, out_dtype=out_dtype)
        assert L.ms_query(_lib.MS_QUERY_LAST_LAUNCHES) == 2
        L.ms_set_variant(8)
        one = ms.gemm_os(A4, B4, out_dtype=out_dtype)
        assert L.ms_query(_lib.MS_QUERY_LAST_LAUNCHES) == 1
        L.ms_set_variant(0)
        assert torch.equal(got, one)
    rows = np.random.default_rng(3).choice(4096, 24, replace=False)
    assert orc.rel_frobenius(_f64(got[rows]), _f64(X[rows]) @ _f64(W)) <= 1e-5 * 50    # fp32 out of bf16 operands
    # fused epilogue through the split: GELU, a residual that spans both parts, row moments added by both launches
    R = _randn_bf16((4096, 9216), 1.0, 42)
    s1 = torch.zeros(4096, device="cuda"); s2 = torch.zeros(4096, device="cuda")
    fused = ms.gemm_os(A4, B4, activation="gelu", residual=R, row_moments=(s1, s2))
    assert L.ms_query(_lib.MS_QUERY_LAST_LAUNCHES) == 2
    L.ms_set_variant(8)
    t1 = torch.zeros(4096, device="cuda"); t2 = torch.zeros(4096, device="cuda")
    fused_one = ms.gemm_os(A4, B4, activation="gelu", residual=R, row_moments=(t1, t2))
    L.ms_set_variant(0)
    assert torch.equal(fused, fused_one)
    assert orc.rel_frobenius(_f64(s1), _f64(t1)) <= 1e-5 and orc.rel_frobenius(_f64(s2), _f64(t2)) <= 1e-5
    want = torch.nn.functional.gelu(got.float(), approximate="tanh") + R.float()
    assert orc.rel_frobenius(_f64(fused), _f64(want)) <= TOL_BF16
    # both launches are recorded when the call is captured in a HIP graph
    out = torch.empty((4096, 9216), dtype=torch.bfloat16, device="cuda")
    ms.gemm_os(A4, B4, out=out)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        ms.gemm_os(A4, B4, out=out)
    for _ in range(2):
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, ms.gemm_os(A4, B4))
    # a product that one shape covers in whole rounds stays one launch
    ms.gemm_os(_slices_cols(X, 4), _slices_rows(_randn_bf16((12288, 12288), 0.02, 43), 4))
    assert L.ms_query(_lib.MS_QUERY_LAST_LAUNCHES) == 1

