"""Parity of the HIP path against the oracle, through the C ABI, on the GPU.

Tolerances (rel-Frobenius error ||C - C_ref||_F / ||C_ref||_F against the float64 oracle evaluated on
the dtype-rounded inputs): 1e-5 for fp32 in / fp32 out, 1e-2 for bf16 in / fp32 accumulate.
"""
import ctypes
import itertools
import json
import os

import numpy as np
import pytest
import torch

from oracle import meshslice_oracle as orc
import meshslice_amd as ms
from meshslice_amd import _lib
from meshslice_amd import TensorParallel as TP
from meshslice_amd.ShardedLayers import ShardedFFLayer
from meshslice_amd.mesh import Mesh, create_device_mesh

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOL_F32 = 1e-5
TOL_BF16 = 1e-2


def dev(a, dtype=torch.float32):
    return torch.from_numpy(np.ascontiguousarray(a)).to("cuda").to(dtype)


def host(t):
    return t.detach().float().cpu().numpy().astype(np.float64)


@pytest.fixture(autouse=True)
def _default_variant():
    _lib.load().ms_set_variant(0)
    yield
    _lib.load().ms_set_variant(0)
    torch.cuda.synchronize()


# ------------------------------------------------------------------ the fp32 plumbing configuration (2x2 mesh, 1024^2, S=4)
def test_config1_fp32_os_device00_matches_oracle():
    rng = np.random.default_rng(0)
    A = rng.standard_normal((1024, 1024)).astype(np.float32)
    B = rng.standard_normal((1024, 1024)).astype(np.float32)
    R = C = 2; S = 4; blk = 8
    As, Bs = orc.device_operands_os(A, B, R, C, 0, 0, S, blk)
    assert As[0].shape == (512, 256) and Bs[0].shape == (256, 512)
    got = ms.gemm_os([dev(a) for a in As], [dev(b) for b in Bs])
    want = orc.oracle_os_block(As, Bs)
    assert np.array_equal(want, A[:512].astype(np.float64) @ B[:, :512].astype(np.float64)) or \
        orc.rel_frobenius(want, A[:512].astype(np.float64) @ B[:, :512].astype(np.float64)) < 1e-14
    assert orc.rel_frobenius(host(got), want) <= TOL_F32
    # the same block through the reference-shaped API
    mesh = Mesh(create_device_mesh((2, 2)), ("row", "col"))
    blk00 = TP.SPMD(mesh, "meshflow").OS(4).device(0, 0)(dev(A), dev(B))
    assert torch.equal(blk00, got)


# ------------------------------------------------------------------ notebook walkthrough (known answers)
@pytest.fixture(scope="module")
def nb():
    d = orc.notebook_inputs(np.float32)
    g = json.load(open(os.path.join(ROOT, "tests", "golden", "notebook_blocks.json")))
    return d, g


@pytest.mark.parametrize("alg", ["collective", "meshflow"])
@pytest.mark.parametrize("flow", ["os", "ls", "rs"])
def test_notebook_whole_mesh_matches_golden_and_reference_allclose(nb, alg, flow):
    d, g = nb
    mesh = Mesh(create_device_mesh(d["mesh"]), ("row", "col"))
    X, W = {"os": (d["X"], d["W"]), "ls": (d["dY"], d["W"]), "rs": (d["X"], d["dY"])}[flow]
    f = getattr(TP.SPMD(mesh, alg), flow.upper())()         # default K=8, blocksize=8 as in the notebook
    Y = host(f(dev(X), dev(W)))
    want = orc.dense(flow, X, W)
    assert orc.allclose(Y, want)                              # the reference's own criterion
    assert orc.rel_frobenius(Y, want) <= TOL_F32
    R, C = d["mesh"]
    for key, st in g[flow].items():
        i, j = map(int, key.split(","))
        blk = orc.shard(Y, R, C, i, j)
        assert blk.sum() == pytest.approx(st["sum"], rel=1e-5)
        assert np.allclose([blk[0, 0], blk[0, -1], blk[-1, 0], blk[-1, -1]], st["corners"], rtol=2e-5, atol=0)


def test_selfcheck_chain_on_one_device():
    """TensorParallel.py:433-457 on the 4x4 mesh: Yo=OS(X,W); LS(Yo,W); RS(X,Yo); device (2,1)."""
    d = orc.selfcheck_inputs(np.float32)
    R, C = d["mesh"]; S, B = d["K"], d["blocksize"]
    mesh = Mesh(create_device_mesh((R, C)), ("x", "y"))
    alg = TP.SPMD(mesh, "meshflow")
    X, W = dev(d["X"]), dev(d["W"])
    i, j = 2, 1
    blk = alg.OS().device(i, j)(X, W)
    want = orc.oracle_os_block(*orc.device_operands_os(d["X"], d["W"], R, C, i, j, S, B))
    assert orc.rel_frobenius(host(blk), want) <= TOL_F32
    Yo = (d["X"].astype(np.float64) @ d["W"].astype(np.float64)).astype(np.float32)
    chunks = alg.LS().device(i, j)(dev(Yo), W)
    want = orc.oracle_ls_chunks(*orc.device_operands_ls(Yo, d["W"], R, C, i, j, S, B))
    assert max(orc.rel_frobenius(host(c), w) for c, w in zip(chunks, want)) <= TOL_F32
    chunks = alg.RS().device(i, j)(X, dev(Yo))
    want = orc.oracle_rs_chunks(*orc.device_operands_rs(d["X"], Yo, R, C, i, j, S, B))
    assert max(orc.rel_frobenius(host(c), w) for c, w in zip(chunks, want)) <= TOL_F32


# ------------------------------------------------------------------ seeded random cases, every kernel variant
SHAPES = [  # (m, n, k_or_slice, S)
    (512, 512, 256, 4),
    (256, 256, 64, 1),       # a single K step
    (256, 256, 192, 1),      # odd number of K steps
    (1000, 776, 328, 3),     # ragged in every dimension, K tail of 8
    (264, 520, 72, 2),       # K tail after one full step, per slice
    (8, 8, 8, 1),            # smallest admissible problem
    (40, 4096, 136, 16),     # wide and thin, many slices
]


def _rand_case(flow, m, n, k, S, seed, dtype):
    rng = np.random.default_rng(seed)
    rnd = (lambda s, sc=1.0: orc.bf16_round(rng.standard_normal(s).astype(np.float32) * sc)) if dtype == torch.bfloat16 \
        else (lambda s, sc=1.0: rng.standard_normal(s).astype(np.float32) * np.float32(sc))
    if flow == "os":
        return [rnd((m, k)) for _ in range(S)], [rnd((k, n), 0.05) for _ in range(S)]
    if flow == "ls":
        return rnd((m, k)), [rnd((n, k), 0.05) for _ in range(S)]
    return [rnd((k, m)) for _ in range(S)], rnd((k, n), 0.05)


def _run_and_compare(flow, ops, dtype, tol, out_dtype=None):
    if flow == "os":
        A, B = ops
        got = ms.gemm_os([dev(a, dtype) for a in A], [dev(b, dtype) for b in B], out_dtype=out_dtype)
        err = orc.rel_frobenius(host(got), orc.oracle_os_block(A, B))
    elif flow == "ls":
        A, W = ops
        got = ms.gemm_ls(dev(A, dtype), [dev(w, dtype) for w in W])
        err = max(orc.rel_frobenius(host(g), w) for g, w in zip(got, orc.oracle_ls_chunks(A, W)))
    else:
        X, W = ops
        got = ms.gemm_rs([dev(x, dtype) for x in X], dev(W, dtype))
        err = max(orc.rel_frobenius(host(g), w) for g, w in zip(got, orc.oracle_rs_chunks(X, W)))
    assert err <= tol, f"{flow}: rel-Frobenius {err:.3e} > {tol}"
    return err


@pytest.mark.parametrize("variant", [1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14])
@pytest.mark.parametrize("flow", ["os", "ls", "rs"])
def test_bf16_random_cases_all_variants(flow, variant):
    _lib.check(_lib.load().ms_set_variant(variant))
    for idx, (m, n, k, S) in enumerate(SHAPES):
        ops = _rand_case(flow, m, n, k, S, seed=100 * idx + variant, dtype=torch.bfloat16)
        _run_and_compare(flow, ops, torch.bfloat16, TOL_BF16)
        if flow != "os":
            continue
        # fp32 output of the same accumulators is far inside the bf16 tolerance
        err = _run_and_compare(flow, ops, torch.bfloat16, TOL_BF16, out_dtype=torch.float32)
        assert err < 1e-5


@pytest.mark.parametrize("variant", [3, 7, 8, 10, 11, 12, 13, 14])
@pytest.mark.parametrize("flow", ["os", "rs"])
def test_more_tiles_than_compute_units_with_a_partly_filled_last_round(flow, variant):
    """5120 x 5120 outputs are 280 to 1600 tiles, a whole number of rounds for none of the tile shapes on a device of
    some hundred compute units: such launches run on fewer workgroups, evenly filled, and every tile must still be
    computed exactly once (an fp32 result far inside the bf16 tolerance says so: a tile done twice would not show, a
    tile left out would)."""
    m = n = 5120; k = 64; S = 2
    _lib.check(_lib.load().ms_set_variant(variant))
    ops = _rand_case(flow, m if flow == "os" else m // S, n, k, S, seed=variant, dtype=torch.bfloat16)
    if flow == "os":
        got = ms.gemm_os([dev(a, torch.bfloat16) for a in ops[0]], [dev(b, torch.bfloat16) for b in ops[1]], out_dtype=torch.float32)
        err = orc.rel_frobenius(host(got), orc.oracle_os_block(*ops))
    else:
        got = ms.gemm_rs([dev(x, torch.bfloat16) for x in ops[0]], dev(ops[1], torch.bfloat16))
        err = max(orc.rel_frobenius(host(g), w) for g, w in zip(got, orc.oracle_rs_chunks(*ops)))
    assert err < 1e-5, err


@pytest.mark.parametrize("flow", ["os", "ls", "rs"])
def test_fp32_random_cases(flow):
    for idx, (m, n, k, S) in enumerate(SHAPES + [(200, 136, 100, 3), (68, 60, 20, 2)]):
        ops = _rand_case(flow, m, n, k, S, seed=7 + idx, dtype=torch.float32)
        _run_and_compare(flow, ops, torch.float32, TOL_F32)


@pytest.mark.parametrize("tile", [21, 22, 23, 24, 25])
@pytest.mark.parametrize("flow", ["os", "ls", "rs"])
def test_fp32_random_cases_on_every_tile(flow, tile):
    """The fp32 kernel's five tiles (256x128 and 128x192 on eight waves, 128x128, 64x64 and 192x192 on four), each forced."""
    lib = _lib.load()
    _lib.check(lib.ms_set_variant(tile))
    for idx, (m, n, k, S) in enumerate(SHAPES + [(200, 136, 100, 3), (300, 1000, 260, 1)]):
        ops = _rand_case(flow, m, n, k, S, seed=31 * tile + idx, dtype=torch.float32)
        _run_and_compare(flow, ops, torch.float32, TOL_F32)
        assert lib.ms_query(_lib.MS_QUERY_LAST_VARIANT) == tile


@pytest.mark.parametrize("flow", ["os", "ls", "rs"])
def test_fp32_long_all_positive_contraction_is_summed_in_blocks(flow):
    """16384 all-positive terms per output: one fp32 accumulator through the whole contraction drifts to about 2e-6 of
    the result (measured, with the vendor library as well); summed in blocks of 128 terms the kernel stays near 2e-7.
    The bound sits between the two, so it fails if the blocks are lost, well before the 1e-5 of the other fp32 tests."""
    m, n, k, S = 320, 264, 16384, 2
    g = torch.Generator(device="cuda").manual_seed(11)
    X = torch.rand((m, k), generator=g, device="cuda")
    W = torch.rand((k, n), generator=g, device="cuda")
    want = X.double() @ W.double()
    if flow == "os":
        got = ms.gemm_os([X[:, :k // 2].contiguous(), X[:, k // 2:].contiguous()], [W[:k // 2].contiguous(), W[k // 2:].contiguous()])
    elif flow == "ls":
        Wt = W.t().contiguous()
        got = torch.cat(ms.gemm_ls(X, [Wt[:n // 2].contiguous(), Wt[n // 2:].contiguous()], out_dtype=torch.float32), dim=1)
    else:
        Xt = X.t().contiguous()
        got = torch.cat(ms.gemm_rs([Xt[:, :m // 2].contiguous(), Xt[:, m // 2:].contiguous()], W, out_dtype=torch.float32), dim=0)
    err = ((got.double() - want).norm() / want.norm()).item()
    assert err < 6e-7, err


def test_bf16_output_is_one_rounding_of_the_fp32_accumulator():
    """OS accumulates all slices in fp32 and rounds once: the bf16 result equals the round-to-nearest-even
    of the fp32-output result of the same call, bit for bit."""
    A, B = _rand_case("os", 512, 768, 256, 4, seed=3, dtype=torch.bfloat16)
    a = [dev(x, torch.bfloat16) for x in A]; b = [dev(x, torch.bfloat16) for x in B]
    c32 = ms.gemm_os(a, b, out_dtype=torch.float32)
    c16 = ms.gemm_os(a, b, out_dtype=torch.bfloat16)
    want = orc.bf16_bits(c32.cpu().numpy())
    got = c16.view(torch.int16).cpu().numpy().view(np.uint16)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("variant", [0, 1, 3, 5, 8, 10, 11, 12, 13, 14, 21, 22, 23, 24, 25])
@pytest.mark.parametrize("flow", ["ls", "rs"])
@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32])
def test_bf16_chunks_are_one_rounding_of_the_fp32_chunks(flow, variant, in_dtype):
    """ms_gemm_ls_ex / ms_gemm_rs_ex with bf16 chunks (what the reference's einsum hands to its reduce-scatter):
    every chunk equals the round-to-nearest-even of the fp32 chunk of the same call, bit for bit, also on
    ragged shapes, and nothing is written outside a strided chunk."""
    if variant and (in_dtype == torch.float32) != (variant >= 21):
        pytest.skip("variants 1-14 are tiles of the bf16 kernels, 21-25 of the fp32 kernel")
    _lib.check(_lib.load().ms_set_variant(variant))
    for (m, n, k, S) in [(512, 768, 256, 3), (264, 520, 72, 2), (1000, 776, 328, 2)]:
        ops = _rand_case(flow, m, n, k, S, seed=17 + variant, dtype=in_dtype)
        if flow == "ls":
            A, W = ops
            a = dev(A, in_dtype); w = [dev(x, in_dtype) for x in W]
            y32 = ms.gemm_ls(a, w)
            pad = torch.zeros((S, m, n + 8), dtype=torch.bfloat16, device="cuda")
            y16 = ms.gemm_ls(a, w, out=[pad[s][:, :n] for s in range(S)])
        else:
            X, W = ops
            x = [dev(t, in_dtype) for t in X]; w = dev(W, in_dtype)
            y32 = ms.gemm_rs(x, w)
            pad = torch.zeros((S, m, n + 8), dtype=torch.bfloat16, device="cuda")
            y16 = ms.gemm_rs(x, w, out=[pad[s][:, :n] for s in range(S)])
        for c32, c16 in zip(y32, y16):
            assert c16.dtype == torch.bfloat16
            want = orc.bf16_bits(c32.cpu().numpy())
            got = c16.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)
            assert np.array_equal(got, want)
        assert float(pad[:, :, n:].abs().max()) == 0.0
    fresh = ms.gemm_ls(a, w, out_dtype=torch.bfloat16) if flow == "ls" else ms.gemm_rs(x, w, out_dtype=torch.bfloat16)
    assert all(torch.equal(f, c) for f, c in zip(fresh, y16))


def test_strided_operands_and_outputs():
    """Leading dimensions larger than the row length (slices that are views of a bigger buffer)."""
    rng = np.random.default_rng(5)
    m, n, k, S = 300, 264, 128, 2
    bigA = orc.bf16_round(rng.standard_normal((m, S * k + 16)).astype(np.float32))
    bigB = orc.bf16_round(rng.standard_normal((S * k, n + 40)).astype(np.float32) * 0.05)
    dA, dB = dev(bigA, torch.bfloat16), dev(bigB, torch.bfloat16)
    A = [dA[:, s * k:(s + 1) * k] for s in range(S)]
    B = [dB[s * k:(s + 1) * k, :n] for s in range(S)]
    out = torch.zeros((m, n + 24), dtype=torch.bfloat16, device="cuda")
    ms.gemm_os(A, B, out=out[:, :n])
    want = orc.oracle_os_block([bigA[:, s * k:(s + 1) * k] for s in range(S)], [bigB[s * k:(s + 1) * k, :n] for s in range(S)])
    assert orc.rel_frobenius(host(out[:, :n]), want) <= TOL_BF16
    assert float(out[:, n:].abs().max()) == 0.0            # nothing written outside the block


# ------------------------------------------------------------------ whole-mesh API on random bf16 data
@pytest.mark.parametrize("R,C,K", [(2, 2, 2), (4, 2, 4), (2, 4, 2)])
@pytest.mark.parametrize("flow", ["os", "ls", "rs"])
def test_meshflow_equals_collective_equals_dense(flow, R, C, K):
    rng = np.random.default_rng(R * 10 + C + K)
    u = R * C * K * 8
    shp = {"os": ((4 * R * 8, u), (u, 2 * u)), "ls": ((4 * R * 8, 2 * C * 16), (u, 2 * C * 16)),
           "rs": ((4 * R * 8, u), (4 * R * 8, 3 * C * 8))}[flow]
    X = orc.bf16_round(rng.standard_normal(shp[0]).astype(np.float32))
    W = orc.bf16_round(rng.standard_normal(shp[1]).astype(np.float32) * 0.1)
    mesh = Mesh(create_device_mesh((R, C)), ("row", "col"))
    dX, dW = dev(X, torch.bfloat16), dev(W, torch.bfloat16)
    want = orc.dense(flow, X, W)
    y_c = getattr(TP.SPMD(mesh, "collective"), flow.upper())(K)(dX, dW)
    y_m = getattr(TP.SPMD(mesh, "meshflow"), flow.upper())(K)(dX, dW)
    assert y_c.dtype == torch.bfloat16 and y_m.dtype == torch.bfloat16 and tuple(y_m.shape) == want.shape
    assert orc.rel_frobenius(host(y_c), want) <= TOL_BF16
    assert orc.rel_frobenius(host(y_m), want) <= TOL_BF16
    assert TP.allclose(y_m, y_c)
    # the sliced result also matches the literal whole-mesh emulation of the reference body
    lit = orc.literal_meshflow(flow, X.astype(np.float64), W.astype(np.float64), R, C, K, 8)
    assert orc.rel_frobenius(host(y_m), lit) <= TOL_BF16


@pytest.mark.parametrize("algorithm,R,C", [("wang", 2, 4), ("wang", 4, 2), ("cannon", 2, 2), ("cannon", 4, 4)])
@pytest.mark.parametrize("flow", ["os", "ls", "rs"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_ring_baselines_equal_dense_and_the_literal_emulation(flow, algorithm, R, C, dtype):
    """SPMD(mesh, 'wang' | 'cannon'): every device multiplies its 2 * size half-blocks in ring order in one kernel
    call; the whole-mesh result equals the dense product, the collective body's result and the literal emulation
    of the reference's ring bodies; a device's partial equals the collective body's partial."""
    rng = np.random.default_rng(R * 10 + C)
    u = R * C * 2 * 8
    shp = {"os": ((4 * R * 8, 2 * u), (2 * u, 3 * C * 8)), "ls": ((4 * R * 8, 2 * C * 16), (2 * u, 2 * C * 16)),
           "rs": ((4 * R * 8, 2 * u), (4 * R * 8, 3 * C * 8))}[flow]
    rnd = (lambda a: orc.bf16_round(a)) if dtype == torch.bfloat16 else (lambda a: a)
    X = rnd(rng.standard_normal(shp[0]).astype(np.float32))
    W = rnd(rng.standard_normal(shp[1]).astype(np.float32) * np.float32(0.1))
    tol = TOL_BF16 if dtype == torch.bfloat16 else TOL_F32
    mesh = Mesh(create_device_mesh((R, C)), ("row", "col"))
    dX, dW = dev(X, dtype), dev(W, dtype)
    ring = getattr(TP.SPMD(mesh, algorithm), flow.upper())()
    coll = getattr(TP.SPMD(mesh, "collective"), flow.upper())()
    y = ring(dX, dW)
    want = orc.dense(flow, X, W)
    assert y.dtype == dtype and tuple(y.shape) == want.shape
    assert orc.rel_frobenius(host(y), want) <= tol
    assert orc.rel_frobenius(host(y), orc.literal_ring(algorithm, flow, X.astype(np.float64), W.astype(np.float64), R, C)) <= tol
    assert TP.allclose(y, coll(dX, dW))
    i, j = R - 1, C // 2
    got, ref = ring.device(i, j)(dX, dW), coll.device(i, j)(dX, dW)
    if flow == "os":
        blk = want[i * want.shape[0] // R:(i + 1) * want.shape[0] // R, j * want.shape[1] // C:(j + 1) * want.shape[1] // C]
        assert orc.rel_frobenius(host(got), blk) <= tol
    else:
        assert len(got) == 1 and tuple(got[0].shape) == tuple(ref[0].shape)
        assert orc.rel_frobenius(host(got[0]), host(ref[0])) <= 1e-6      # same terms per element, same k order


@pytest.mark.parametrize("dataflow", ["os", "ls", "rs"])
def test_sharded_ff_layer_forward_and_vjp(dataflow):
    """reference ShardedLayers.py:41-81: (fwd, dx, dw) = (OS,LS,RS) / (LS,OS,RS) / (RS,LS,OS)."""
    mesh = Mesh(create_device_mesh((2, 2)), ("row", "col"))
    tokens, in_dim, out_dim, ks = 128, 64, 96, 2
    layer = ShardedFFLayer(mesh, "meshflow", dataflow, ks, in_dim, out_dim, seed=4)
    assert tuple(layer.weight.shape) == ((out_dim, in_dim) if dataflow == "ls" else (in_dim, out_dim))
    assert layer.weight.dtype == torch.bfloat16
    g = torch.Generator().manual_seed(9)
    xs = (in_dim, tokens) if dataflow == "rs" else (tokens, in_dim)
    x = torch.randn(xs, generator=g).to(torch.bfloat16).cuda().requires_grad_(True)
    w = layer.weight.clone().requires_grad_(True)
    y = layer.forward(x, w)
    xr = x.detach().double().requires_grad_(True); wr = w.detach().double().requires_grad_(True)
    yr = {"os": lambda: xr @ wr, "ls": lambda: xr @ wr.t(), "rs": lambda: xr.t() @ wr}[dataflow]()
    assert orc.rel_frobenius(host(y), yr.detach().cpu().numpy()) <= TOL_BF16
    dy = torch.randn(tuple(y.shape), generator=g).to(torch.bfloat16).cuda()
    y.backward(dy)
    yr.backward(dy.double())
    assert orc.rel_frobenius(host(x.grad), xr.grad.cpu().numpy()) <= TOL_BF16
    assert orc.rel_frobenius(host(w.grad), wr.grad.cpu().numpy()) <= TOL_BF16


# ------------------------------------------------------------------ error behaviour through the C ABI
def test_c_abi_rejects_bad_arguments():
    lib = _lib.load()
    a = torch.zeros((64, 64), dtype=torch.bfloat16, device="cuda")
    c = torch.zeros((64, 64), dtype=torch.bfloat16, device="cuda")
    pa, _k1 = _lib.ptr_array([a.data_ptr()]); pb, _k2 = _lib.ptr_array([a.data_ptr()])
    vp = ctypes.c_void_p
    call = lambda **kw: lib.ms_gemm_os(kw.get("pa", pa), kw.get("pb", pb), kw.get("S", 1), kw.get("m", 64), kw.get("n", 64),
                                       kw.get("k", 64), kw.get("lda", 64), kw.get("ldb", 64), vp(kw.get("c", c.data_ptr())),
                                       kw.get("ldc", 64), kw.get("idt", 1), kw.get("odt", 1), None)
    assert call() == _lib.MS_OK
    assert call(S=0) == _lib.MS_ERR_ARG and "S = 0" in _lib.last_error()
    assert call(S=65) == _lib.MS_ERR_ARG
    assert call(m=0) == _lib.MS_ERR_ARG
    assert call(k=60) == _lib.MS_ERR_ARG           # contiguous extent not a multiple of 8
    assert call(lda=32) == _lib.MS_ERR_ARG         # leading dimension smaller than the row
    assert call(c=c.data_ptr() + 2) == _lib.MS_ERR_ARG
    assert call(c=0) == _lib.MS_ERR_ARG
    assert call(idt=7) == _lib.MS_ERR_UNSUPPORTED
    null, _k3 = _lib.ptr_array([0])
    assert call(pa=null) == _lib.MS_ERR_ARG
    assert lib.ms_set_variant(99) == _lib.MS_ERR_ARG
    assert lib.ms_set_variant(26) == _lib.MS_ERR_ARG and lib.ms_set_variant(121) == _lib.MS_ERR_ARG      # fp32 tiles are 21-25; a split is 2..8 ways
    with pytest.raises(ValueError):
        ms.gemm_os([a], [torch.zeros((32, 64), dtype=torch.bfloat16, device="cuda")])
    with pytest.raises(ValueError):
        _lib.check(call(S=0))
    torch.cuda.synchronize()


def test_query_reports_the_device():
    lib = _lib.load()
    assert lib.ms_query(_lib.MS_QUERY_IS_GFX950) == 1
    assert lib.ms_query(_lib.MS_QUERY_CU_COUNT) == torch.cuda.get_device_properties(0).multi_processor_count
    assert lib.ms_query(_lib.MS_QUERY_LDS_BYTES) >= 160 * 1024
    assert lib.ms_query(1234) == -1


# ------------------------------------------------------------------ streams, graphs, limits
def test_non_default_stream_and_stream_ordering():
    """Calls are asynchronous on the caller's stream: work queued on a side stream is ordered after the
    producer on that stream and before the consumer."""
    A, B = _rand_case("os", 512, 384, 256, 2, seed=21, dtype=torch.bfloat16)
    want = orc.oracle_os_block(A, B)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        a = [dev(x, torch.bfloat16) for x in A]; b = [dev(x, torch.bfloat16) for x in B]
        out = ms.gemm_os(a, b, out_dtype=torch.float32)
        doubled = out * 2
    torch.cuda.current_stream().wait_stream(side)
    assert orc.rel_frobenius(host(doubled), 2 * want) <= TOL_BF16


def test_hip_graph_capture_and_replay():
    """The entry points launch kernels only (no allocation, no memset), so they can be captured; every
    replay is checked against the eager result, with eager work in between."""
    A, W = _rand_case("ls", 384, 256, 320, 3, seed=22, dtype=torch.bfloat16)
    a = dev(A, torch.bfloat16); ws = [dev(w, torch.bfloat16) for w in W]
    eager = [t.clone() for t in ms.gemm_ls(a, ws)]
    outs = [torch.zeros_like(t) for t in eager]
    ms.gemm_ls(a, ws, out=outs)                      # warm-up outside capture
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        ms.gemm_ls(a, ws, out=outs)
    for rep in range(3):
        for t in outs:
            t.zero_()
        scratch = ms.gemm_os([a], [ws[0].t().contiguous()])   # eager work between replays
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        for got, want in zip(outs, eager):
            assert torch.equal(got, want), f"replay {rep} differs from the eager result"
        del scratch


def test_maximum_slice_count_and_one_beyond():
    S = 64
    A, B = _rand_case("os", 72, 136, 16, S, seed=23, dtype=torch.bfloat16)
    _run_and_compare("os", (A, B), torch.bfloat16, TOL_BF16)
    X, W = _rand_case("rs", 40, 264, 24, S, seed=24, dtype=torch.bfloat16)
    _run_and_compare("rs", (X, W), torch.bfloat16, TOL_BF16)
    a = [dev(x, torch.bfloat16) for x in A] + [dev(A[0], torch.bfloat16)]
    b = [dev(x, torch.bfloat16) for x in B] + [dev(B[0], torch.bfloat16)]
    with pytest.raises(ValueError, match="S = 65"):
        ms.gemm_os(a, b)


def test_concurrent_host_threads_on_separate_streams():
    import threading
    cases = [_rand_case("os", 256 + 8 * t, 264, 128, 2, seed=30 + t, dtype=torch.bfloat16) for t in range(4)]
    results, errors = [None] * 4, []

    def work(t):
        try:
            torch.cuda.set_device(0)
            st = torch.cuda.Stream()
            with torch.cuda.stream(st):
                A, B = cases[t]
                for _ in range(5):
                    out = ms.gemm_os([dev(x, torch.bfloat16) for x in A], [dev(x, torch.bfloat16) for x in B],
                                     out_dtype=torch.float32)
                st.synchronize()
                results[t] = host(out)
        except Exception as e:  # pragma: no cover
            errors.append(e)

    threads = [threading.Thread(target=work, args=(t,)) for t in range(4)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors
    for t in range(4):
        assert orc.rel_frobenius(results[t], orc.oracle_os_block(*cases[t])) <= TOL_BF16


def test_nan_and_inf_propagate():
    A, B = _rand_case("os", 64, 64, 64, 1, seed=40, dtype=torch.bfloat16)
    A[0][3, 5] = np.nan
    B[0][7, 9] = np.inf
    got = host(ms.gemm_os([dev(A[0], torch.bfloat16)], [dev(B[0], torch.bfloat16)], out_dtype=torch.float32))
    assert np.isnan(got[3]).all()                    # a NaN in row 3 of A poisons row 3 of C
    col = np.delete(got[:, 9], 3)
    assert np.isinf(col).all() or np.isnan(col).any() is False and np.isinf(col).all()
    clean = np.delete(np.delete(got, 3, axis=0), 9, axis=1)
    assert np.isfinite(clean).all()


# ------------------------------------------------------------------ fused output-stationary epilogue
@pytest.mark.parametrize("variant", [0, 1, 3, 4, 7, 8, 9, 10, 11, 12, 13, 14])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
def test_fused_epilogue_gelu_residual_moments(variant, out_dtype):
    """ms_gemm_os_fused: Y = gelu(sum_k A_k B_k) + residual, plus the row sums / sums of squares of Y
    (the local layer-norm moments of reference ShardedLayers.py:125-126) against the float64 oracle."""
    _lib.check(_lib.load().ms_set_variant(variant))
    m, n, k, S = 520, 776, 136, 3
    A, B = _rand_case("os", m, n, k, S, seed=50 + variant, dtype=torch.bfloat16)
    rng = np.random.default_rng(99)
    R = rng.standard_normal((m, n)).astype(np.float32)
    R = orc.bf16_round(R) if out_dtype == torch.bfloat16 else R
    a = [dev(x, torch.bfloat16) for x in A]; b = [dev(x, torch.bfloat16) for x in B]
    s1 = torch.zeros(m, device="cuda"); s2 = torch.zeros(m, device="cuda")
    got = ms.gemm_os(a, b, out_dtype=out_dtype, activation="gelu", residual=dev(R, out_dtype), row_moments=(s1, s2))
    want, w1, w2 = orc.oracle_os_fused(A, B, "gelu", R)
    tol = TOL_BF16 if out_dtype == torch.bfloat16 else 1e-5
    assert orc.rel_frobenius(host(got), want) <= tol
    assert orc.rel_frobenius(host(s1), w1) <= 1e-4          # moments come from the fp32 values before rounding
    assert orc.rel_frobenius(host(s2), w2) <= 1e-4
    # each part alone
    plain = ms.gemm_os(a, b, out_dtype=torch.float32)
    only_act = ms.gemm_os(a, b, out_dtype=torch.float32, activation="gelu")
    assert orc.rel_frobenius(host(only_act), orc.gelu_tanh(host(plain))) <= 1e-6
    only_res = ms.gemm_os(a, b, out_dtype=torch.float32, residual=dev(R.astype(np.float32), torch.float32))
    assert torch.equal(only_res, plain + dev(R.astype(np.float32), torch.float32))
    s1b = torch.zeros(m, device="cuda")
    again = ms.gemm_os(a, b, out_dtype=torch.float32, row_moments=(s1b, None))
    assert torch.equal(again, plain)
    assert orc.rel_frobenius(host(s1b), host(plain).sum(1)) <= 1e-4


@pytest.mark.parametrize("variant", [0, 3, 7, 8, 10, 11, 12, 13, 14])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_one_call_per_slice_accumulating_in_place_through_the_residual(variant, out_dtype):
    """The output-stationary product slice by slice, as a mesh would issue it when each slice's call waits for that
    slice's all-gather: call s adds A_s B_s to C in place (residual = out).  With a bf16 C that is the reference's own
    arithmetic (the running sum is carried in the input dtype, TensorParallel.py:167); with an fp32 C it equals the
    one-call product up to the order of the fp32 additions."""
    _lib.check(_lib.load().ms_set_variant(variant))
    m, n, k, S = 520, 776, 136, 4
    A, B = _rand_case("os", m, n, k, S, seed=70 + variant, dtype=torch.bfloat16)
    a = [dev(x, torch.bfloat16) for x in A]; b = [dev(x, torch.bfloat16) for x in B]
    C = ms.gemm_os(a[:1], b[:1], out_dtype=out_dtype)
    for s in range(1, S):
        ms.gemm_os(a[s:s + 1], b[s:s + 1], out=C, residual=C)
    if out_dtype == torch.float32:
        assert orc.rel_frobenius(host(C), orc.oracle_os_block(A, B)) <= 1e-5
    else:
        # the oracle's statement of the reference's slice loop: every partial product and every sum rounded to bf16 ...
        want = orc.bf16_round((A[0].astype(np.float64) @ B[0].astype(np.float64)).astype(np.float32))
        for s in range(1, S):
            # ... except that here the product of slice s is added in fp32 before the one rounding of the sum
            want = orc.bf16_round((want.astype(np.float64) + A[s].astype(np.float64) @ B[s].astype(np.float64)).astype(np.float32))
        assert orc.rel_frobenius(host(C), want.astype(np.float64)) <= 2e-3       # a bf16 tie now and then falls the other way
        assert orc.rel_frobenius(host(C), orc.oracle_os_block(A, B)) <= TOL_BF16


def test_operand_span_of_2gib_is_rejected():
    """32-bit byte offsets inside the kernels: an operand slice of 2 GiB or more is refused, not mis-addressed."""
    lib = _lib.load()
    a = torch.zeros((8, 8), dtype=torch.bfloat16, device="cuda")
    pa, _ka = _lib.ptr_array([a.data_ptr()]); pc = ctypes.c_void_p(a.data_ptr())
    big_ld = 1 << 20                       # 1024 rows x 2^20 elements x 2 bytes = 2 GiB
    rc = lib.ms_gemm_os(pa, pa, 1, 1024, 8, 8, big_ld, 8, pc, 8, _lib.MS_DTYPE_BF16, _lib.MS_DTYPE_BF16, None)
    assert rc == _lib.MS_ERR_UNSUPPORTED and b"2 GiB" in lib.ms_last_error()


def test_fused_epilogue_rejections():
    a = torch.zeros((64, 64), dtype=torch.float32, device="cuda")
    with pytest.raises(_lib.MeshSliceError):                 # fp32 operands: no fused kernel
        ms.gemm_os([a], [a], activation="gelu")
    h = torch.zeros((64, 64), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError):
        ms.gemm_os([h], [h], activation="relu")
    with pytest.raises(ValueError):
        ms.gemm_os([h], [h], residual=torch.zeros((64, 32), dtype=torch.bfloat16, device="cuda"))
    with pytest.raises(ValueError):
        ms.gemm_os([h], [h], row_moments=(torch.zeros(63, device="cuda"), None))


@pytest.mark.parametrize("shape,wps", [("32x32x16", 1), ("32x32x16", 2), ("16x16x32", 1), ("16x16x32", 2)])
def test_mfma_stream_probe_reports_a_plausible_rate(shape, wps):
    """The measurement aid runs for either instruction shape at one and two waves per SIMD, stays under the
    data-sheet peak and above a tenth of it."""
    from meshslice_amd.local_gemm import mfma_stream_rate
    rate = mfma_stream_rate(iters=500, warmup=2, reps=5, shape=shape, waves_per_simd=wps)
    assert 0.25e15 < rate < 2.5166e15 * 1.02


def test_mfma_stream_probe_rejects_bad_arguments():
    from meshslice_amd.local_gemm import mfma_stream_rate
    L = _lib.load()
    ms_out, fl = ctypes.c_float(), ctypes.c_double()
    x = torch.zeros(8192, dtype=torch.bfloat16, device="cuda"); sink = torch.zeros(512 * 256, device="cuda")
    xp, sp = ctypes.c_void_p(x.data_ptr()), ctypes.c_void_p(sink.data_ptr())
    out = (ctypes.byref(ms_out), ctypes.byref(fl), None)
    assert L.ms_probe_mfma_stream(None, sp, 10, 0, 1, *out) == _lib.MS_ERR_ARG
    assert L.ms_probe_mfma_stream(xp, sp, 0, 0, 1, *out) == _lib.MS_ERR_ARG
    assert L.ms_probe_mfma_stream_ex(xp, sp, 2, 1, 10, 0, 1, *out) == _lib.MS_ERR_ARG        # unknown shape
    assert L.ms_probe_mfma_stream_ex(xp, sp, 0, 3, 10, 0, 1, *out) == _lib.MS_ERR_ARG        # three waves per SIMD
    with pytest.raises(ValueError):
        mfma_stream_rate(torch.zeros(16, dtype=torch.bfloat16, device="cuda"))
    with pytest.raises(ValueError):
        mfma_stream_rate(shape="4x4x4")


def test_time_call_checks_its_arguments_like_the_gemm_calls():
    """The timing helper validates shapes, dtypes and devices before any pointer reaches the library, accepts bf16
    chunks, and returns one positive time per repetition."""
    A = torch.zeros((64, 32), dtype=torch.bfloat16, device="cuda"); B = torch.zeros((32, 48), dtype=torch.bfloat16, device="cuda")
    W = torch.zeros((48, 32), dtype=torch.bfloat16, device="cuda"); Xt = torch.zeros((32, 64), dtype=torch.bfloat16, device="cuda")
    C = torch.empty((64, 48), dtype=torch.bfloat16, device="cuda")
    t = ms.time_call("os", ([A], [B]), C, warmup=1, reps=3)
    assert len(t) == 3 and all(x > 0 for x in t)
    for dt in (torch.float32, torch.bfloat16):
        Y = [torch.empty((64, 48), dtype=dt, device="cuda")]
        assert len(ms.time_call("ls", (A, [W]), Y, warmup=0, reps=2)) == 2
        assert len(ms.time_call("rs", ([Xt], B), Y, warmup=0, reps=2)) == 2
    small = [torch.empty((64, 40), dtype=torch.float32, device="cuda")]
    with pytest.raises(ValueError):
        ms.time_call("ls", (A, [W]), small)                      # undersized chunk
    with pytest.raises(ValueError):
        ms.time_call("rs", ([Xt], B), small)
    with pytest.raises(ValueError):
        ms.time_call("os", ([A], [B]), torch.empty((64, 40), dtype=torch.bfloat16, device="cuda"))
    with pytest.raises(ValueError):
        ms.time_call("os", ([A], [B.t()]), C)                    # not row-major
    with pytest.raises(ValueError):
        ms.time_call("ls", (A, [W]), [torch.empty((64, 48), dtype=torch.float16, device="cuda")])
    with pytest.raises(ValueError):
        ms.time_call("os", ([A], [B]), None)
    with pytest.raises(ValueError):
        ms.time_call("xs", ([A], [B]), C)
    with pytest.raises(ValueError):
        ms.time_call("os", ([A], [B]), C, reps=0)
    with pytest.raises(_lib.MeshSliceError):
        ms.time_call("os", ([A.cpu()], [B.cpu()]), C)
