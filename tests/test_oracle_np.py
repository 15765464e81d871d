"""Pins the numpy oracle: exact rational closed forms on the reference's own arange fixtures
(MeshFlowCPU.ipynb cells 2-4), brute-force index enumeration, partition invariants, and the
identity sliced == unsliced == dense that the reference itself asserts (ipynb:80,102,111,130-132;
TensorParallel.py:447,452,457)."""
import itertools
from fractions import Fraction

import numpy as np
import pytest
import torch

from oracle import meshslice_oracle as orc


# ---------------------------------------------------------------- slice selector
def _sel_bruteforce(L, S, B, k):
    """Enumerate the (L/(S*B), S, B) view element by element, keep axis-1 index k."""
    out = []
    g = 0
    for q in range(L // (S * B)):
        for s in range(S):
            for b in range(B):
                if s == k:
                    out.append(g)
                g += 1
    return out


@pytest.mark.parametrize("L,S,B", [(16, 2, 2), (64, 4, 8), (64, 8, 8), (96, 3, 8), (48, 1, 8), (120, 5, 4)])
def test_sel_matches_reshape_enumeration(L, S, B):
    seen = []
    for k in range(S):
        s = orc.sel(L, S, B, k)
        assert list(s) == _sel_bruteforce(L, S, B, k)
        assert len(s) == L // S
        seen.extend(s)
    assert sorted(seen) == list(range(L))          # slices partition the range


def test_sel_rejects_bad_shapes():
    with pytest.raises(ValueError):
        orc.sel(60, 4, 8, 0)
    with pytest.raises(ValueError):
        orc.sel(64, 4, 8, 4)


# ---------------------------------------------------------------- layout steps

@pytest.mark.parametrize("r,c,S,B", [(16, 32, 2, 2), (24, 64, 4, 8), (48, 96, 3, 8), (40, 120, 5, 4), (8, 16, 1, 8)])
def test_pack_slices_matches_the_index_rule_and_brute_force(r, c, S, B):
    """The literal reshape + dynamic_slice equals plain indexing with the closed-form rule, and with the
    loop enumeration of the (.., S, B) view; the slices partition the shard."""
    rng = np.random.default_rng(r * c + S)
    blk = rng.integers(0, 1 << 30, size=(r, c)).astype(np.int64)
    if c % (S * B) == 0:
        sl = orc.pack_slices(blk, S, B, 1)
        for k in range(S):
            assert np.array_equal(sl[k], blk[:, orc.sel(c, S, B, k)])
            assert np.array_equal(sl[k], blk[:, _sel_bruteforce(c, S, B, k)])
        assert sorted(np.concatenate([x.ravel() for x in sl]).tolist()) == sorted(blk.ravel().tolist())
    if r % (S * B) == 0:
        sl = orc.pack_slices(blk, S, B, 0)
        for k in range(S):
            assert np.array_equal(sl[k], blk[orc.sel(r, S, B, k), :])
            assert np.array_equal(sl[k], blk[_sel_bruteforce(r, S, B, k), :])


@pytest.mark.parametrize("axis", [0, 1])
@pytest.mark.parametrize("S,B,parts", [(2, 2, 2), (4, 8, 2), (3, 8, 1), (8, 8, 4)])
def test_unpack_chunks_inverts_pack_and_matches_assembly(S, B, parts, axis):
    """unpack(pack(x)) == x (one peer, one window); with several peers and windows it equals the closed-form
    assembly (assemble_ls / assemble_rs), which the literal whole-mesh emulation pins elsewhere."""
    rng = np.random.default_rng(S * 100 + B * 10 + parts + axis)
    L = S * B * parts * 3
    shape = (24, L) if axis == 1 else (L, 24)
    x = rng.standard_normal(shape).astype(np.float32)
    assert np.array_equal(orc.unpack_chunks([orc.pack_slices(x, S, B, axis)], B, axis), x)
    cshape = (24, L // S) if axis == 1 else (L // S, 24)
    peers = [[rng.standard_normal(cshape).astype(np.float32) for _ in range(S)] for _ in range(parts)]
    for w in range(parts):
        got = orc.unpack_chunks(peers, B, axis, window=w, parts=parts)
        want = orc.assemble_ls(peers, 1, parts, w, S, B) if axis == 1 else orc.assemble_rs(peers, parts, 1, w, S, B)
        assert np.allclose(got, want, rtol=1e-6, atol=1e-6)
        if parts <= 2:  # a two-term fp32 sum has one rounding whatever the order
            assert np.array_equal(got, want)
        got16 = orc.unpack_chunks(peers, B, axis, window=w, parts=parts, out_dtype="bf16")
        assert np.array_equal(got16, orc.bf16_round(got))


# ---------------------------------------------------------------- ring baselines

RING_MESHES = [("wang", 2, 4), ("wang", 4, 2), ("wang", 2, 2), ("wang", 1, 3), ("cannon", 2, 2), ("cannon", 4, 4), ("cannon", 3, 3)]


@pytest.mark.parametrize("algorithm,R,C", RING_MESHES)
@pytest.mark.parametrize("dataflow", ["os", "ls", "rs"])
def test_literal_ring_baselines_equal_the_dense_product(algorithm, R, C, dataflow):
    """Integer-valued operands: the statement-by-statement emulation of Wang_* / Cannon_* equals X@W, X@W^T,
    X^T@W exactly (this is what fixes the reading of the device position and of every shift direction: any
    other pairing of half-blocks misses or doubles a term)."""
    rng = np.random.default_rng(R * 10 + C)
    L = R * C * 2 * 3
    shapes = {"os": ((L, L), (L, 2 * L)), "ls": ((L, L), (2 * L, L)), "rs": ((L, 2 * L), (L, L))}[dataflow]
    X = rng.integers(-3, 4, shapes[0]).astype(np.float64)
    W = rng.integers(-3, 4, shapes[1]).astype(np.float64)
    assert np.array_equal(orc.literal_ring(algorithm, dataflow, X, W, R, C), orc.dense(dataflow, X, W))


@pytest.mark.parametrize("algorithm,R,C", RING_MESHES)
def test_ring_order_matches_labels_carried_round_the_ring(algorithm, R, C):
    """ring_order() against labels moved with the same ppermute primitive and directions the literal
    emulation uses: which (block, half) a device holds, or works on, at every step."""
    lab = lambda h: [[(j, h) for j in range(C)] for _ in range(R)]
    for dataflow in ("os", "ls", "rs"):
        seen = [[[] for _ in range(C)] for _ in range(R)]
        if algorithm == "wang":
            lo, hi = lab(0), lab(1)
            if dataflow == "ls":   # partial outputs travel: the device holding block b's partial adds its term
                lo = [[((j - 1) % C, 0) for j in range(C)] for _ in range(R)]
                hi = [[((j + 1) % C, 1) for j in range(C)] for _ in range(R)]
            for t in range(C):
                for i in range(R):
                    for j in range(C):
                        seen[i][j] += [lo[i][j], hi[i][j]]
                if dataflow == "ls":   # the label a device receives is the block it must NOT redo: it works on the one before
                    lo = [[((b - 1) % C, h) for b, h in row] for row in lo]
                    hi = [[((b + 1) % C, h) for b, h in row] for row in hi]
                else:
                    lo, hi = orc._ppermute(lo, R, C, "col", +1), orc._ppermute(hi, R, C, "col", -1)
        else:
            lo = [[((i + j) % C, 0) for j in range(C)] for i in range(R)]
            hi = [[((i + j) % C, 1) for j in range(C)] for i in range(R)]
            for t in range(C):
                for i in range(R):
                    for j in range(C):
                        seen[i][j] += [lo[i][j], hi[i][j]]
                axis = "col" if dataflow != "ls" else "row"   # the operand halves that move: X along col (OS, RS), W along row (LS)
                lo, hi = orc._ppermute(lo, R, C, axis, -1), orc._ppermute(hi, R, C, axis, +1)
        for i in range(R):
            for j in range(C):
                assert seen[i][j] == orc.ring_order(algorithm, dataflow, R, C, i, j), (dataflow, i, j)


# ---------------------------------------------------------------- bf16 rounding
def test_bf16_round_matches_torch_and_special_values():
    rng = np.random.default_rng(1)
    x = np.concatenate([
        rng.standard_normal(20000).astype(np.float32),
        (rng.standard_normal(2000) * 1e-40).astype(np.float32),          # subnormals
        np.array([0.0, -0.0, np.inf, -np.inf, 1.0, 1.00390625, 1.01171875,  # ties: 1+2^-8, 1+3*2^-8
                  3.3895314e38, 65504.0, 1e-45], np.float32),
    ])
    want = torch.from_numpy(x).to(torch.bfloat16).to(torch.float32).numpy()
    got = orc.bf16_round(x)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert orc.bf16_round(np.float32([1.00390625]))[0] == 1.0            # tie -> even (down)
    assert orc.bf16_round(np.float32([1.01171875]))[0] == 1.015625       # tie -> even (up)
    assert np.isnan(orc.bf16_round(np.float32([np.nan]))[0])
    assert np.array_equal(orc.bits_to_f32(orc.bf16_bits(x)).view(np.uint32), got.view(np.uint32))


# ---------------------------------------------------------------- notebook fixture, exact
def _notebook_exact():
    """Exact integer numerators of Y, dX, dW for the notebook inputs (all operands are
    integers over a power of two, so every product and sum is exact)."""
    Bt, I, O = 512, 256, 1024
    r = np.arange(Bt, dtype=object)[:, None]
    c = np.arange(O, dtype=object)[None, :]
    s1 = I * (I - 1) // 2
    s2 = (I - 1) * I * (2 * I - 1) // 6
    # Y[r,c] = sum_k (r*I+k)*(k*O+c) / ((B*I)*(I*O))
    Ynum = r * I * O * s1 + r * I * c * I + O * s2 + c * s1
    Yden = (Bt * I) * (I * O)
    # dX[r,i] = sum_o W[i,o] / (B*O) = sum_o (i*O+o) / ((I*O)*(B*O))
    i = np.arange(I, dtype=object)[None, :]
    dXnum = np.repeat(i * O * O + O * (O - 1) // 2, Bt, axis=0)
    dXden = (I * O) * (Bt * O)
    # dW[i,o] = sum_b X[b,i] / (B*O) = sum_b (b*I+i) / ((B*I)*(B*O))
    ii = np.arange(I, dtype=object)[:, None]
    dWnum = np.repeat(I * Bt * (Bt - 1) // 2 + Bt * ii, O, axis=1)
    dWden = (Bt * I) * (Bt * O)
    f = lambda num, den: (num.astype(np.float64) / float(den))
    return f(Ynum, Yden), f(dXnum, dXden), f(dWnum, dWden)


@pytest.fixture(scope="module")
def nb():
    d = orc.notebook_inputs(np.float64)
    # arange / 2^k is exact in fp32, so the float64 copies carry the reference's fp32 values
    assert np.array_equal(d["X"], orc.notebook_inputs(np.float32)["X"].astype(np.float64))
    return d


def test_notebook_dense_equals_exact_closed_form(nb):
    Y, dX, dW = _notebook_exact()
    assert np.array_equal(orc.dense("os", nb["X"], nb["W"]), Y)
    assert np.array_equal(orc.dense("ls", nb["dY"], nb["W"]), dX)
    assert np.array_equal(orc.dense("rs", nb["X"], nb["dY"]), dW)
    # a spot value by exact rational arithmetic, independent of the polynomial above
    r, c = 311, 777
    v = sum(Fraction((r * 256 + k) * (k * 1024 + c), (512 * 256) * (256 * 1024)) for k in range(256))
    assert Y[r, c] == float(v)


@pytest.mark.parametrize("dataflow", ["os", "ls", "rs"])
def test_notebook_collective_and_meshflow_equal_exact(nb, dataflow):
    Y, dX, dW = _notebook_exact()
    R, C = nb["mesh"]
    X, W, want = {"os": (nb["X"], nb["W"], Y), "ls": (nb["dY"], nb["W"], dX), "rs": (nb["X"], nb["dY"], dW)}[dataflow]
    got_c = orc.literal_collective(dataflow, X, W, R, C)
    got_m = orc.literal_meshflow(dataflow, X, W, R, C, nb["K"], nb["blocksize"])
    assert np.array_equal(got_c, want)
    assert np.array_equal(got_m, want)            # exact: every partial sum is an integer / 2^k


@pytest.mark.parametrize("dataflow", ["os", "ls", "rs"])
def test_notebook_device_blocks_and_assembly(nb, dataflow):
    Y, dX, dW = _notebook_exact()
    R, C = nb["mesh"]; S = nb["K"]; B = nb["blocksize"]
    X, W, want = {"os": (nb["X"], nb["W"], Y), "ls": (nb["dY"], nb["W"], dX), "rs": (nb["X"], nb["dY"], dW)}[dataflow]
    orc.check_divisibility(dataflow, X.shape, W.shape, R, C, S, B)
    if dataflow == "os":
        for i, j in itertools.product(range(R), range(C)):
            A, Bs = orc.device_operands_os(X, W, R, C, i, j, S, B)
            assert A[0].shape == (512 // R, 256 // S) and Bs[0].shape == (256 // S, 1024 // C)
            assert np.array_equal(orc.oracle_os_block(A, Bs), orc.shard(want, R, C, i, j))
    elif dataflow == "ls":
        for i in range(R):
            chunks = []
            for j in range(C):
                A, Ws = orc.device_operands_ls(X, W, R, C, i, j, S, B)
                chunks.append(orc.oracle_ls_chunks(A, Ws))
            for j in range(C):
                assert np.array_equal(orc.assemble_ls(chunks, R, C, j, S, B), orc.shard(want, R, C, i, j))
    else:
        for j in range(C):
            chunks = []
            for i in range(R):
                Xs, Wl = orc.device_operands_rs(X, W, R, C, i, j, S, B)
                chunks.append(orc.oracle_rs_chunks(Xs, Wl))
            for i in range(R):
                assert np.array_equal(orc.assemble_rs(chunks, R, C, i, S, B), orc.shard(want, R, C, i, j))


# ---------------------------------------------------------------- integer-valued random cases, exact
def _int_mats(rng, shape_x, shape_w):
    return (rng.integers(-4, 5, size=shape_x).astype(np.float64),
            rng.integers(-4, 5, size=shape_w).astype(np.float64))


CASES = [  # (R, C, S, B, dims)  dims = (a, b, c): os X[a,b] W[b,c]; ls X[a,b] W[c,b]; rs X[a,b] W[a,c]
    (2, 2, 2, 2, (16, 16, 16)),
    (2, 2, 1, 2, (8, 8, 8)),
    (4, 2, 4, 8, (64, 128, 128)),
    (2, 4, 8, 8, (32, 256, 256)),
    (1, 1, 4, 8, (8, 32, 64)),
    (2, 2, 3, 4, (24, 48, 48)),
]


@pytest.mark.parametrize("R,C,S,B,dims", CASES)
@pytest.mark.parametrize("dataflow", ["os", "ls", "rs"])
def test_literal_meshflow_equals_dense_and_closed_form(R, C, S, B, dims, dataflow):
    rng = np.random.default_rng(hash((R, C, S, B, dataflow)) % (1 << 31))
    a, b, c = dims
    if dataflow == "os":
        X, W = _int_mats(rng, (a, b), (b, c))
    elif dataflow == "ls":
        X, W = _int_mats(rng, (a, b), (c, b))
    else:
        X, W = _int_mats(rng, (b, a * 4), (b, c))      # N = 4a keeps N % (S*B*R) == 0
    try:
        orc.check_divisibility(dataflow, X.shape, W.shape, R, C, S, B)
    except ValueError:
        pytest.skip("shape not admissible for this mesh/slice count")
    want = orc.dense(dataflow, X, W)
    assert np.array_equal(orc.literal_collective(dataflow, X, W, R, C), want)
    if not (dataflow == "os" and S == 1):
        assert np.array_equal(orc.literal_meshflow(dataflow, X, W, R, C, S, B), want)
    # closed-form device operands + block oracle + mesh completion reproduce the same thing
    if dataflow == "os":
        for i, j in itertools.product(range(R), range(C)):
            assert np.array_equal(orc.oracle_os_block(*orc.device_operands_os(X, W, R, C, i, j, S, B)),
                                  orc.shard(want, R, C, i, j))
    elif dataflow == "ls":
        for i in range(R):
            ch = [orc.oracle_ls_chunks(*orc.device_operands_ls(X, W, R, C, i, j, S, B)) for j in range(C)]
            for j in range(C):
                assert np.array_equal(orc.assemble_ls(ch, R, C, j, S, B), orc.shard(want, R, C, i, j))
    else:
        for j in range(C):
            ch = [orc.oracle_rs_chunks(*orc.device_operands_rs(X, W, R, C, i, j, S, B)) for i in range(R)]
            for i in range(R):
                assert np.array_equal(orc.assemble_rs(ch, R, C, i, S, B), orc.shard(want, R, C, i, j))


def test_meshflow_os_k1_quirk_is_a_double_count():
    """TensorParallel.py:163 asks for slice 1 of a 1-slice view; dynamic_slice clamps it to slice 0
    and :172 adds it again, so the reference's sliced OS body returns 2*X@W for K=1.  The build
    never routes S=1 through that body (S=1 is the 'collective' contraction)."""
    rng = np.random.default_rng(5)
    X, W = _int_mats(rng, (8, 16), (16, 8))
    got = orc.literal_meshflow_os(X, W, 2, 2, 1, 2)
    assert np.array_equal(got, 2.0 * (X @ W))
    assert np.array_equal(orc.literal_meshflow_os(X, W, 2, 2, 2, 2), X @ W)


def test_selfcheck_fixture_chain_matches_polynomial():
    """TensorParallel.py:433-457 chain Yo=OS(X,W), LS(Yo,W), RS(X,Yo) on the 4x4 mesh; checked on
    one device block each against the dense product and a polynomial closed form of X@W."""
    d = orc.selfcheck_inputs(np.float32)
    X, W = d["X"].astype(np.float64), d["W"].astype(np.float64)
    R, C = d["mesh"]; S, B = d["K"], d["blocksize"]
    i, j = 2, 1
    A, Bs = orc.device_operands_os(X, W, R, C, i, j, S, B)
    blk = orc.oracle_os_block(A, Bs)
    n, dd = X.shape[0], X.shape[1]
    o = W.shape[1]
    r = np.arange(i * n // R, (i + 1) * n // R, dtype=np.float64)[:, None]
    c = np.arange(j * o // C, (j + 1) * o // C, dtype=np.float64)[None, :]
    s1 = dd * (dd - 1) / 2
    s2 = (dd - 1) * dd * (2 * dd - 1) / 6
    poly = (r * dd * o * s1 + r * dd * c * dd + o * s2 + c * s1) / (float(n * dd) * float(4 * dd * dd))
    assert orc.rel_frobenius(blk, poly) < 1e-6     # fp32 rounding of arange/denominator only
    assert orc.rel_frobenius(blk, (X @ W)[orc.block_range(n, R, i), orc.block_range(o, C, j)]) < 1e-13


# ---------------------------------------------------------------- backward wiring
@pytest.mark.parametrize("dataflow", ["os", "ls", "rs"])
def test_vjp_permutation_matches_autograd(dataflow):
    """ShardedLayers.py:41-81: the (fwd, dx, dw) triples are (OS,LS,RS), (LS,OS,RS), (RS,LS,OS)."""
    g = torch.Generator().manual_seed(3)
    x = torch.randn(12, 20, dtype=torch.float64, generator=g, requires_grad=True)
    if dataflow == "os":      # y = x @ w, w [in,out]
        w = torch.randn(20, 28, dtype=torch.float64, generator=g, requires_grad=True)
        y = x @ w
    elif dataflow == "ls":    # y = x @ w^T, w [out,in]
        w = torch.randn(28, 20, dtype=torch.float64, generator=g, requires_grad=True)
        y = x @ w.t()
    else:                     # y = x^T @ w, x [in, tokens]
        w = torch.randn(12, 28, dtype=torch.float64, generator=g, requires_grad=True)
        y = x.t() @ w
    dy = torch.randn(*y.shape, dtype=torch.float64, generator=g)
    y.backward(dy)
    xn, wn, dyn = x.detach().numpy(), w.detach().numpy(), dy.numpy()
    if dataflow == "os":
        dx, dw = orc.dense("ls", dyn, wn), orc.dense("rs", xn, dyn)
    elif dataflow == "ls":
        dx, dw = orc.dense("os", dyn, wn), orc.dense("rs", dyn, xn)
    else:
        dx, dw = orc.dense("ls", wn, dyn), orc.dense("os", xn, dyn)
    assert np.allclose(dx, x.grad.numpy(), rtol=1e-12, atol=1e-12)
    assert np.allclose(dw, w.grad.numpy(), rtol=1e-12, atol=1e-12)


# ---------------------------------------------------------------- fused epilogue oracle
def test_gelu_tanh_matches_torch_and_identities():
    x = np.concatenate([np.linspace(-12, 12, 4001), [0.0, 1e-8, -1e-8, 30.0, -30.0]])
    want = torch.nn.functional.gelu(torch.from_numpy(x), approximate="tanh").numpy()
    got = orc.gelu_tanh(x)
    assert np.allclose(got, want, rtol=1e-13, atol=1e-15)
    assert orc.gelu_tanh(0.0) == 0.0
    assert np.allclose(orc.gelu_tanh(x) - orc.gelu_tanh(-x), x, rtol=1e-13, atol=1e-15)   # x*Phi(x) - (-x)*Phi(-x) = x
    assert orc.gelu_tanh(30.0) == 30.0 and orc.gelu_tanh(-30.0) == 0.0
    assert orc.gelu_tanh(1.0) == pytest.approx(0.8411919906082768, rel=1e-14)             # 0.5*(1+tanh(sqrt(2/pi)*1.044715))


def test_oracle_os_fused_composes_the_parts():
    rng = np.random.default_rng(8)
    A = [rng.integers(-3, 4, (6, 8)).astype(np.float64) for _ in range(2)]
    B = [rng.integers(-3, 4, (8, 5)).astype(np.float64) * 0.25 for _ in range(2)]
    R = rng.integers(-3, 4, (6, 5)).astype(np.float64)
    y, s1, s2 = orc.oracle_os_fused(A, B, "gelu", R)
    base = A[0] @ B[0] + A[1] @ B[1]
    assert np.array_equal(y, orc.gelu_tanh(base) + R)
    assert np.allclose(s1, y.sum(1)) and np.allclose(s2, (y ** 2).sum(1))
    y0, _, _ = orc.oracle_os_fused(A, B)
    assert np.array_equal(y0, base)
    with pytest.raises(ValueError):
        orc.oracle_os_fused(A, B, "relu")
