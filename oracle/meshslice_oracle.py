"""CPU oracle for the MeshSlice per-device sliced GEMM (TEST INFRASTRUCTURE ONLY).

This module restates, in numpy, the algorithm of the reference's 2-D tensor-parallel
GEMM bodies so that the HIP path can be checked against it.  It is a checker: only the
test-suite, the smoke test and the benchmark's CPU-baseline leg may import it.  Nothing
in the shipped package imports it, and the shipped package has no CPU fallback.

Two independent restatements live here:

* the *literal* whole-mesh emulation (``literal_*``): every mesh device's body is executed
  step by step with the same reshape / dynamic-slice / all-gather / psum-scatter sequence
  the reference uses (TensorParallel.py:19-32 for the unsliced "collective" bodies and
  :153-214 for the sliced "meshflow" bodies);
* the *closed-form* device-block oracle (``sel``, ``device_operands_*``, ``oracle_*``):
  slice k of an index range is ``{g : (g // B) % S == k}`` and the device block is a plain
  float64 matrix product restricted to that device's rows/columns.

The tests pin one against the other, both against exact rational arithmetic on the
reference's own ``arange`` fixtures (MeshFlowCPU.ipynb cells 2-4, TensorParallel.py:425-457),
and against the C restatement in ``ms_oracle.c``.

``pack_slices`` / ``unpack_chunks`` restate the layout statements either side of the contraction on their own.

Parity status of every function: pinned (see tests/test_oracle_*.py).  What is NOT pinned,
because only an import of JAX could pin it and JAX is not installed: the bit-exact rounding
order of XLA:CPU's dot_general and the sample stream of ``jax.random.normal`` used by
``createMultihostMatrix`` (TensorParallel.py:419-423).  Parity is therefore stated to a
tolerance (rel-Frobenius 1e-5 fp32, 1e-2 bf16), never bitwise.
"""
from __future__ import annotations

import numpy as np

# --------------------------------------------------------------------------------------
# dtype helpers
# --------------------------------------------------------------------------------------

def bf16_round(x: np.ndarray) -> np.ndarray:
    """Round fp32 values to the nearest bfloat16 (ties to even) and return them as fp32.

    bfloat16 keeps the top 16 bits of the IEEE-754 binary32 pattern; the reference's bf16
    operands (createMultihostMatrix dtype, TensorParallel.py:419) are exactly such values.
    """
    a = np.ascontiguousarray(x, dtype=np.float32)
    u = a.view(np.uint32).astype(np.uint64)
    lsb = (u >> 16) & 1
    r = ((u + 0x7FFF + lsb) >> 16) << 16
    out = r.astype(np.uint32).view(np.float32).reshape(a.shape)
    nan = np.isnan(a)
    if nan.any():
        out = out.copy()
        out[nan] = np.nan
    return out


def bf16_bits(x: np.ndarray) -> np.ndarray:
    """uint16 bit patterns of ``bf16_round(x)`` (what is uploaded to the GPU)."""
    return (bf16_round(x).view(np.uint32) >> 16).astype(np.uint16)


def bits_to_f32(b: np.ndarray) -> np.ndarray:
    """Inverse of :func:`bf16_bits`."""
    return (b.astype(np.uint32) << 16).view(np.float32)


def rel_frobenius(got: np.ndarray, ref: np.ndarray) -> float:
    """``||got - ref||_F / ||ref||_F`` in float64 (the parity metric of this build)."""
    g = np.asarray(got, dtype=np.float64)
    r = np.asarray(ref, dtype=np.float64)
    den = np.linalg.norm(r)
    return float(np.linalg.norm(g - r) / (den if den > 0 else 1.0))


def allclose(a, b) -> bool:
    """The reference's own acceptance test (TensorParallel.py:16-17): atol=rtol=1e-2."""
    return bool(np.allclose(np.asarray(a, np.float64), np.asarray(b, np.float64), atol=1e-2, rtol=1e-2))


# --------------------------------------------------------------------------------------
# index rules (closed form)
# --------------------------------------------------------------------------------------

def sel(L: int, S: int, B: int, k: int) -> np.ndarray:
    """Indices of slice ``k`` of a length-``L`` range: ``{g : (g // B) % S == k}``, ascending.

    Follows the ``(..., L/(S*B), S, B)`` view + ``dynamic_slice_in_dim(.., k, 1, axis_of_S)``
    at TensorParallel.py:155-158, :177-178, :198-199.  Requires ``L % (S*B) == 0``.
    """
    if S < 1 or B < 1 or L % (S * B) != 0:
        raise ValueError(f"length {L} is not a multiple of S*B = {S}*{B}")
    if not 0 <= k < S:
        raise ValueError(f"slice index {k} outside [0,{S})")
    g = np.arange(L)
    return g[(g // B) % S == k]


def block_range(L: int, parts: int, idx: int) -> slice:
    """Rows/cols of shard ``idx`` of ``parts`` along a length-``L`` axis (P(row,col) sharding,
    TensorParallel.py:351,364-365)."""
    if L % parts != 0:
        raise ValueError(f"length {L} is not divisible by mesh axis size {parts}")
    n = L // parts
    return slice(idx * n, (idx + 1) * n)


def shard(G: np.ndarray, R: int, C: int, i: int, j: int) -> np.ndarray:
    """Device (i,j)'s block of a global matrix sharded P(row,col)."""
    return G[block_range(G.shape[0], R, i), block_range(G.shape[1], C, j)]


def check_divisibility(dataflow: str, Xshape, Wshape, R: int, C: int, S: int, B: int) -> None:
    """Shape rules implied by the reference's reshapes (TensorParallel.py:155-156,177-179,198-200)."""
    def need(v, d, what):
        if v % d != 0:
            raise ValueError(f"{dataflow}: {what} = {v} is not a multiple of {d}")
    if dataflow == "os":
        (M, Kx), (Kw, N) = Xshape, Wshape
        if Kx != Kw:
            raise ValueError("os: contraction sizes differ")
        need(M, R, "rows of X"); need(N, C, "cols of W")
        need(Kx, C * S * B, "cols of X"); need(Kw, R * S * B, "rows of W")
    elif dataflow == "ls":
        (M, I), (O, Iw) = Xshape, Wshape
        if I != Iw:
            raise ValueError("ls: contraction sizes differ")
        need(M, R, "rows of X"); need(I, C, "cols of X")
        need(O, R * S * B, "rows of W"); need(O, S * B * C, "rows of W (scatter)")
    elif dataflow == "rs":
        (I, N), (Iw, O) = Xshape, Wshape
        if I != Iw:
            raise ValueError("rs: contraction sizes differ")
        need(I, R, "rows of X"); need(O, C, "cols of W")
        need(N, C * S * B, "cols of X"); need(N, S * B * R, "cols of X (scatter)")
    else:
        raise ValueError(f"unknown dataflow {dataflow!r}")


# --------------------------------------------------------------------------------------
# what device (i,j) holds in HBM after the (emulated) all-gathers
# --------------------------------------------------------------------------------------

def device_operands_os(X, W, R, C, i, j, S, B):
    """OS: gathered slices ``A_k = X[rows_i, sel_k]`` and ``B_k = W[sel_k, cols_j]``
    (TensorParallel.py:157-160,163-164,168-169; S=1 is Collective_OS :19-22)."""
    Kd = X.shape[1]
    rows = block_range(X.shape[0], R, i)
    cols = block_range(W.shape[1], C, j)
    A = [np.ascontiguousarray(X[rows, :][:, sel(Kd, S, B, k)]) for k in range(S)]
    Bs = [np.ascontiguousarray(W[:, cols][sel(Kd, S, B, k), :]) for k in range(S)]
    return A, Bs


def device_operands_ls(X, W, R, C, i, j, S, B):
    """LS: local ``A = X_ij`` and gathered row-slices ``W_k = W[sel_k(O), cols_j(I)]``
    stored ``[O/S, I/C]`` (TensorParallel.py:177-180,186)."""
    O = W.shape[0]
    A = np.ascontiguousarray(shard(X, R, C, i, j))
    cols = block_range(W.shape[1], C, j)
    Ws = [np.ascontiguousarray(W[:, cols][sel(O, S, B, k), :]) for k in range(S)]
    return A, Ws


def device_operands_rs(X, W, R, C, i, j, S, B):
    """RS: gathered column-slices ``X_k = X[rows_i(I), sel_k(N)]`` stored ``[I/R, N/S]``
    (used transposed) and local ``W_ij`` (TensorParallel.py:198-202,208)."""
    N = X.shape[1]
    rows = block_range(X.shape[0], R, i)
    Xs = [np.ascontiguousarray(X[rows, :][:, sel(N, S, B, k)]) for k in range(S)]
    Wl = np.ascontiguousarray(shard(W, R, C, i, j))
    return Xs, Wl


# --------------------------------------------------------------------------------------
# float64 device-block oracles (what the HIP kernels are compared with)
# --------------------------------------------------------------------------------------

def oracle_os_block(A_slices, B_slices) -> np.ndarray:
    """``C = sum_k A_k @ B_k`` in float64 (TensorParallel.py:162,167,172)."""
    acc = None
    for a, b in zip(A_slices, B_slices):
        p = np.asarray(a, np.float64) @ np.asarray(b, np.float64)
        acc = p if acc is None else acc + p
    return acc


def oracle_ls_chunks(A, W_slices):
    """``Y_k = A @ W_k^T`` in float64: the partial chunks fed to psum_scatter
    (TensorParallel.py:181,187)."""
    a = np.asarray(A, np.float64)
    return [a @ np.asarray(w, np.float64).T for w in W_slices]


def oracle_rs_chunks(X_slices, W):
    """``Y_k = X_k^T @ W`` in float64 (TensorParallel.py:203,209)."""
    w = np.asarray(W, np.float64)
    return [np.asarray(x, np.float64).T @ w for x in X_slices]


def gelu_tanh(x: np.ndarray) -> np.ndarray:
    """GELU in the tanh form ``0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3)))`` in float64: what
    ``jax.nn.gelu`` computes by default, applied by the reference after ff1 (ShardedLayers.py:182)."""
    x = np.asarray(x, np.float64)
    return 0.5 * x * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (x + 0.044715 * x ** 3)))


def oracle_os_fused(A_slices, B_slices, activation=None, residual=None):
    """Float64 oracle of the output-stationary block with the element-wise work that follows it in the
    reference's transformer block folded in: ``Y = act(sum_k A_k @ B_k) + residual`` (ShardedLayers.py:181-184)
    and the local row moments of ``Y`` that the layer norm sums over the mesh columns (:125-126, as sums).
    Returns ``(Y, row_sum, row_sumsq)``."""
    y = oracle_os_block(A_slices, B_slices)
    if activation == "gelu":
        y = gelu_tanh(y)
    elif activation is not None:
        raise ValueError(f"unknown activation {activation!r}")
    if residual is not None:
        y = y + np.asarray(residual, np.float64)
    return y, y.sum(axis=1), (y * y).sum(axis=1)


def assemble_ls(chunks_by_col, R, C, j, S, B):
    """Mesh completion of LS for device column j: ``chunks_by_col[j'][k]`` are the partial
    chunks ``[m, O/S]`` of the C devices of one mesh row.  psum_scatter over ``col`` along
    dim 1 (TensorParallel.py:182,188) then the ``(.., S, B)`` interleave and reshape
    (:184,190,193).  Returns device (i,j)'s ``[m, O/C]`` block."""
    m, Os = chunks_by_col[0][0].shape
    O = Os * S
    out = np.zeros((m, O // C), dtype=chunks_by_col[0][0].dtype)
    for k in range(S):
        red = sum(chunks_by_col[jj][k] for jj in range(C))
        g = sel(O, S, B, k)
        lo, hi = j * (O // C), (j + 1) * (O // C)
        keep = (g >= lo) & (g < hi)
        out[:, g[keep] - lo] = red[:, keep]
    return out


def assemble_rs(chunks_by_row, R, C, i, S, B):
    """Mesh completion of RS for device row i: psum_scatter over ``row`` along dim 0
    (TensorParallel.py:204,210), interleave (:206,211), reshape (:214)."""
    Ns, n = chunks_by_row[0][0].shape
    N = Ns * S
    out = np.zeros((N // R, n), dtype=chunks_by_row[0][0].dtype)
    for k in range(S):
        red = sum(chunks_by_row[ii][k] for ii in range(R))
        g = sel(N, S, B, k)
        lo, hi = i * (N // R), (i + 1) * (N // R)
        keep = (g >= lo) & (g < hi)
        out[g[keep] - lo, :] = red[keep, :]
    return out


# --------------------------------------------------------------------------------------
# the layout steps either side of the contraction, statement by statement
# --------------------------------------------------------------------------------------

def pack_slices(block: np.ndarray, S: int, B: int, axis: int):
    """The S slices a device cuts out of its shard before the all-gathers: the reshape to
    ``(rows, cols/(S*B), S, B)`` (axis 1, TensorParallel.py:155,157,198-199) or
    ``(rows/(S*B), S, B, cols)`` (axis 0, :156,158,177-178) followed by ``dynamic_slice_in_dim(.., k, 1)``
    along the S axis and the flattening the einsum subscripts imply."""
    r, c = block.shape
    if S < 1 or B < 1 or (c if axis == 1 else r) % (S * B):
        raise ValueError("sliced extent is not a multiple of S*B")
    out = []
    for k in range(S):
        if axis == 1:
            v = block.reshape(r, c // (S * B), S, B)
            out.append(np.ascontiguousarray(_dyn_slice(v, k, 1, 2)).reshape(r, c // S))
        else:
            v = block.reshape(r // (S * B), S, B, c)
            out.append(np.ascontiguousarray(_dyn_slice(v, k, 1, 1)).reshape(r // S, c))
    return out


def unpack_chunks(chunks_by_peer, B: int, axis: int, window: int = 0, parts: int = 1, out_dtype=np.float32):
    """A device's output shard from its peers' partial chunks: tiled ``psum_scatter`` of chunk k along
    ``axis`` over ``parts`` devices, of which this one is number ``window`` (TensorParallel.py:182,188,
    204,210: sum over the peers in fp32, in peer order; keep the window), ``dynamic_update_slice_in_dim``
    at position k of the zero-initialised ``(.., S, B)`` view (:179,184,190 / :200,206,211), final reshape
    (:193,:214).  ``out_dtype`` np.float32, or "bf16" for the fp32 sum rounded once to bf16 (returned as
    float32 values)."""
    S = len(chunks_by_peer[0])
    cr, cc = chunks_by_peer[0][0].shape
    cut = cc if axis == 1 else cr
    if cut % parts or (cut // parts) % B:
        raise ValueError("chunk does not split into windows of whole blocks")
    keep = cut // parts
    nb = keep // B
    Y = np.zeros((cr, nb, S, B), np.float32) if axis == 1 else np.zeros((nb, S, B, cc), np.float32)
    for k in range(S):
        tot = np.array(chunks_by_peer[0][k], dtype=np.float32)
        for peer in chunks_by_peer[1:]:
            tot = tot + np.asarray(peer[k], dtype=np.float32)
        mine = _dyn_slice(tot, window * keep, keep, axis)
        if axis == 1:
            Y[:, :, k:k + 1, :] = mine.reshape(cr, nb, 1, B)
        else:
            Y[:, k:k + 1, :, :] = mine.reshape(nb, 1, B, cc)
    Y = Y.reshape(cr, keep * S) if axis == 1 else Y.reshape(keep * S, cc)
    return bf16_round(Y) if out_dtype == "bf16" else Y


# --------------------------------------------------------------------------------------
# literal whole-mesh emulation of the reference bodies
# --------------------------------------------------------------------------------------

def _dyn_slice(a, start, size, axis):
    """jax.lax.dynamic_slice_in_dim: the start index is CLAMPED so the slice stays in range."""
    start = max(0, min(int(start), a.shape[axis] - size))
    idx = [slice(None)] * a.ndim
    idx[axis] = slice(start, start + size)
    return a[tuple(idx)]


def _all_gather(blocks, R, C, over, axis):
    """tiled all_gather over mesh axis ``over`` ('row' or 'col'): every device receives the
    concatenation, in axis-index order, of its peers' blocks along ``axis``."""
    out = [[None] * C for _ in range(R)]
    for i in range(R):
        for j in range(C):
            peers = [blocks[i][jj] for jj in range(C)] if over == "col" else [blocks[ii][j] for ii in range(R)]
            out[i][j] = np.concatenate(peers, axis=axis)
    return out


def _psum_scatter(blocks, R, C, over, axis):
    """tiled psum_scatter: sum over the peers of mesh axis ``over``; peer p keeps the p-th of
    ``size`` equal parts along ``axis``."""
    out = [[None] * C for _ in range(R)]
    for i in range(R):
        for j in range(C):
            if over == "col":
                tot = sum(blocks[i][jj] for jj in range(C)); parts, me = C, j
            else:
                tot = sum(blocks[ii][j] for ii in range(R)); parts, me = R, i
            n = tot.shape[axis] // parts
            out[i][j] = _dyn_slice(tot, me * n, n, axis)
    return out


def _shards(G, R, C):
    return [[np.array(shard(G, R, C, i, j)) for j in range(C)] for i in range(R)]


def _unshard(blocks):
    return np.concatenate([np.concatenate(row, axis=1) for row in blocks], axis=0)


def _map2(f, a, b, R, C):
    return [[f(a[i][j], b[i][j]) for j in range(C)] for i in range(R)]


def literal_collective(dataflow, X, W, R, C):
    """Whole-mesh emulation of Collective_OS/LS/RS (TensorParallel.py:19-32)."""
    Xs, Ws = _shards(X, R, C), _shards(W, R, C)
    if dataflow == "os":
        Xi = _all_gather(Xs, R, C, "col", 1)
        Wj = _all_gather(Ws, R, C, "row", 0)
        return _unshard(_map2(lambda a, b: a @ b, Xi, Wj, R, C))
    if dataflow == "ls":
        Wj = _all_gather(Ws, R, C, "row", 0)
        Yp = _map2(lambda a, b: np.einsum("mn,kn->mk", a, b), Xs, Wj, R, C)
        return _unshard(_psum_scatter(Yp, R, C, "col", 1))
    if dataflow == "rs":
        Xi = _all_gather(Xs, R, C, "col", 1)
        Yp = _map2(lambda a, b: np.einsum("ib,io->bo", a, b), Xi, Ws, R, C)
        return _unshard(_psum_scatter(Yp, R, C, "row", 0))
    raise ValueError(dataflow)


def literal_meshflow_os(X, W, R, C, K, B):
    """Whole-mesh emulation of MeshFlow_OS, statement by statement (TensorParallel.py:153-172),
    including the clamped ``dynamic_slice`` that makes ``K == 1`` add slice 0 twice."""
    Xs, Ws = _shards(X, R, C), _shards(W, R, C)
    Xsp = [[x.reshape(x.shape[0], x.shape[1] // (K * B), K, B) for x in row] for row in Xs]
    Wsp = [[w.reshape(w.shape[0] // (K * B), K, B, w.shape[1]) for w in row] for row in Ws]
    xb = lambda k: [[_dyn_slice(x, k, 1, 2) for x in row] for row in Xsp]
    wb = lambda k: [[_dyn_slice(w, k, 1, 1) for w in row] for row in Wsp]
    dot = lambda a, b: np.einsum("nikb,ikbo->no", a, b)
    Xk = _all_gather(xb(0), R, C, "col", 1)
    Wk = _all_gather(wb(0), R, C, "row", 0)
    Y = _map2(dot, Xk, Wk, R, C)
    Xk = _all_gather(xb(1), R, C, "col", 1)
    Wk = _all_gather(wb(1), R, C, "row", 0)
    for kk in range(1, K - 1):
        Y = _map2(lambda y, p: y + p, Y, _map2(dot, Xk, Wk, R, C), R, C)
        Xk = _all_gather(xb(kk + 1), R, C, "col", 1)
        Wk = _all_gather(wb(kk + 1), R, C, "row", 0)
    Y = _map2(lambda y, p: y + p, Y, _map2(dot, Xk, Wk, R, C), R, C)
    return _unshard(Y)


def literal_meshflow_ls(X, W, R, C, K, B):
    """Whole-mesh emulation of MeshFlow_LS (TensorParallel.py:174-193)."""
    Xs, Ws = _shards(X, R, C), _shards(W, R, C)
    O = Ws[0][0].shape[0] * R
    Wsp = [[w.reshape(w.shape[0] // K // B, K, B, w.shape[1]) for w in row] for row in Ws]
    Y = [[np.zeros((x.shape[0], O // (K * B * C), K, B), X.dtype) for x in row] for row in Xs]
    for kk in range(K):
        Wk = _all_gather([[_dyn_slice(w, kk, 1, 1) for w in row] for row in Wsp], R, C, "row", 0)
        Yk = _map2(lambda a, b: np.einsum("ni,okbi->nokb", a, b), Xs, Wk, R, C)
        Yk2 = _psum_scatter(Yk, R, C, "col", 1)
        for i in range(R):
            for j in range(C):
                Y[i][j][:, :, kk:kk + 1, :] = Yk2[i][j]
    return _unshard([[y.reshape(y.shape[0], -1) for y in row] for row in Y])


def literal_meshflow_rs(X, W, R, C, K, B):
    """Whole-mesh emulation of MeshFlow_RS (TensorParallel.py:195-214)."""
    Xs, Ws = _shards(X, R, C), _shards(W, R, C)
    N = Xs[0][0].shape[1] * C
    Xsp = [[x.reshape(x.shape[0], x.shape[1] // K // B, K, B) for x in row] for row in Xs]
    Y = [[np.zeros((N // (K * B * R), K, B, w.shape[1]), X.dtype) for w in row] for row in Ws]
    for kk in range(K):
        Xk = _all_gather([[_dyn_slice(x, kk, 1, 2) for x in row] for row in Xsp], R, C, "col", 1)
        Yk = _map2(lambda a, b: np.einsum("inkb,io->nkbo", a, b), Xk, Ws, R, C)
        Yk2 = _psum_scatter(Yk, R, C, "row", 0)
        for i in range(R):
            for j in range(C):
                Y[i][j][:, kk:kk + 1, :, :] = Yk2[i][j]
    return _unshard([[y.reshape(-1, y.shape[-1]) for y in row] for row in Y])


def literal_meshflow(dataflow, X, W, R, C, K, B):
    return {"os": literal_meshflow_os, "ls": literal_meshflow_ls, "rs": literal_meshflow_rs}[dataflow](X, W, R, C, K, B)


# --------------------------------------------------------------------------------------
# literal whole-mesh emulation of the ring baselines (Wang, Cannon)
# --------------------------------------------------------------------------------------
# The reference's bodies read the device's position with ``jax.lax.ax_index`` (TensorParallel.py:37,67,
# 122,219-220,264-265,305-306), a name JAX does not have; they are restated here with the position taken
# as ``axis_index`` would give it, which is the only reading under which they compute the product.

def _ppermute(blocks, R, C, over, shift):
    """jax.lax.ppermute with perm [(p, (p + shift) % size)]: every device sends its block to the peer
    ``shift`` places further along mesh axis ``over``; returned is what each device receives."""
    out = [[None] * C for _ in range(R)]
    for i in range(R):
        for j in range(C):
            if over == "col":
                out[i][(j + shift) % C] = blocks[i][j]
            else:
                out[(i + shift) % R][j] = blocks[i][j]
    return out


def _grid(f, R, C):
    return [[f(i, j) for j in range(C)] for i in range(R)]


def literal_wang_os(X, W, R, C):
    """Wang_OS (TensorParallel.py:34-61): W gathered over the rows; the two halves of the X shard travel
    round the mesh row in opposite directions, each multiplied with the matching half-block of W."""
    Xs, Ws = _shards(X, R, C), _shards(W, R, C)
    Wj = _all_gather(Ws, R, C, "row", 0)
    size = C
    up = lambda b: _ppermute(b, R, C, "col", +1)
    dn = lambda b: _ppermute(b, R, C, "col", -1)
    B = Wj[0][0].shape[0] // size // 2
    wb = lambda i, j, blk, hi: _dyn_slice(Wj[i][j], (2 * blk + hi) * B, B, 0)
    lo = _grid(lambda i, j: np.split(Xs[i][j], 2, axis=1)[0], R, C)
    hi = _grid(lambda i, j: np.split(Xs[i][j], 2, axis=1)[1], R, C)
    out = _grid(lambda i, j: lo[i][j] @ wb(i, j, j, 0) + hi[i][j] @ wb(i, j, j, 1), R, C)
    lo, hi = up(lo), dn(hi)
    for ii in range(1, size):
        lo2, hi2 = up(lo), dn(hi)
        out = _grid(lambda i, j: out[i][j] + lo[i][j] @ wb(i, j, (j - ii) % size, 0) + hi[i][j] @ wb(i, j, (j + ii) % size, 1), R, C)
        lo, hi = lo2, hi2
    return _unshard(out)


def literal_wang_ls(X, W, R, C):
    """Wang_LS (TensorParallel.py:64-90): W ([out, in]) gathered over the rows; partial outputs for one
    half-block of the output columns at a time travel round the mesh row and pick up every device's term."""
    Xs, Ws = _shards(X, R, C), _shards(W, R, C)
    Wj = _all_gather(Ws, R, C, "row", 0)
    size = C
    up = lambda b: _ppermute(b, R, C, "col", +1)
    dn = lambda b: _ppermute(b, R, C, "col", -1)
    B = Wj[0][0].shape[0] // size // 2
    wb = lambda i, j, blk, hi: _dyn_slice(Wj[i][j], (2 * blk + hi) * B, B, 0)
    dot = lambda a, b: np.einsum("bi,oi->bo", a, b)
    ylo = _grid(lambda i, j: dot(Xs[i][j], wb(i, j, (j - 1) % size, 0)), R, C)
    yhi = _grid(lambda i, j: dot(Xs[i][j], wb(i, j, (j + 1) % size, 1)), R, C)
    for ii in range(1, size):
        ylo, yhi = up(ylo), dn(yhi)
        ylo = _grid(lambda i, j: ylo[i][j] + dot(Xs[i][j], wb(i, j, (j - ii - 1) % size, 0)), R, C)
        yhi = _grid(lambda i, j: yhi[i][j] + dot(Xs[i][j], wb(i, j, (j + ii + 1) % size, 1)), R, C)
    return _unshard(_grid(lambda i, j: np.concatenate([ylo[i][j], yhi[i][j]], axis=1), R, C))


def literal_wang_rs(X, W, R, C):
    """Wang_RS, the branch the reference takes (TensorParallel.py:120-149): the halves of the X shard
    ([in, tokens]) travel round the mesh row; every device fills its [tokens, out/C] partial block by block,
    then psum_scatter over the rows."""
    Xs, Ws = _shards(X, R, C), _shards(W, R, C)
    size = C
    up = lambda b: _ppermute(b, R, C, "col", +1)
    dn = lambda b: _ppermute(b, R, C, "col", -1)
    dot = lambda a, b: np.einsum("ib,io->bo", a, b)
    Yj = _grid(lambda i, j: np.zeros((Xs[i][j].shape[1] * C, Ws[i][j].shape[1]), X.dtype), R, C)
    B = Yj[0][0].shape[0] // size // 2

    def put(y, blk, start):
        y = y.copy(); y[start:start + blk.shape[0]] = blk
        return y
    Yj = _grid(lambda i, j: put(Yj[i][j], dot(Xs[i][j], Ws[i][j]), 2 * (j % size) * B), R, C)
    lo = up(_grid(lambda i, j: np.split(Xs[i][j], 2, axis=1)[0], R, C))
    hi = dn(_grid(lambda i, j: np.split(Xs[i][j], 2, axis=1)[1], R, C))
    for ii in range(1, size):
        Yj = _grid(lambda i, j: put(Yj[i][j], dot(lo[i][j], Ws[i][j]), 2 * ((j - ii) % size) * B), R, C)
        Yj = _grid(lambda i, j: put(Yj[i][j], dot(hi[i][j], Ws[i][j]), 2 * ((j + ii) % size) * B + B), R, C)
        lo, hi = up(lo), dn(hi)
    return _unshard(_psum_scatter(Yj, R, C, "row", 0))


def literal_cannon_os(X, W, R, C):
    """Cannon_OS (TensorParallel.py:218-260), square mesh: device (r, c) starts at half-block pair
    k = (c + r) % N; the halves of both operands move on in opposite directions every step."""
    assert R == C
    N = C
    Xs, Ws = _shards(X, R, C), _shards(W, R, C)
    Xi = _all_gather(Xs, R, C, "col", 1)
    Wj = _all_gather(Ws, R, C, "row", 0)
    B = Xi[0][0].shape[1] // N // 2
    k = lambda i, j: (j + i) % N
    xl = _grid(lambda i, j: _dyn_slice(Xi[i][j], 2 * k(i, j) * B, B, 1), R, C)
    xh = _grid(lambda i, j: _dyn_slice(Xi[i][j], (2 * k(i, j) + 1) * B, B, 1), R, C)
    wl = _grid(lambda i, j: _dyn_slice(Wj[i][j], 2 * k(i, j) * B, B, 0), R, C)
    wh = _grid(lambda i, j: _dyn_slice(Wj[i][j], (2 * k(i, j) + 1) * B, B, 0), R, C)
    out = _grid(lambda i, j: xl[i][j] @ wl[i][j] + xh[i][j] @ wh[i][j], R, C)
    step = lambda xl, xh, wl, wh: (_ppermute(xl, R, C, "col", -1), _ppermute(xh, R, C, "col", +1),
                                   _ppermute(wl, R, C, "row", -1), _ppermute(wh, R, C, "row", +1))
    xl, xh, wl, wh = step(xl, xh, wl, wh)
    for _ in range(1, N):
        nxt = step(xl, xh, wl, wh)
        out = _grid(lambda i, j: out[i][j] + xl[i][j] @ wl[i][j] + xh[i][j] @ wh[i][j], R, C)
        xl, xh, wl, wh = nxt
    return _unshard(out)


def literal_cannon_ls(X, W, R, C):
    """Cannon_LS (TensorParallel.py:262-300)."""
    assert R == C
    N = C
    Xs, Ws = _shards(X, R, C), _shards(W, R, C)
    k = lambda i, j: (j + i) % N
    B = Ws[0][0].shape[0] // 2
    Wj = _all_gather(Ws, R, C, "row", 0)
    wl = _grid(lambda i, j: _dyn_slice(Wj[i][j], 2 * k(i, j) * B, B, 0), R, C)
    wh = _grid(lambda i, j: _dyn_slice(Wj[i][j], (2 * k(i, j) + 1) * B, B, 0), R, C)
    dot = lambda a, b: np.einsum("bi,oi->bo", a, b)
    yl = _map2(dot, Xs, wl, R, C)
    yh = _map2(dot, Xs, wh, R, C)
    for _ in range(1, N):
        wl, wh = _ppermute(wl, R, C, "row", -1), _ppermute(wh, R, C, "row", +1)
        yl, yh = _ppermute(yl, R, C, "col", -1), _ppermute(yh, R, C, "col", +1)
        yl = _map2(lambda y, p: y + p, yl, _map2(dot, Xs, wl, R, C), R, C)
        yh = _map2(lambda y, p: y + p, yh, _map2(dot, Xs, wh, R, C), R, C)
    yl, yh = _ppermute(yl, R, C, "col", -1), _ppermute(yh, R, C, "col", +1)
    Yik = _grid(lambda i, j: np.concatenate([yl[i][j], yh[i][j]], axis=1), R, C)
    Yi = _all_gather(Yik, R, C, "col", 1)
    return _unshard(_grid(lambda i, j: _dyn_slice(Yi[i][j], 2 * ((j - i) % N) * B, 2 * B, 1), R, C))


def literal_cannon_rs(X, W, R, C):
    """Cannon_RS (TensorParallel.py:379-417, the definition in force; the earlier one at :302-342 that it shadows
    issues the same products, shifts and sums in the same order)."""
    assert R == C
    N = C
    Xs, Ws = _shards(X, R, C), _shards(W, R, C)
    k = lambda i, j: (j + i) % N
    B = Xs[0][0].shape[1] // 2
    Xi = _all_gather(Xs, R, C, "col", 1)
    xl = _grid(lambda i, j: _dyn_slice(Xi[i][j], 2 * k(i, j) * B, B, 1), R, C)
    xh = _grid(lambda i, j: _dyn_slice(Xi[i][j], (2 * k(i, j) + 1) * B, B, 1), R, C)
    dot = lambda a, b: np.einsum("ib,io->bo", a, b)
    yl = _map2(dot, xl, Ws, R, C)
    yh = _map2(dot, xh, Ws, R, C)
    for _ in range(1, N):
        xl, xh = _ppermute(xl, R, C, "col", -1), _ppermute(xh, R, C, "col", +1)
        yl, yh = _ppermute(yl, R, C, "row", -1), _ppermute(yh, R, C, "row", +1)
        yl = _map2(lambda y, p: y + p, yl, _map2(dot, xl, Ws, R, C), R, C)
        yh = _map2(lambda y, p: y + p, yh, _map2(dot, xh, Ws, R, C), R, C)
    yl, yh = _ppermute(yl, R, C, "row", -1), _ppermute(yh, R, C, "row", +1)
    Ykj = _grid(lambda i, j: np.concatenate([yl[i][j], yh[i][j]], axis=0), R, C)
    Yj = _all_gather(Ykj, R, C, "row", 0)
    return _unshard(_grid(lambda i, j: _dyn_slice(Yj[i][j], 2 * ((i - j) % N) * B, 2 * B, 0), R, C))


def literal_ring(algorithm, dataflow, X, W, R, C):
    return {("wang", "os"): literal_wang_os, ("wang", "ls"): literal_wang_ls, ("wang", "rs"): literal_wang_rs,
            ("cannon", "os"): literal_cannon_os, ("cannon", "ls"): literal_cannon_ls,
            ("cannon", "rs"): literal_cannon_rs}[(algorithm, dataflow)](X, W, R, C)


# the order in which device (i, j) multiplies its 2 * size half-blocks (what its local kernel call is given)
def ring_order(algorithm: str, dataflow: str, R: int, C: int, i: int, j: int):
    """[(block, half)] in step order for device (i, j): block indexes the contraction (OS) or output (LS /
    RS) range in units of two half-blocks.  Wang: the ring is the mesh row (size C), Cannon: N = R = C."""
    if algorithm == "wang":
        size = C
        if dataflow == "os":
            return [p for t in range(size) for p in (((j - t) % size, 0), ((j + t) % size, 1))]
        if dataflow == "ls":
            return [p for t in range(size) for p in (((j - 1 - t) % size, 0), ((j + 1 + t) % size, 1))]
        return [p for t in range(size) for p in (((j - t) % size, 0), ((j + t) % size, 1))]
    N = C
    k = (i + j) % N
    return [p for t in range(N) for p in (((k + t) % N, 0), ((k - t) % N, 1))]


def dense(dataflow, X, W):
    """What each dataflow computes on the global operands (MeshFlowCPU.ipynb cells 2-3):
    OS ``X@W``; LS ``X@W^T``; RS ``X^T@W``."""
    X = np.asarray(X, np.float64); W = np.asarray(W, np.float64)
    return {"os": lambda: X @ W, "ls": lambda: X @ W.T, "rs": lambda: X.T @ W}[dataflow]()


# --------------------------------------------------------------------------------------
# the reference's deterministic fixtures
# --------------------------------------------------------------------------------------

def notebook_inputs(dtype=np.float32):
    """MeshFlowCPU.ipynb cell 2-3: 4x2 mesh, (B,I,O)=(512,256,1024), arange-scaled operands."""
    Bt, I, O = 512, 256, 1024
    X = (np.arange(Bt * I, dtype=np.float32).reshape(Bt, I) / np.float32(Bt * I)).astype(dtype)
    W = (np.arange(I * O, dtype=np.float32).reshape(I, O) / np.float32(I * O)).astype(dtype)
    dY = (np.ones(Bt * O, dtype=np.float32).reshape(Bt, O) / np.float32(Bt * O)).astype(dtype)
    return dict(mesh=(4, 2), B=Bt, I=I, O=O, X=X, W=W, dY=dY, K=8, blocksize=8)


def selfcheck_inputs(dtype=np.float32):
    """TensorParallel.py:427-434: 4x4 mesh, X[512,3072], W[3072,12288], arange-scaled."""
    Bb, S, H, D = 4, 128, 48, 64
    n, d = Bb * S, H * D
    X = (np.arange(n * d, dtype=np.float32).reshape(n, d) / np.float32(n * d)).astype(dtype)
    W = (np.arange(d * 4 * d, dtype=np.float32).reshape(d, 4 * d) / np.float32(4 * d * d)).astype(dtype)
    return dict(mesh=(4, 4), X=X, W=W, K=8, blocksize=8)


# --------------------------------------------------------------------------------------
# CPU restatement of one device's body, as timed for the CPU baseline
# --------------------------------------------------------------------------------------

def cpu_device_body_os(A_slices, B_slices, out_dtype=np.float32):
    """One device's MeshFlow_OS work on already-gathered slices: S matmuls accumulated
    slice by slice (TensorParallel.py:162-172) in fp32 BLAS."""
    acc = A_slices[0] @ B_slices[0]
    for a, b in zip(A_slices[1:], B_slices[1:]):
        acc += a @ b
    return acc.astype(out_dtype, copy=False)


def cpu_device_body_ls(A, W_slices):
    """One device's MeshFlow_LS work: S chunk matmuls ``A @ W_k^T`` (TensorParallel.py:181,187)."""
    return [A @ w.T for w in W_slices]


def cpu_device_body_rs(X_slices, W):
    """One device's MeshFlow_RS work: S chunk matmuls ``X_k^T @ W`` (TensorParallel.py:203,209)."""
    return [x.T @ W for x in X_slices]
