"""2-D tensor-parallel GEMM: the reference's ``SPMD(mesh, algorithm, blocksize).OS/LS/RS(K)`` surface
with the mesh emulated on the host and the local contraction running in hand-written gfx950 kernels.

Mirrors reference TensorParallel.py: the unsliced bodies ``Collective_OS/LS/RS`` (:19-32), the sliced
bodies ``MeshFlow_OS/LS/RS`` (:153-214) and the builder ``SPMD`` (:346-377).  Differences, all forced
by having one GPU and no tracing compiler:

* the callable returned by ``OS/LS/RS`` takes the GLOBAL operands (torch tensors on the GPU), logically
  sharded ``P(row, col)``, and returns the GLOBAL result; it runs every mesh device's body in turn;
* ``.device(i, j)`` runs ONE device's body and returns what that device produces before any
  cross-device reduction: its output block (OS) or its S fp32 partial chunks (LS / RS);
* all_gather / psum_scatter move data between the emulated devices' buffers on the one GPU: the
  block-cyclic slicing, the placement of gathered slices and the reduce + interleave of the chunks run
  in the layout kernels of libmeshslice_hip.so (slice_layout.py), not in torch indexing;
* the local contraction accumulates in fp32 over all slices and rounds once (the reference carries
  the running sum in the input dtype, :167);
* the sliced OS body rejects ``K == 1``: the reference adds slice 0 twice in that case (:163,:172);
  use ``algorithm='collective'`` for the unsliced product;
* the ring baselines 'wang' and 'cannon' (:34-149, :218-342) drive the same kernels with 2 * size
  half-block slices in ring order; the hops themselves are host index arithmetic.
"""
from __future__ import annotations

from typing import Callable, List, Sequence

import torch

from . import local_gemm, slice_layout
from .mesh import Mesh, PartitionSpec as P  # noqa: F401  (re-exported like the reference's imports)


def allclose(a, b) -> bool:
    """The reference's acceptance test (TensorParallel.py:16-17)."""
    return bool(torch.allclose(torch.as_tensor(a).float().cpu(), torch.as_tensor(b).float().cpu(), atol=1e-2, rtol=1e-2))


# ------------------------------------------------------------------------------------------------
# host-side mesh plumbing
# ------------------------------------------------------------------------------------------------

def _shards(G: torch.Tensor, R: int, C: int) -> List[List[torch.Tensor]]:
    """blocks[i][j] = device (i,j)'s shard of a matrix sharded P(row, col) (views, no copies)."""
    if G.dim() != 2:
        raise ValueError("operands must be 2-D")
    if G.shape[0] % R or G.shape[1] % C:
        raise ValueError(f"matrix {tuple(G.shape)} does not shard evenly over a {R}x{C} mesh")
    h, w = G.shape[0] // R, G.shape[1] // C
    return [[G[i * h:(i + 1) * h, j * w:(j + 1) * w] for j in range(C)] for i in range(R)]


def _need(v: int, d: int, what: str) -> None:
    if d <= 0 or v % d:
        raise ValueError(f"{what} = {v} is not a multiple of {d}")


def _own(block: torch.Tensor) -> torch.Tensor:
    """A device's shard as the kernels can address it: the view itself when its first element and its rows
    are 16-byte aligned (a real device's shard is its own buffer), else a contiguous copy."""
    if block.stride(1) == 1 and block.data_ptr() % 16 == 0 and (block.stride(0) * block.element_size()) % 16 == 0:
        return block
    return block.contiguous()


def _gather(parts: Sequence[torch.Tensor], axis: int) -> torch.Tensor:
    """tiled all_gather of whole shards as the receiving device sees it: peers' parts concatenated in axis
    order, materialised contiguous in HBM (what a real all-gather delivers)."""
    return torch.cat(list(parts), dim=axis).contiguous()


def _gather_col_slices(peers: Sequence[torch.Tensor], K: int, B: int) -> List[torch.Tensor]:
    """The K gathered column slices ``[rows, len(peers) * cols / K]``: every peer cuts its shard's columns into
    K block-cyclic slices (reference :155,157,198-199) and slice k of peer p lands at column block p of
    gathered slice k (all_gather over the peers' axis, tiled along the columns).  One kernel per peer writes
    its K slices straight into their places; there is no separate concatenation."""
    r, c = peers[0].shape
    _need(c, K * B, "sliced extent")
    w = c // K
    buf = torch.empty((K, r, len(peers) * w), dtype=peers[0].dtype, device=peers[0].device)
    for p, blk in enumerate(peers):
        slice_layout.pack_slices(blk, K, B, 1, out=[buf[k][:, p * w:(p + 1) * w] for k in range(K)])
    return [buf[k] for k in range(K)]


def _gather_row_slices(peers: Sequence[torch.Tensor], K: int, B: int) -> List[torch.Tensor]:
    """The K gathered row slices ``[len(peers) * rows / K, cols]`` (reference :156,158,177-178), peer p's part
    of slice k at row block p."""
    r, c = peers[0].shape
    _need(r, K * B, "sliced extent")
    h = r // K
    buf = torch.empty((K, len(peers) * h, c), dtype=peers[0].dtype, device=peers[0].device)
    for p, blk in enumerate(peers):
        slice_layout.pack_slices(blk, K, B, 0, out=[buf[k][p * h:(p + 1) * h] for k in range(K)])
    return [buf[k] for k in range(K)]


# ------------------------------------------------------------------------------------------------
# per-device bodies.  X, W are the shard grids; (i, j) the device; the return value is what that
# device holds after its local contractions.
# ------------------------------------------------------------------------------------------------

def Collective_OS(X, W, i, j, R, C, K, B):
    """reference TensorParallel.py:19-22: gather X over col, W over row, one contraction."""
    Xi = _gather([X[i][jj] for jj in range(C)], 1)
    Wj = _gather([W[ii][j] for ii in range(R)], 0)
    return local_gemm.gemm_os([Xi], [Wj])


def Collective_LS(X, W, i, j, R, C, K, B):
    """reference :24-27: gather W over row; partial product X_ij @ Wj^T (input of psum_scatter)."""
    Wj = _gather([W[ii][j] for ii in range(R)], 0)
    return local_gemm.gemm_ls(_own(X[i][j]), [Wj])


def Collective_RS(X, W, i, j, R, C, K, B):
    """reference :29-32: gather X over col; partial product Xi^T @ W_ij (input of psum_scatter)."""
    Xi = _gather([X[i][jj] for jj in range(C)], 1)
    return local_gemm.gemm_rs([Xi], _own(W[i][j]))


def MeshFlow_OS(X, W, i, j, R, C, K, B):
    """reference :153-172: K gathered slice pairs, accumulated into one output block."""
    if K == 1:
        raise ValueError("the sliced OS body is undefined for K == 1 (the reference adds slice 0 twice); "
                         "use algorithm='collective' for the unsliced product")
    A_slices = _gather_col_slices([X[i][jj] for jj in range(C)], K, B)
    B_slices = _gather_row_slices([W[ii][j] for ii in range(R)], K, B)
    return local_gemm.gemm_os(A_slices, B_slices)


_gather_streams = {}
OVERLAP_RESERVED_CUS = 32      # compute units left to the emulated gathers' copy kernels beside the waiting product


def _col_slice_filler(peers, K, B):
    """(buffer ``[K, rows, len(peers) * cols / K]`` for the K gathered column slices, ``fill(k)`` that gathers slice k into
    it on the current stream): slice k of a shard is its B-wide column blocks b with b % K == k (reference :155,157,198-199)."""
    r, c = peers[0].shape
    _need(c, K * B, "sliced extent")
    w = c // K
    buf = torch.empty((K, r, len(peers) * w), dtype=peers[0].dtype, device=peers[0].device)

    def fill(k):
        for p, blk in enumerate(peers):
            buf[k][:, p * w:(p + 1) * w].copy_(blk.reshape(r, w // B, K, B)[:, :, k, :].reshape(r, w))
    return buf, fill


def _row_slice_filler(peers, K, B):
    """The same for the K gathered row slices ``[K, len(peers) * rows / K, cols]`` (reference :156,158,177-178)."""
    h, n = peers[0].shape
    _need(h, K * B, "sliced extent")
    hk = h // K
    buf = torch.empty((K, len(peers) * hk, n), dtype=peers[0].dtype, device=peers[0].device)

    def fill(k):
        for p, blk in enumerate(peers):
            buf[k][p * hk:(p + 1) * hk].copy_(blk.reshape(hk // B, K, B, n)[:, k].reshape(hk, n))
    return buf, fill


def _launch_ahead_of_gathers(K, dev, launch, fills):
    """``launch(ready)`` enqueues the gated product on the current stream with all K flags down; the emulated gather
    stream then fills slice after slice (``fills``: one callable per gathered operand) and raises its flag.  On a real
    mesh that stream is the collective's."""
    ready = torch.zeros(K + 1, dtype=torch.int32, device=dev)
    lib = local_gemm._lib.load()
    cur = torch.cuda.current_stream(dev)
    gather = _gather_streams.setdefault(dev, torch.cuda.Stream(dev))
    gather.wait_stream(cur)                              # the flags are cleared and the shards are there
    try:
        lib.ms_set_reserved_cus(OVERLAP_RESERVED_CUS)
        out = launch(ready)
    finally:
        lib.ms_set_reserved_cus(0)
    with torch.cuda.stream(gather):
        for k in range(K):
            for fill in fills:
                fill(k)
            local_gemm.signal_set(ready, k)
    cur.wait_stream(gather)
    if local_gemm.gate_timed_out(ready):
        raise local_gemm._lib.MeshSliceError("the gated product gave up waiting for a slice: the gathers did not run beside it")
    return out


def MeshFlow_OS_overlap(X, W, i, j, R, C, K, B):
    """MeshFlow_OS in the order the reference's schedule runs it (:163-171): the product is launched once, before any
    slice has arrived, and multiplies slice k while the gathers of the later slices are still under way
    (``gemm_os_gated``).  The emulated gather stream fills slice k of both operands, peer by peer, and raises flag k.
    Same result as MeshFlow_OS, bit for bit."""
    if K == 1:
        raise ValueError("the sliced OS body is undefined for K == 1 (the reference adds slice 0 twice); "
                         "use algorithm='collective' for the unsliced product")
    bufA, fillA = _col_slice_filler([X[i][jj] for jj in range(C)], K, B)
    bufB, fillB = _row_slice_filler([W[ii][j] for ii in range(R)], K, B)
    return _launch_ahead_of_gathers(K, bufA.device, lambda ready: local_gemm.gemm_os_gated([bufA[k] for k in range(K)], [bufB[k] for k in range(K)], ready),
                                    (fillA, fillB))


def MeshFlow_LS_overlap(X, W, i, j, R, C, K, B):
    """MeshFlow_LS with the one launch ahead of the gathers of W's row slices (:176-189; ``gemm_ls_gated``): chunk k is
    multiplied as soon as slice k has arrived.  Same chunks as MeshFlow_LS, bit for bit."""
    bufW, fillW = _row_slice_filler([W[ii][j] for ii in range(R)], K, B)
    own = _own(X[i][j])
    return _launch_ahead_of_gathers(K, bufW.device, lambda ready: local_gemm.gemm_ls_gated(own, [bufW[k] for k in range(K)], ready), (fillW,))


def MeshFlow_RS_overlap(X, W, i, j, R, C, K, B):
    """MeshFlow_RS with the one launch ahead of the gathers of X's column slices (:198-212; ``gemm_rs_gated``)."""
    bufX, fillX = _col_slice_filler([X[i][jj] for jj in range(C)], K, B)
    own = _own(W[i][j])
    return _launch_ahead_of_gathers(K, bufX.device, lambda ready: local_gemm.gemm_rs_gated([bufX[k] for k in range(K)], own, ready), (fillX,))


def MeshFlow_LS(X, W, i, j, R, C, K, B):
    """reference :174-193: K gathered row slices of W; K fp32 partial chunks X_ij @ W_k^T."""
    W_slices = _gather_row_slices([W[ii][j] for ii in range(R)], K, B)
    return local_gemm.gemm_ls(_own(X[i][j]), W_slices)


def MeshFlow_RS(X, W, i, j, R, C, K, B):
    """reference :195-214: K gathered column slices of X; K fp32 partial chunks X_k^T @ W_ij."""
    X_slices = _gather_col_slices([X[i][jj] for jj in range(C)], K, B)
    return local_gemm.gemm_rs(X_slices, _own(W[i][j]))


# ------------------------------------------------------------------------------------------------
# ring baselines.  In the reference the halves of one operand (or of the partial output) travel round a
# mesh axis with ppermute, one hop per step, and each step multiplies two half-blocks (Wang_OS/LS/RS,
# reference :34-149; Cannon_OS/LS/RS, :218-342).  Seen from one device that is the same local
# contraction as the unsliced body, cut into 2 * size half-blocks taken in the order of their arrival:
# one kernel call with 2 * size slices (OS) or 2 * size chunks written to their places in the device's
# partial output (LS / RS).  The reference reads the device's ring position with ``jax.lax.ax_index``,
# a name JAX does not have; the position is taken here as ``axis_index`` gives it.
# ------------------------------------------------------------------------------------------------

def _ring_order(algorithm: str, dataflow: str, R: int, C: int, i: int, j: int):
    """[(block, half)] in step order for device (i, j).  Wang: ring = the mesh row; the low halves come from
    the left (block j, j-1, ..), the high halves from the right (j, j+1, ..); for LS the partial outputs
    travel instead and a device works on block j-1-t / j+1+t in step t (reference :45-59, :76-89,
    :132-146).  Cannon (square mesh): both start at k = (i + j) % N, low halves move on to k+1, k+2, ..,
    high halves to k-1, k-2, .. (:235-259, :268-294, :309-335)."""
    if algorithm == "wang":
        if dataflow == "ls":
            return [p for t in range(C) for p in (((j - 1 - t) % C, 0), ((j + 1 + t) % C, 1))]
        return [p for t in range(C) for p in (((j - t) % C, 0), ((j + t) % C, 1))]
    k = (i + j) % C
    return [p for t in range(C) for p in (((k + t) % C, 0), ((k - t) % C, 1))]


def _usable(views: Sequence[torch.Tensor]) -> List[torch.Tensor]:
    """The views themselves if the kernels can address all of them in place, else contiguous copies of all
    (slices of one call share a leading dimension)."""
    if all(_own(v) is v for v in views):
        return list(views)
    return [v.contiguous() for v in views]


def _ring_os(algorithm, X, W, i, j, R, C):
    Wj = _gather([W[ii][j] for ii in range(R)], 0)                       # [Kd, n/C]
    _need(X[i][j].shape[1], 2, "columns of an X shard"); _need(Wj.shape[0], 2 * C, "gathered rows of W")
    h = Wj.shape[0] // C // 2
    order = _ring_order(algorithm, "os", R, C, i, j)
    A = _usable([X[i][b][:, hi * h:(hi + 1) * h] for b, hi in order])
    Bs = [Wj[(2 * b + hi) * h:(2 * b + hi + 1) * h] for b, hi in order]
    return local_gemm.gemm_os(A, Bs)


def _ring_ls(algorithm, X, W, i, j, R, C):
    Wj = _gather([W[ii][j] for ii in range(R)], 0)                       # [O, I/C]
    _need(Wj.shape[0], 2 * C, "gathered rows of W")
    h = Wj.shape[0] // C // 2
    order = _ring_order(algorithm, "ls", R, C, i, j)
    Xij = _own(X[i][j])
    part = torch.empty((Xij.shape[0], Wj.shape[0]), dtype=torch.float32, device=Xij.device)
    outs = [part[:, (2 * b + hi) * h:(2 * b + hi + 1) * h] for b, hi in order]
    if any(o.data_ptr() % 16 for o in outs):
        raise ValueError(f"half-blocks of {h} output columns are not 16-byte aligned")
    local_gemm.gemm_ls(Xij, [Wj[(2 * b + hi) * h:(2 * b + hi + 1) * h] for b, hi in order], out=outs)
    return [part]


def _ring_rs(algorithm, X, W, i, j, R, C):
    _need(X[i][j].shape[1], 2, "columns of an X shard")
    h = X[i][j].shape[1] // 2
    order = _ring_order(algorithm, "rs", R, C, i, j)
    Xs = _usable([X[i][b][:, hi * h:(hi + 1) * h] for b, hi in order])
    Wij = _own(W[i][j])
    part = torch.empty((2 * h * C, Wij.shape[1]), dtype=torch.float32, device=Wij.device)
    local_gemm.gemm_rs(Xs, Wij, out=[part[(2 * b + hi) * h:(2 * b + hi + 1) * h] for b, hi in order])
    return [part]


def Wang_OS(X, W, i, j, R, C, K, B):
    """reference :34-61."""
    return _ring_os("wang", X, W, i, j, R, C)


def Wang_LS(X, W, i, j, R, C, K, B):
    """reference :64-90; returns the device's whole partial output ``X_ij @ Wj^T`` (what the travelling
    half-blocks sum up over the mesh row)."""
    return _ring_ls("wang", X, W, i, j, R, C)


def Wang_RS(X, W, i, j, R, C, K, B):
    """reference :92-149 (the branch it takes, :120-149); returns the device's partial ``Xi^T @ W_ij``."""
    return _ring_rs("wang", X, W, i, j, R, C)


def Cannon_OS(X, W, i, j, R, C, K, B):
    """reference :218-260."""
    return _ring_os("cannon", X, W, i, j, R, C)


def Cannon_LS(X, W, i, j, R, C, K, B):
    """reference :262-300."""
    return _ring_ls("cannon", X, W, i, j, R, C)


def Cannon_RS(X, W, i, j, R, C, K, B):
    """reference :379-417 (the definition in force: it shadows the one at :302-342, which computes the same product)."""
    return _ring_rs("cannon", X, W, i, j, R, C)


# ------------------------------------------------------------------------------------------------
# mesh completion: what psum_scatter + the (.., K, B) interleave do with the partial chunks
# ------------------------------------------------------------------------------------------------

def _block(extent: int, B: int) -> int:
    """Largest block size <= B (a power of two) in which ``extent`` divides: the unsliced bodies have no block size of
    their own, and a window of any width is a whole number of blocks of 1."""
    while B > 1 and extent % B:
        B //= 2
    return max(B, 1)


def _finish(chunks_by_peer, me, axis, B, dtype):
    """psum_scatter over the peers (device ``me`` of them keeps its window of every summed chunk) and the
    interleave of the K windows into the output shard: reference :182-193 (LS: peers = the mesh row,
    axis 1) and :204-214 (RS: peers = the mesh column, axis 0); with one chunk per peer it is the tiled scatter of
    the unsliced bodies (:27, :32).  One layout kernel; the sum is fp32 in peer order with one rounding to ``dtype``.
    More than 64 chunk pointers (P * K) do not fit one launch: the peers are then summed group by group into fp32
    shards, and one more launch adds those up and rounds."""
    P, K = len(chunks_by_peer), len(chunks_by_peer[0])
    if P * K <= 64:
        return slice_layout.unpack_chunks(chunks_by_peer, B, axis, window=me, parts=P, out_dtype=dtype)
    g = max(1, 64 // K)
    partial = [slice_layout.unpack_chunks(chunks_by_peer[p0:p0 + g], B, axis, window=me, parts=P, out_dtype=torch.float32)
               for p0 in range(0, P, g)]
    width = partial[0].shape[1] if axis == 1 else partial[0].shape[0]
    return slice_layout.unpack_chunks([[t] for t in partial], _block(width, 8), axis, window=0, parts=1, out_dtype=dtype)


class ShardedMatmul:
    """What ``SPMD.OS/LS/RS(K)`` returns: ``f(X, W) -> Y`` on global operands, plus ``f.device(i, j)``."""

    def __init__(self, dataflow: str, body: Callable, mesh: Mesh, K: int, B: int, sliced: bool):
        self.dataflow, self.body, self.mesh, self.K, self.B, self.sliced = dataflow, body, mesh, int(K), int(B), sliced
        self.R, self.C = mesh.shape

    # shape rules implied by the reference's reshapes (:155-156,177-179,198-200)
    def _validate(self, X: torch.Tensor, W: torch.Tensor) -> None:
        R, C = self.R, self.C
        S = self.K if self.sliced else 1
        B = self.B if self.sliced else 1
        if S < 1:
            raise ValueError(f"slice count must be >= 1, got {S}")
        for t, name in ((X, "X"), (W, "W")):
            if not isinstance(t, torch.Tensor) or t.dim() != 2:
                raise ValueError(f"{name} must be a 2-D torch tensor")
        if X.dtype != W.dtype:
            raise ValueError("X and W must share a dtype")
        if self.dataflow == "os":
            if X.shape[1] != W.shape[0]:
                raise ValueError(f"os: cannot contract {tuple(X.shape)} @ {tuple(W.shape)}")
            _need(X.shape[0], R, "rows of X"); _need(W.shape[1], C, "cols of W")
            _need(X.shape[1], C * S * B, "cols of X"); _need(W.shape[0], R * S * B, "rows of W")
        elif self.dataflow == "ls":
            if X.shape[1] != W.shape[1]:
                raise ValueError(f"ls: cannot contract {tuple(X.shape)} @ {tuple(W.shape)}^T")
            _need(X.shape[0], R, "rows of X"); _need(X.shape[1], C, "cols of X")
            _need(W.shape[0], R * S * B, "rows of W"); _need(W.shape[0], C * S * B, "rows of W")
        else:
            if X.shape[0] != W.shape[0]:
                raise ValueError(f"rs: cannot contract {tuple(X.shape)}^T @ {tuple(W.shape)}")
            _need(X.shape[0], R, "rows of X"); _need(W.shape[1], C, "cols of W")
            _need(X.shape[1], C * S * B, "cols of X"); _need(X.shape[1], R * S * B, "cols of X")
        for t, name in ((X, "X"), (W, "W")):
            if not t.is_cuda:
                raise local_gemm._lib.MeshSliceError(f"{name} must live on the GPU: there is no CPU path")

    def device(self, i: int, j: int) -> Callable:
        """Body of mesh device (i, j): returns its output block (OS) or its fp32 partial chunks."""
        if not (0 <= i < self.R and 0 <= j < self.C):
            raise ValueError(f"device ({i},{j}) is outside the {self.R}x{self.C} mesh")

        def run(X, W):
            self._validate(X, W)
            return self.body(_shards(X, self.R, self.C), _shards(W, self.R, self.C), i, j, self.R, self.C, self.K, self.B)
        return run

    def __call__(self, X: torch.Tensor, W: torch.Tensor) -> torch.Tensor:
        self._validate(X, W)
        R, C = self.R, self.C
        K = self.K if self.sliced else 1
        B = self.B if self.sliced else 1
        Xs, Ws = _shards(X, R, C), _shards(W, R, C)
        run = lambda i, j: self.body(Xs, Ws, i, j, R, C, self.K, self.B)
        if self.dataflow == "os":
            return torch.cat([torch.cat([run(i, j) for j in range(C)], dim=1) for i in range(R)], dim=0)
        if self.dataflow == "ls":
            rows = []
            for i in range(R):
                chunks = [run(i, j) for j in range(C)]
                # (unsliced bodies bring one chunk each: the tiled scatter of contiguous column blocks)
                Bw = B if self.sliced else _block(chunks[0][0].shape[1] // C, 8)
                rows.append(torch.cat([_finish(chunks, j, 1, Bw, X.dtype) for j in range(C)], dim=1))
            return torch.cat(rows, dim=0)
        cols = []
        for j in range(C):
            chunks = [run(i, j) for i in range(R)]
            Bw = B if self.sliced else _block(chunks[0][0].shape[0] // R, 8)
            cols.append(torch.cat([_finish(chunks, i, 0, Bw, X.dtype) for i in range(R)], dim=0))
        return torch.cat(cols, dim=1)


class SPMD:
    """reference TensorParallel.py:346-377.  ``jit`` is accepted and ignored: kernels are ahead-of-time
    compiled."""

    def __init__(self, mesh: Mesh, algorithm: str = "collective", blocksize: int = 8, jit: bool = True):
        self.mesh = mesh
        self.rowaxis = mesh.axis_names[0]
        self.colaxis = mesh.axis_names[1]
        self.spec = P(self.rowaxis, self.colaxis)
        self.blocksize = blocksize
        self.jit = jit
        self.algorithm = algorithm
        if algorithm == "collective":
            self.funcs = {"os": Collective_OS, "ls": Collective_LS, "rs": Collective_RS}
            self.sliced = False
        elif algorithm == "wang":
            self.funcs = {"os": Wang_OS, "ls": Wang_LS, "rs": Wang_RS}
            self.sliced = False
        elif algorithm == "cannon":
            assert mesh.devices.shape[0] == mesh.devices.shape[1], "cannon needs a square mesh"
            self.funcs = {"os": Cannon_OS, "ls": Cannon_LS, "rs": Cannon_RS}
            self.sliced = False
        elif algorithm == "meshflow_overlap":      # MeshFlow with each device's one product launched ahead of its gathers
            self.funcs = {"os": MeshFlow_OS_overlap, "ls": MeshFlow_LS_overlap, "rs": MeshFlow_RS_overlap}
            self.sliced = True
        else:  # like the reference, any other name selects the sliced MeshFlow bodies
            self.funcs = {"os": MeshFlow_OS, "ls": MeshFlow_LS, "rs": MeshFlow_RS}
            self.sliced = True

    def _build(self, which: str, K: int) -> ShardedMatmul:
        if int(K) < 1:
            raise ValueError(f"slice count K must be >= 1, got {K}")
        return ShardedMatmul(which, self.funcs[which], self.mesh, K, self.blocksize, self.sliced)

    def OS(self, K: int = 8) -> ShardedMatmul:
        return self._build("os", K)

    def LS(self, K: int = 8) -> ShardedMatmul:
        return self._build("ls", K)

    def RS(self, K: int = 8) -> ShardedMatmul:
        return self._build("rs", K)


def createMultihostMatrix(mesh: Mesh, sharding, global_shape, dtype=torch.bfloat16, seed: int = 0, device="cuda"):
    """reference :419-423: a random N(0,1) matrix of ``global_shape`` sharded over the mesh.  The
    reference seeds JAX's generator with the process index; this build has one process and uses
    torch's generator with ``seed`` (the sample streams differ; nothing depends on them)."""
    g = torch.Generator(device="cpu").manual_seed(int(seed))
    return torch.randn(tuple(global_shape), generator=g, dtype=torch.float32).to(dtype).to(device)
