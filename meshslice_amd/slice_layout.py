"""Block-cyclic slices and chunks on torch device tensors: the data movement either side of the local
contraction, done by the HIP kernels of libmeshslice_hip.so (``ms_pack_slices``, ``ms_unpack_chunks``).

``pack_slices`` is what a mesh device does to its shard before the all-gathers of a sliced dataflow: the
``(.., L/(S*B), S, B)`` view and the ``dynamic_slice_in_dim`` along the S axis of reference
TensorParallel.py:155-158, :177-178, :198-199, for all S slices in one pass.  ``unpack_chunks`` is what it
does with the chunks afterwards: ``psum_scatter`` (:182,188,204,210), ``dynamic_update_slice_in_dim`` into
the ``(.., S, B)`` view (:184,190,206,211) and the final reshape (:193,:214).
"""
from __future__ import annotations

import ctypes
from typing import List, Optional, Sequence

import torch

from . import _lib
from .local_gemm import _check2d, _dt, _same, _stream


def pack_slices(block: torch.Tensor, S: int, B: int, axis: int,
                out: Optional[Sequence[torch.Tensor]] = None) -> List[torch.Tensor]:
    """The S block-cyclic slices of ``block`` along ``axis`` (1 = columns, 0 = rows): slice s holds the
    B-wide blocks ``b`` with ``b % S == s`` in ascending order.  ``out`` may be S row-major views into a
    larger buffer (for example a peer's place in a gathered slice); they share one leading dimension."""
    _check2d(block, "block")
    if axis not in (0, 1):
        raise ValueError("axis must be 0 or 1")
    S, B = int(S), int(B)
    r, c = block.shape
    if S < 1 or B < 1 or (c if axis == 1 else r) % (S * B):
        raise ValueError(f"sliced extent {c if axis == 1 else r} is not a multiple of S*B = {S}*{B}")
    shape = (r, c // S) if axis == 1 else (r // S, c)
    if out is None:
        buf = torch.empty((S,) + shape, dtype=block.dtype, device=block.device)
        out = [buf[s] for s in range(S)]
    o0 = _same(out, "out")
    if len(out) != S or tuple(o0.shape) != shape or o0.dtype != block.dtype or o0.device != block.device:
        raise ValueError(f"out must be S slices of shape {shape} and the dtype of block")
    pd, _kd = _lib.ptr_array([t.data_ptr() for t in out])
    with torch.cuda.device(block.device):
        rc = _lib.load().ms_pack_slices(ctypes.c_void_p(block.data_ptr()), block.stride(0), r, c, axis, S, B,
                                        pd, o0.stride(0), _dt(block), _stream())
    _lib.check(rc)
    return list(out)


def unpack_chunks(chunks_by_peer: Sequence[Sequence[torch.Tensor]], B: int, axis: int,
                  window: int = 0, parts: int = 1, out: Optional[torch.Tensor] = None,
                  out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """A device's output shard from partial chunks: ``chunks_by_peer[p][s]`` is peer p's chunk s (all of one
    shape).  Along ``axis`` every chunk is cut into ``parts`` equal windows of which this device keeps number
    ``window`` (what a tiled ``psum_scatter`` over ``parts`` devices hands to device ``window``); the
    windows are summed over the peers in fp32, rounded once to ``out_dtype`` and interleaved: block ``h`` of
    chunk ``s`` lands at block ``h * S + s`` of the output."""
    P = len(chunks_by_peer)
    if P < 1:
        raise ValueError("need at least one peer's chunks")
    S = len(chunks_by_peer[0])
    flat = [t for peer in chunks_by_peer for t in peer]
    if any(len(peer) != S for peer in chunks_by_peer):
        raise ValueError("every peer must bring the same number of chunks")
    c0 = _same(flat, "chunks")
    if axis not in (0, 1):
        raise ValueError("axis must be 0 or 1")
    B, parts, window = int(B), int(parts), int(window)
    cr, cc = c0.shape
    cut = cc if axis == 1 else cr
    if parts < 1 or not 0 <= window < parts or cut % parts or (cut // parts) % B:
        raise ValueError(f"chunk extent {cut} does not split into {parts} windows of whole blocks of {B}")
    keep = cut // parts
    rows, cols = (cr, keep * S) if axis == 1 else (keep * S, cc)
    row_off, col_off = (0, window * keep) if axis == 1 else (window * keep, 0)
    if out is None:
        out = torch.empty((rows, cols), dtype=out_dtype or c0.dtype, device=c0.device)
    _check2d(out, "out")
    if tuple(out.shape) != (rows, cols) or out.device != c0.device or (out_dtype is not None and out.dtype != out_dtype):
        raise ValueError(f"out must be a [{rows}, {cols}] tensor of the requested dtype on the chunks' device")
    pc, _kc = _lib.ptr_array([t.data_ptr() for t in flat])
    with torch.cuda.device(c0.device):
        rc = _lib.load().ms_unpack_chunks(pc, P, S, c0.stride(0), row_off, col_off, rows, cols, axis, B,
                                          ctypes.c_void_p(out.data_ptr()), out.stride(0), _dt(c0), _dt(out), _stream())
    _lib.check(rc)
    return out


def measure_rates(rows: int = 4096, cols: int = 12288, S: int = 8, B: int = 8, reps: int = 48, nset: int = 4,
                  dtypes=(torch.bfloat16, torch.float32), reduce_case: bool = True):
    """Time the layout kernels on [rows, cols] shards (HIP events on the current stream).  Returns a list of
    (label, seconds, algorithmic bytes): bytes read once + bytes written once.  Launches rotate over ``nset``
    separate source / destination sets, together larger than the 256 MB last-level cache, so that every launch
    streams from and to HBM."""
    def timed(f):
        for i in range(2 * nset):
            f(i % nset)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize(); e0.record()
        for i in range(reps):
            f(i % nset)
        e1.record(); torch.cuda.synchronize()
        return e0.elapsed_time(e1) / reps * 1e-3

    out = []
    for dtype in dtypes:
        name = str(dtype)[6:]
        xs = [torch.randn(rows, cols, device="cuda").to(dtype) for _ in range(nset)]
        ys = [torch.empty_like(x) for x in xs]
        nbytes = 2 * xs[0].numel() * xs[0].element_size()
        out.append((f"{name} device copy of the shard", timed(lambda i: ys[i].copy_(xs[i])), nbytes))
        for axis in (1, 0):
            slices = [pack_slices(x, S, B, axis) for x in xs]
            out.append((f"{name} pack axis {axis} S={S}", timed(lambda i: pack_slices(xs[i], S, B, axis, out=slices[i])), nbytes))
            out.append((f"{name} unpack axis {axis} S={S} P=1", timed(lambda i: unpack_chunks([slices[i]], B, axis, out=ys[i])), nbytes))
        del xs, ys, slices
    if reduce_case:
        # what follows the LHS-stationary GEMM of the large configuration on a 4-wide mesh row: 4 peers' S fp32
        # chunks [rows, cols / S], this device keeps a quarter of each, bf16 shard out
        peers = [[[torch.randn(rows, cols // S, device="cuda") for _ in range(S)] for _ in range(4)] for _ in range(2)]
        y = torch.empty(rows, cols // 4, dtype=torch.bfloat16, device="cuda")
        nbytes = 4 * S * rows * (cols // S // 4) * 4 + y.numel() * 2
        out.append((f"fp32->bf16 reduce 4 peers + unpack axis 1 S={S}", timed(lambda i: unpack_chunks(peers[i % 2], B, 1, window=1, parts=4, out=y)), nbytes))
    return out


if __name__ == "__main__":
    # python -m meshslice_amd.slice_layout: microseconds and algorithmic GB/s of every layout kernel
    for label, t, nbytes in measure_rates():
        print(f"{label:48s} {t * 1e6:7.1f} us {nbytes / t / 1e9:7.0f} GB/s", flush=True)
