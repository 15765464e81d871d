"""The per-device local contraction of the three dataflows on torch device tensors.

These functions are what the per-device bodies in TensorParallel.py call where the reference calls
``jnp.einsum`` / ``@`` (reference TensorParallel.py:22,26,31,162,167,172,181,187,203,209).  torch is
used only to own device memory and to name the current stream; all arithmetic happens in
libmeshslice_hip.so.
"""
from __future__ import annotations

import ctypes
import threading
from typing import List, Optional, Sequence

import torch

from . import _lib

_DT = {torch.float32: _lib.MS_DTYPE_F32, torch.bfloat16: _lib.MS_DTYPE_BF16}


def _dt(t: torch.Tensor) -> int:
    if t.dtype not in _DT:
        raise TypeError(f"unsupported dtype {t.dtype}: the local GEMM takes float32 or bfloat16")
    return _DT[t.dtype]


def _check2d(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise _lib.MeshSliceError(f"{name} is not on the GPU: the local GEMM has no CPU path")
    if t.dim() != 2 or t.stride(1) != 1:
        raise ValueError(f"{name} must be a row-major 2-D tensor (got shape {tuple(t.shape)}, strides {t.stride()})")


def _stream() -> ctypes.c_void_p:
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _same(ts: Sequence[torch.Tensor], name: str):
    if len(ts) < 1:
        raise ValueError(f"{name}: need at least one slice")
    s0 = ts[0]
    for t in ts:
        _check2d(t, name)
        if t.shape != s0.shape or t.dtype != s0.dtype or t.stride(0) != s0.stride(0) or t.device != s0.device:
            raise ValueError(f"{name}: all slices must share shape, dtype, leading dimension and device")
    return s0


_workspaces = {}            # (device index, stream handle) -> uint8 tensor, least recently used first
_workspaces_lock = threading.Lock()
_WORKSPACE_CACHE_MAX = 8      # streams per device that keep a workspace of their own (about 100 MB each)


def workspace(device, stream=None) -> torch.Tensor:
    """The split-contraction workspace of ``(device, stream)`` (a uint8 tensor of ``ms_workspace_bytes()`` bytes,
    allocated and prepared with ``ms_workspace_init`` on first use, then kept): ``gemm_os`` hands it to
    ``ms_gemm_os_ws`` so that products with few output tiles can spread their contraction over the idle compute units.

    Calls that share a workspace must not overlap on the device (they share its arrival counters and partial tiles).
    Work on ONE stream never overlaps, so every stream gets a workspace of its own (``stream`` defaults to the current
    one): calls issued from several host threads or on several streams cannot meet in one.  At most
    ``_WORKSPACE_CACHE_MAX`` streams per device keep one; a further stream evicts the least recently used, after
    waiting for the device to finish what is queued (the evicted stream may still be running a product on it).

    While a ``torch.cuda.graph`` capture is under way on the current stream the workspace is allocated inside the capture
    (from the graph's own memory pool, so it lives as long as the graph and later captured calls of the same graph
    reuse it), prepared by a captured fill kernel and not kept here: a graph's replays never share counters with eager
    calls or with another graph's."""
    device = torch.device(device)
    idx = device.index if device.index is not None else torch.cuda.current_device()
    if stream is None:
        stream = torch.cuda.current_stream(idx)
    key = (idx, int(stream.cuda_stream))
    capturing = torch.cuda.is_current_stream_capturing()
    if not capturing:
        with _workspaces_lock:
            ws = _workspaces.pop(key, None)
            if ws is not None:
                _workspaces[key] = ws      # most recently used last
                return ws
    lib = _lib.load()
    with torch.cuda.device(idx), torch.cuda.stream(stream):
        nbytes = int(lib.ms_workspace_bytes())
        if nbytes <= 0:
            raise _lib.MeshSliceError("could not size the workspace: " + _lib.last_error())
        ws = torch.empty(nbytes, dtype=torch.uint8, device=torch.device("cuda", idx))
        _lib.check(lib.ms_workspace_init(ctypes.c_void_p(ws.data_ptr()), nbytes, ctypes.c_void_p(stream.cuda_stream)))
    if capturing:
        return ws
    with _workspaces_lock:
        have = _workspaces.setdefault(key, ws)      # (another thread on the same stream may have been faster)
        mine = [k for k in _workspaces if k[0] == idx and k != key]
        evicted = [_workspaces.pop(k) for k in mine[:max(0, len(mine) + 1 - _WORKSPACE_CACHE_MAX)]]
    if evicted:
        torch.cuda.synchronize(idx)     # their streams may still be running products that use them
        del evicted
    return have


def _ws_args(device):
    """(pointer, bytes, tensor): the caller keeps the tensor until its call has been issued"""
    ws = workspace(device)
    return ctypes.c_void_p(ws.data_ptr()), ws.numel(), ws


class _Call:
    """One validated local contraction: the C entry points' argument list up to (not including) ``stream``,
    the device it runs on, the output it writes and the Python objects that keep the pointer tables alive."""

    def __init__(self, device, args, out, keep):
        self.device, self.args, self.out, self.keep = device, args, out, keep


def _prepare_os(A_slices, B_slices, out, out_dtype) -> _Call:
    a0 = _same(A_slices, "A_slices"); b0 = _same(B_slices, "B_slices")
    if len(A_slices) != len(B_slices):
        raise ValueError("A_slices and B_slices differ in length")
    if a0.shape[1] != b0.shape[0] or a0.dtype != b0.dtype or a0.device != b0.device:
        raise ValueError(f"slice shapes do not contract: {tuple(a0.shape)} @ {tuple(b0.shape)}")
    m, k = a0.shape; n = b0.shape[1]
    if out is None:
        out = torch.empty((m, n), dtype=out_dtype or a0.dtype, device=a0.device)
    _check2d(out, "out")
    if tuple(out.shape) != (m, n) or out.device != a0.device:
        raise ValueError("out has the wrong shape or device")
    pa, _ka = _lib.ptr_array([t.data_ptr() for t in A_slices])
    pb, _kb = _lib.ptr_array([t.data_ptr() for t in B_slices])
    args = (pa, pb, len(A_slices), m, n, k, a0.stride(0), b0.stride(0),
            ctypes.c_void_p(out.data_ptr()), out.stride(0), _dt(a0), _dt(out))
    return _Call(a0.device, args, out, (_ka, _kb))


def _prepare_ls(A, W_slices, out, out_dtype) -> _Call:
    _check2d(A, "A"); w0 = _same(W_slices, "W_slices")
    if A.shape[1] != w0.shape[1] or A.dtype != w0.dtype or A.device != w0.device:
        raise ValueError(f"shapes do not contract: {tuple(A.shape)} @ {tuple(w0.shape)}^T")
    m, k = A.shape; ns = w0.shape[0]; S = len(W_slices)
    dt = _chunk_dtype(out, out_dtype)
    if out is None:
        buf = torch.empty((S, m, ns), dtype=dt, device=A.device)
        out = [buf[s] for s in range(S)]
    o0 = _same(out, "out")
    if len(out) != S or tuple(o0.shape) != (m, ns) or o0.dtype not in (torch.float32, torch.bfloat16) or o0.device != A.device:
        raise ValueError("out must be S fp32 or bf16 chunks of shape [m, n_slice] on the operands' device")
    pw, _kw = _lib.ptr_array([t.data_ptr() for t in W_slices])
    py, _ky = _lib.ptr_array([t.data_ptr() for t in out])
    args = (ctypes.c_void_p(A.data_ptr()), A.stride(0), pw, w0.stride(0), S, m, ns, k, py, o0.stride(0), _dt(A), _dt(o0))
    return _Call(A.device, args, list(out), (_kw, _ky))


def _prepare_rs(X_slices, W, out, out_dtype) -> _Call:
    _check2d(W, "W"); x0 = _same(X_slices, "X_slices")
    if x0.shape[0] != W.shape[0] or x0.dtype != W.dtype or x0.device != W.device:
        raise ValueError(f"shapes do not contract: {tuple(x0.shape)}^T @ {tuple(W.shape)}")
    k, ms = x0.shape; n = W.shape[1]; S = len(X_slices)
    dt = _chunk_dtype(out, out_dtype)
    if out is None:
        buf = torch.empty((S, ms, n), dtype=dt, device=W.device)
        out = [buf[s] for s in range(S)]
    o0 = _same(out, "out")
    if len(out) != S or tuple(o0.shape) != (ms, n) or o0.dtype not in (torch.float32, torch.bfloat16) or o0.device != W.device:
        raise ValueError("out must be S fp32 or bf16 chunks of shape [m_slice, n] on the operands' device")
    px, _kx = _lib.ptr_array([t.data_ptr() for t in X_slices])
    py, _ky = _lib.ptr_array([t.data_ptr() for t in out])
    args = (px, x0.stride(0), ctypes.c_void_p(W.data_ptr()), W.stride(0), S, ms, n, k, py, o0.stride(0), _dt(W), _dt(o0))
    return _Call(W.device, args, list(out), (_kx, _ky))


def gemm_os(A_slices: Sequence[torch.Tensor], B_slices: Sequence[torch.Tensor],
            out: Optional[torch.Tensor] = None, out_dtype: Optional[torch.dtype] = None,
            activation: Optional[str] = None, residual: Optional[torch.Tensor] = None,
            row_moments=None) -> torch.Tensor:
    """``C = sum_s A_s @ B_s`` with fp32 accumulation over all slices, rounded once.

    Optional fused epilogue (bf16 operands): ``C = act(sum) + residual`` with ``activation='gelu'`` (tanh
    form) and ``residual`` of C's shape and dtype; ``row_moments=(row_sum, row_sumsq)`` are fp32 vectors of
    length m (either may be None) to which the row sums / sums of squares of the fp32 result are ADDED."""
    call = _prepare_os(A_slices, B_slices, out, out_dtype)
    out = call.out
    m, n = out.shape
    if activation not in (None, "gelu"):
        raise ValueError(f"unknown activation {activation!r} (None or 'gelu')")
    res_ptr, ldr = None, 0
    if residual is not None:
        _check2d(residual, "residual")
        if tuple(residual.shape) != (m, n) or residual.dtype != out.dtype or residual.device != out.device:
            raise ValueError("residual must have the shape, dtype and device of the output")
        res_ptr, ldr = ctypes.c_void_p(residual.data_ptr()), residual.stride(0)
    moments = [None, None]
    for idx, t in enumerate(row_moments or (None, None)):
        if t is not None:
            if not (t.is_cuda and t.dtype == torch.float32 and t.dim() == 1 and t.numel() == m and t.is_contiguous()
                    and t.device == out.device):
                raise ValueError("row moments must be contiguous fp32 GPU vectors of length m on the output's device")
            moments[idx] = ctypes.c_void_p(t.data_ptr())
    ws_ptr, ws_bytes, _ws_keep = _ws_args(call.device)
    with torch.cuda.device(call.device):
        rc = _lib.load().ms_gemm_os_ws(*call.args,
                                       _lib.MS_ACT_GELU if activation == "gelu" else _lib.MS_ACT_NONE,
                                       res_ptr, ldr, moments[0], moments[1], ws_ptr, ws_bytes, _stream())
    _lib.check(rc)
    return out


def _chunk_dtype(out, out_dtype):
    """dtype of the LS / RS chunks: that of ``out`` if given, else ``out_dtype``, else fp32."""
    if out is not None and len(out) > 0:
        if out_dtype is not None and out[0].dtype != out_dtype:
            raise ValueError("out_dtype contradicts the dtype of out")
        return out[0].dtype
    dt = torch.float32 if out_dtype is None else out_dtype
    if dt not in (torch.float32, torch.bfloat16):
        raise ValueError("chunks are fp32 or bf16")
    return dt


def gemm_os_gated(A_slices: Sequence[torch.Tensor], B_slices: Sequence[torch.Tensor], slice_ready: torch.Tensor,
                  out: Optional[torch.Tensor] = None, out_dtype: Optional[torch.dtype] = None,
                  timeout_ms: int = 2000) -> torch.Tensor:
    """gemm_os as ONE launch that may be enqueued before its slices have arrived (``ms_gemm_os_gated``): the kernel
    reads slice s of A and of B only after ``slice_ready[s]`` has become non-zero, the way the reference's
    output-stationary body multiplies slice k while slice k + 1 is still being gathered (MeshFlow_OS,
    TensorParallel.py:163-171).  ``slice_ready`` is an int32 GPU tensor of S + 1 words: the flags (set them with
    ``signal_set`` on the stream that fills the slice, after the fill) and, last, a status word that must be zero before
    the call and reads 1 afterwards if a wait lasted longer than ``timeout_ms`` (the result is then void: check it with
    ``gate_timed_out`` once the stream has been synchronised).  A producer that needs compute units of this device
    only runs beside the waiting product when units have been reserved (``ms_set_reserved_cus``)."""
    call = _prepare_os(A_slices, B_slices, out, out_dtype)
    _check_flags(slice_ready, len(A_slices), call.device)
    ws_ptr, ws_bytes, _ws_keep = _ws_args(call.device)
    with torch.cuda.device(call.device):
        rc = _lib.load().ms_gemm_os_gated(*call.args, ws_ptr, ws_bytes, ctypes.c_void_p(slice_ready.data_ptr()),
                                          int(timeout_ms), _stream())
    _lib.check(rc)
    return call.out


def _check_flags(slice_ready, S, device):
    if not (isinstance(slice_ready, torch.Tensor) and slice_ready.is_cuda and slice_ready.dtype == torch.int32
            and slice_ready.dim() == 1 and slice_ready.numel() == S + 1 and slice_ready.is_contiguous()
            and slice_ready.device == device):
        raise ValueError("slice_ready must be a contiguous int32 GPU tensor of S + 1 words on the operands' device")


def _chunks_gated(entry, call, S, slice_ready, chunk_done, timeout_ms):
    _check_flags(slice_ready, S, call.device)
    tiles = ctypes.c_int(0)
    if chunk_done is not None:
        _check_counters(chunk_done, S, call.device)
    with torch.cuda.device(call.device):
        rc = entry(*call.args, ctypes.c_void_p(chunk_done.data_ptr()) if chunk_done is not None else None,
                   ctypes.byref(tiles) if chunk_done is not None else None,
                   ctypes.c_void_p(slice_ready.data_ptr()), int(timeout_ms), _stream())
    _lib.check(rc)
    return call.out if chunk_done is None else (call.out, tiles.value)


def gemm_ls_gated(A: torch.Tensor, W_slices: Sequence[torch.Tensor], slice_ready: torch.Tensor,
                  out: Optional[List[torch.Tensor]] = None, out_dtype: Optional[torch.dtype] = None,
                  chunk_done: Optional[torch.Tensor] = None, timeout_ms: int = 2000):
    """gemm_ls as one launch that may be enqueued before the weight slices have arrived (``ms_gemm_ls_gated``): ``W_s`` is
    read only after ``slice_ready[s]`` has become non-zero (MeshFlow_LS gathers slice k + 1 while chunk k is multiplied,
    TensorParallel.py:176-189); flags, status word and time limit as for ``gemm_os_gated``.  With ``chunk_done`` (see
    ``gemm_ls_signal``) the call also counts finished tiles per chunk and returns ``(chunks, tiles_per_chunk)``."""
    return _chunks_gated(_lib.load().ms_gemm_ls_gated, _prepare_ls(A, W_slices, out, out_dtype), len(W_slices), slice_ready, chunk_done, timeout_ms)


def gemm_rs_gated(X_slices: Sequence[torch.Tensor], W: torch.Tensor, slice_ready: torch.Tensor,
                  out: Optional[List[torch.Tensor]] = None, out_dtype: Optional[torch.dtype] = None,
                  chunk_done: Optional[torch.Tensor] = None, timeout_ms: int = 2000):
    """gemm_rs behind the input gate (``ms_gemm_rs_gated``; see gemm_ls_gated; reference TensorParallel.py:198-212):
    ``X_s`` is read only after ``slice_ready[s]`` has become non-zero."""
    return _chunks_gated(_lib.load().ms_gemm_rs_gated, _prepare_rs(X_slices, W, out, out_dtype), len(X_slices), slice_ready, chunk_done, timeout_ms)


def signal_set(flags: torch.Tensor, index: int, value: int = 1) -> None:
    """``flags[index] = value`` on the current stream, after everything enqueued on it before, as a release at system
    scope (``ms_signal_set``): the producer's half of the gated calls."""
    if not (isinstance(flags, torch.Tensor) and flags.is_cuda and flags.dtype == torch.int32 and flags.dim() == 1 and flags.is_contiguous()):
        raise ValueError("flags must be a contiguous int32 GPU vector")
    if not 0 <= index < flags.numel():
        raise IndexError(f"flag index {index} outside [0, {flags.numel()})")
    with torch.cuda.device(flags.device):
        rc = _lib.load().ms_signal_set(ctypes.c_void_p(flags.data_ptr() + 4 * index), int(value), _stream())
    _lib.check(rc)


def gate_timed_out(slice_ready: torch.Tensor) -> bool:
    """Whether a gated call with these flags gave up waiting for a slice (synchronises with the device)."""
    return bool(slice_ready[-1].item() != 0)


def gemm_ls(A: torch.Tensor, W_slices: Sequence[torch.Tensor],
            out: Optional[List[torch.Tensor]] = None, out_dtype: Optional[torch.dtype] = None) -> List[torch.Tensor]:
    """``Y_s = A @ W_s^T``, W_s stored ``[n_slice, k]``.  Chunks are fp32 by default (exact partial sums for
    the reduce-scatter); ``out_dtype=torch.bfloat16`` gives what the reference's einsum returns for bf16
    operands (TensorParallel.py:181-189): one rounding of the fp32 accumulator, half the bytes."""
    call = _prepare_ls(A, W_slices, out, out_dtype)
    with torch.cuda.device(call.device):
        rc = _lib.load().ms_gemm_ls_ex(*call.args, _stream())
    _lib.check(rc)
    return call.out


def gemm_rs(X_slices: Sequence[torch.Tensor], W: torch.Tensor,
            out: Optional[List[torch.Tensor]] = None, out_dtype: Optional[torch.dtype] = None) -> List[torch.Tensor]:
    """``Y_s = X_s^T @ W``, X_s stored ``[k, m_slice]``; chunks fp32 by default, bf16 on request (see gemm_ls)."""
    call = _prepare_rs(X_slices, W, out, out_dtype)
    with torch.cuda.device(call.device):
        rc = _lib.load().ms_gemm_rs_ex(*call.args, _stream())
    _lib.check(rc)
    return call.out


def _check_counters(chunk_done: torch.Tensor, S: int, device) -> None:
    if not (isinstance(chunk_done, torch.Tensor) and chunk_done.is_cuda and chunk_done.device == device
            and chunk_done.dtype == torch.int32 and chunk_done.is_contiguous() and chunk_done.numel() >= S):
        raise ValueError(f"chunk_done must be a contiguous int32 tensor of at least {S} counters on {device}")


def gemm_ls_signal(A: torch.Tensor, W_slices: Sequence[torch.Tensor], chunk_done: torch.Tensor,
                   out: Optional[List[torch.Tensor]] = None, out_dtype: Optional[torch.dtype] = None):
    """gemm_ls with per-chunk completion counters (``ms_gemm_ls_signal``): the kernel adds 1 to ``chunk_done[s]``
    (int32, zero before the call) after each output tile of ``Y_s`` is in memory, so that the reduce-scatter of chunk
    s (reference TensorParallel.py:182-189) can start before the call has ended.  Returns ``(chunks, tiles_per_chunk)``:
    ``Y_s`` is complete when ``chunk_done[s] == tiles_per_chunk``."""
    call = _prepare_ls(A, W_slices, out, out_dtype)
    _check_counters(chunk_done, len(W_slices), call.device)
    tiles = ctypes.c_int(0)
    with torch.cuda.device(call.device):
        rc = _lib.load().ms_gemm_ls_signal(*call.args, ctypes.c_void_p(chunk_done.data_ptr()), ctypes.byref(tiles), _stream())
    _lib.check(rc)
    return call.out, tiles.value


def gemm_rs_signal(X_slices: Sequence[torch.Tensor], W: torch.Tensor, chunk_done: torch.Tensor,
                   out: Optional[List[torch.Tensor]] = None, out_dtype: Optional[torch.dtype] = None):
    """gemm_rs with per-chunk completion counters (``ms_gemm_rs_signal``, see gemm_ls_signal; reference
    TensorParallel.py:204-212)."""
    call = _prepare_rs(X_slices, W, out, out_dtype)
    _check_counters(chunk_done, len(X_slices), call.device)
    tiles = ctypes.c_int(0)
    with torch.cuda.device(call.device):
        rc = _lib.load().ms_gemm_rs_signal(*call.args, ctypes.c_void_p(chunk_done.data_ptr()), ctypes.byref(tiles), _stream())
    _lib.check(rc)
    return call.out, tiles.value


def time_call(flow: str, operands, out, warmup: int = 5, reps: int = 20) -> List[float]:
    """Per-launch milliseconds (HIP events on the current stream) of one local contraction.

    ``flow`` is 'os', 'ls' or 'rs'; ``operands`` / ``out`` are what gemm_os / gemm_ls / gemm_rs take (``out`` is
    required here) and are checked the same way; LS / RS chunks may be fp32 or bf16."""
    if flow not in ("os", "ls", "rs"):
        raise ValueError(f"unknown dataflow {flow!r}")
    if out is None:
        raise ValueError("time_call needs the output buffer(s)")
    if int(warmup) < 0 or int(reps) < 1:
        raise ValueError("time_call needs warmup >= 0 and reps >= 1")
    first, second = operands
    lib = _lib.load()
    if flow == "os":
        call = _prepare_os(first, second, out, None)
        ms = (ctypes.c_float * int(reps))()
        ws_ptr, ws_bytes, _ws_keep = _ws_args(call.device)
        with torch.cuda.device(call.device):
            rc = lib.ms_time_os_ws(*call.args, ws_ptr, ws_bytes, _stream(), int(warmup), int(reps), ms)
        _lib.check(rc)
        return list(ms)
    elif flow == "ls":
        call, fn = _prepare_ls(first, second, out, None), lib.ms_time_ls_ex
    else:
        call, fn = _prepare_rs(first, second, out, None), lib.ms_time_rs_ex
    ms = (ctypes.c_float * int(reps))()
    with torch.cuda.device(call.device):
        rc = fn(*call.args, _stream(), int(warmup), int(reps), ms)
    _lib.check(rc)
    return list(ms)


def mfma_stream_rate(operands: Optional[torch.Tensor] = None, iters: int = 4000, warmup: int = 20, reps: int = 200,
                     shape: str = "32x32x16", waves_per_simd: int = 1) -> float:
    """FLOP/s that the current GPU sustains on a bare stream of one bf16 MFMA instruction
    (``ms_probe_mfma_stream_ex``): the practical ceiling, under the device's power limit, for the operand data
    given (default: N(0,1) values rounded to bf16, seed 0).  ``shape`` is '32x32x16' (the instruction of the
    big-tile kernels) or '16x16x32'; ``waves_per_simd`` 1 or 2.  ``warmup + reps`` launches of about a
    millisecond each, so the figure is the sustained one."""
    shapes = {"32x32x16": _lib.MS_MFMA_32X32X16, "16x16x32": _lib.MS_MFMA_16X16X32}
    if shape not in shapes:
        raise ValueError(f"unknown MFMA shape {shape!r} (one of {sorted(shapes)})")
    if waves_per_simd not in (1, 2):
        raise ValueError("waves_per_simd must be 1 or 2")
    dev = torch.device("cuda", torch.cuda.current_device())
    need = 16 * 64 * 8
    if operands is None:
        g = torch.Generator(device="cpu").manual_seed(0)
        operands = torch.randn(need, generator=g).to(torch.bfloat16).to(dev)
    if not (operands.is_cuda and operands.dtype == torch.bfloat16 and operands.is_contiguous() and operands.numel() >= need):
        raise ValueError(f"operands must be a contiguous bf16 GPU tensor of at least {need} elements")
    with torch.cuda.device(operands.device):
        cus = _lib.load().ms_query(_lib.MS_QUERY_CU_COUNT)
    if cus <= 0:
        raise _lib.MeshSliceError("could not read the compute-unit count of the device")
    sink = torch.empty(256 * waves_per_simd * int(cus), dtype=torch.float32, device=operands.device)
    ms, fl = ctypes.c_float(0.0), ctypes.c_double(0.0)
    with torch.cuda.device(operands.device):
        rc = _lib.load().ms_probe_mfma_stream_ex(ctypes.c_void_p(operands.data_ptr()), ctypes.c_void_p(sink.data_ptr()),
                                                 shapes[shape], int(waves_per_simd), int(iters), int(warmup), int(reps),
                                                 ctypes.byref(ms), ctypes.byref(fl), _stream())
    _lib.check(rc)
    return fl.value / (ms.value * 1e-3)
