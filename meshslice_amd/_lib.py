"""ctypes binding of libmeshslice_hip.so (the C ABI declared in include/meshslice_hip.h).

There is no CPU fallback: if the shared library has not been built, or a call fails, an exception is
raised.  Build it with ``python -c "import __graft_entry__ as g; g.build()"`` or
``make -C meshslice_amd/csrc``.
"""
from __future__ import annotations

import ctypes
import os
import threading

MS_DTYPE_F32 = 0
MS_DTYPE_BF16 = 1
MS_OK = 0
MS_ERR_ARG = -1
MS_ERR_UNSUPPORTED = -2
MS_ERR_HIP = -3
MS_QUERY_CU_COUNT = 0
MS_QUERY_CLOCK_KHZ = 1
MS_QUERY_IS_GFX950 = 2
MS_QUERY_LDS_BYTES = 3
MS_QUERY_MAX_SLICES = 4
MS_QUERY_LAST_LAUNCHES = 5
MS_QUERY_LAST_VARIANT = 6
MS_QUERY_LAST_SPLITS = 7
MS_QUERY_LAST_GRID = 8
MS_ACT_NONE = 0
MS_ACT_GELU = 1
MS_MFMA_32X32X16 = 0
MS_MFMA_16X16X32 = 1

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmeshslice_hip.so")

EXPORTS = (
    "ms_version", "ms_last_error", "ms_query", "ms_set_variant",
    "ms_gemm_os", "ms_gemm_os_fused", "ms_gemm_os_ws", "ms_gemm_os_noalloc", "ms_gemm_os_gated", "ms_gemm_ls_gated", "ms_gemm_rs_gated", "ms_signal_set", "ms_workspace_bytes", "ms_workspace_init", "ms_time_os_ws", "ms_gemm_ls", "ms_gemm_rs", "ms_gemm_ls_ex", "ms_gemm_rs_ex", "ms_gemm_ls_signal", "ms_gemm_rs_signal", "ms_set_reserved_cus",
    "ms_time_os", "ms_time_ls", "ms_time_rs", "ms_time_ls_ex", "ms_time_rs_ex",
    "ms_pack_slices", "ms_unpack_chunks", "ms_probe_mfma_stream", "ms_probe_mfma_stream_ex",
    "ms_probe_os_parts", "ms_probe_l2_lds_stream",
)

_lock = threading.Lock()
_lib = None


class MeshSliceError(RuntimeError):
    """A call into libmeshslice_hip.so failed (HIP error or unsupported configuration)."""


def _declare(lib):
    c_int, c_vp, c_long = ctypes.c_int, ctypes.c_void_p, ctypes.c_long
    vpp = ctypes.POINTER(ctypes.c_void_p)
    fp = ctypes.POINTER(ctypes.c_float)
    lib.ms_version.argtypes = []
    lib.ms_version.restype = c_int
    lib.ms_last_error.argtypes = []
    lib.ms_last_error.restype = ctypes.c_char_p
    lib.ms_query.argtypes = [c_int]
    lib.ms_query.restype = c_long
    lib.ms_set_variant.argtypes = [c_int]
    lib.ms_set_variant.restype = c_int
    lib.ms_set_reserved_cus.argtypes = [c_int]
    lib.ms_set_reserved_cus.restype = c_int
    os_args = [vpp, vpp, c_int, c_int, c_int, c_int, c_int, c_int, c_vp, c_int, c_int, c_int, c_vp]
    ls_args = [c_vp, c_int, vpp, c_int, c_int, c_int, c_int, c_int, vpp, c_int, c_int, c_vp]
    rs_args = [vpp, c_int, c_vp, c_int, c_int, c_int, c_int, c_int, vpp, c_int, c_int, c_vp]
    lib.ms_gemm_os_fused.argtypes = os_args[:-1] + [c_int, c_vp, c_int, c_vp, c_vp, c_vp]
    lib.ms_gemm_os_fused.restype = c_int
    lib.ms_gemm_os.argtypes = os_args
    lib.ms_gemm_os_noalloc.argtypes = os_args
    lib.ms_gemm_os_noalloc.restype = c_int
    # ..., out_dtype, activation, residual, ldr, row_sum, row_sumsq, workspace, workspace_bytes, stream
    lib.ms_gemm_os_ws.argtypes = os_args[:-1] + [c_int, c_vp, c_int, c_vp, c_vp, c_vp, ctypes.c_size_t, c_vp]
    lib.ms_gemm_os_ws.restype = c_int
    # ..., out_dtype, workspace, workspace_bytes, slice_ready, timeout_ms, stream
    lib.ms_gemm_os_gated.argtypes = os_args[:-1] + [c_vp, ctypes.c_size_t, c_vp, ctypes.c_uint, c_vp]
    lib.ms_gemm_os_gated.restype = c_int
    # ..., in_dtype, out_dtype, chunk_done, tiles_per_chunk, slice_ready, timeout_ms, stream
    lib.ms_gemm_ls_gated.argtypes = ls_args[:-1] + [c_int, c_vp, ctypes.POINTER(c_int), c_vp, ctypes.c_uint, c_vp]
    lib.ms_gemm_ls_gated.restype = c_int
    lib.ms_gemm_rs_gated.argtypes = rs_args[:-1] + [c_int, c_vp, ctypes.POINTER(c_int), c_vp, ctypes.c_uint, c_vp]
    lib.ms_gemm_rs_gated.restype = c_int
    lib.ms_signal_set.argtypes = [c_vp, ctypes.c_uint, c_vp]
    lib.ms_signal_set.restype = c_int
    lib.ms_time_os_ws.argtypes = os_args[:-1] + [c_vp, ctypes.c_size_t, c_vp, c_int, c_int, fp]
    lib.ms_time_os_ws.restype = c_int
    lib.ms_workspace_bytes.argtypes = []
    lib.ms_workspace_bytes.restype = ctypes.c_size_t
    lib.ms_workspace_init.argtypes = [c_vp, ctypes.c_size_t, c_vp]
    lib.ms_workspace_init.restype = c_int
    lib.ms_gemm_ls.argtypes = ls_args
    lib.ms_gemm_rs.argtypes = rs_args
    lib.ms_gemm_ls_ex.argtypes = ls_args[:-1] + [c_int, c_vp]      # ..., in_dtype, out_dtype, stream
    lib.ms_gemm_rs_ex.argtypes = rs_args[:-1] + [c_int, c_vp]
    # ..., in_dtype, out_dtype, chunk_done, tiles_per_chunk, stream
    lib.ms_gemm_ls_signal.argtypes = ls_args[:-1] + [c_int, c_vp, ctypes.POINTER(c_int), c_vp]
    lib.ms_gemm_rs_signal.argtypes = rs_args[:-1] + [c_int, c_vp, ctypes.POINTER(c_int), c_vp]
    lib.ms_time_os.argtypes = os_args + [c_int, c_int, fp]
    lib.ms_time_ls.argtypes = ls_args + [c_int, c_int, fp]
    lib.ms_time_rs.argtypes = rs_args + [c_int, c_int, fp]
    lib.ms_time_ls_ex.argtypes = ls_args[:-1] + [c_int, c_vp, c_int, c_int, fp]    # ..., in_dtype, out_dtype, stream, warmup, reps, ms_out
    lib.ms_time_rs_ex.argtypes = rs_args[:-1] + [c_int, c_vp, c_int, c_int, fp]
    # src, ld_src, rows, cols, axis, S, B, dst_slices, ld_dst, dtype, stream
    lib.ms_pack_slices.argtypes = [c_vp, c_int, c_int, c_int, c_int, c_int, c_int, vpp, c_int, c_int, c_vp]
    lib.ms_pack_slices.restype = c_int
    # chunks, P, S, ld_chunk, row_off, col_off, rows, cols, axis, B, out, ld_out, in_dtype, out_dtype, stream
    lib.ms_unpack_chunks.argtypes = [vpp, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_vp, c_int, c_int, c_int, c_vp]
    lib.ms_unpack_chunks.restype = c_int
    # operands, sink, iters, warmup, reps, ms_out, flops_per_launch, stream
    lib.ms_probe_mfma_stream.argtypes = [c_vp, c_vp, c_int, c_int, c_int, fp, ctypes.POINTER(ctypes.c_double), c_vp]
    lib.ms_probe_mfma_stream.restype = c_int
    # operands, sink, shape, waves_per_simd, iters, warmup, reps, ms_out, flops_per_launch, stream
    lib.ms_probe_mfma_stream_ex.argtypes = [c_vp, c_vp, c_int, c_int, c_int, c_int, c_int, fp, ctypes.POINTER(ctypes.c_double), c_vp]
    lib.ms_probe_mfma_stream_ex.restype = c_int
    # skip, A_slices, B_slices, S, m, n, k_slice, lda, ldb, C, ldc, warmup, reps, ms_out, stream
    lib.ms_probe_os_parts.argtypes = [c_int, vpp, vpp, c_int, c_int, c_int, c_int, c_int, c_int, c_vp, c_int, c_int, c_int, fp, c_vp]
    lib.ms_probe_os_parts.restype = c_int
    # buffer, buffer_bytes, region_steps, in_flight_steps, steps, warmup, reps, sink, ms_out, bytes_per_launch, stream
    lib.ms_probe_l2_lds_stream.argtypes = [c_vp, ctypes.c_size_t, c_int, c_int, c_int, c_int, c_int, c_vp, fp, ctypes.POINTER(ctypes.c_double), c_vp]
    lib.ms_probe_l2_lds_stream.restype = c_int
    for n in ("ms_gemm_os", "ms_gemm_ls", "ms_gemm_rs", "ms_gemm_ls_ex", "ms_gemm_rs_ex", "ms_time_os", "ms_time_ls", "ms_time_rs",
              "ms_time_ls_ex", "ms_time_rs_ex", "ms_gemm_ls_signal", "ms_gemm_rs_signal"):
        getattr(lib, n).restype = c_int


def load():
    """Return the loaded library; raise MeshSliceError if it has not been built."""
    global _lib
    with _lock:
        if _lib is None:
            if not os.path.exists(LIB_PATH):
                raise MeshSliceError(
                    f"{LIB_PATH} is missing: the HIP extension has not been built "
                    "(run __graft_entry__.build() or `make -C meshslice_amd/csrc`); there is no CPU fallback")
            lib = ctypes.CDLL(LIB_PATH)
            _declare(lib)
            _lib = lib
        return _lib


def last_error() -> str:
    return load().ms_last_error().decode("utf-8", "replace")


def check(rc: int) -> None:
    """Map a C return code to the exception the reference's Python would raise in that situation:
    shape/argument problems -> ValueError, everything else -> MeshSliceError."""
    if rc == MS_OK:
        return
    msg = last_error()
    if rc == MS_ERR_ARG:
        raise ValueError(msg)
    raise MeshSliceError(f"libmeshslice_hip error {rc}: {msg}")


def ptr_array(ptrs):
    arr = (ctypes.c_void_p * len(ptrs))(*[int(p) for p in ptrs])
    return ctypes.cast(arr, ctypes.POINTER(ctypes.c_void_p)), arr
