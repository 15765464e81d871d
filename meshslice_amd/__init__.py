"""MI355X-native per-device sliced 2-D GEMM for MeshSlice-style tensor parallelism."""
from . import _lib  # noqa: F401
from .local_gemm import (gemm_os, gemm_ls, gemm_rs, gemm_ls_signal, gemm_rs_signal, gemm_os_gated, gemm_ls_gated, gemm_rs_gated, signal_set,  # noqa: F401
                         gate_timed_out, time_call)

__all__ = ["gemm_os", "gemm_ls", "gemm_rs", "gemm_ls_signal", "gemm_rs_signal", "gemm_os_gated", "gemm_ls_gated", "gemm_rs_gated", "signal_set", "gate_timed_out",
           "time_call"]
