"""MI355X-native per-device sliced 2-D GEMM for MeshSlice-style tensor parallelism."""
from . import _lib  # noqa: F401
from .local_gemm import gemm_os, gemm_ls, gemm_rs, gemm_ls_signal, gemm_rs_signal, time_call  # noqa: F401

__all__ = ["gemm_os", "gemm_ls", "gemm_rs", "gemm_ls_signal", "gemm_rs_signal", "time_call"]
