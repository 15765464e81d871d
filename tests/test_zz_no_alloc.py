"""The entry point that allocates nothing (``ms_gemm_os_noalloc``) against ``ms_gemm_os_ws`` through the C ABI: two calls
in a row, the second with a smaller input, bit for bit; an over-sized product is refused with a message."""
import ctypes

import pytest
import torch

from meshslice_amd import _lib, local_gemm

pytestmark = pytest.mark.gpu


def _rand(shape, scale, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return (torch.randn(shape, generator=g, device="cuda") * scale).to(torch.bfloat16)


def _both(L, A, B, m, n, k, S):
    pa, _ka = _lib.ptr_array([t.data_ptr() for t in A]); pb, _kb = _lib.ptr_array([t.data_ptr() for t in B])
    ws = local_gemm.workspace("cuda")
    want = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
    head = lambda C: (pa, pb, S, m, n, k, A[0].stride(0), B[0].stride(0), ctypes.c_void_p(C.data_ptr()), n,
                      _lib.MS_DTYPE_BF16, _lib.MS_DTYPE_BF16)
    _lib.check(L.ms_gemm_os_ws(*head(want), _lib.MS_ACT_NONE, None, 0, None, None, ctypes.c_void_p(ws.data_ptr()), ws.numel(), None))
    splits = L.ms_query(_lib.MS_QUERY_LAST_SPLITS)
    got = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
    torch.cuda.synchronize()
    _lib.check(L.ms_gemm_os_noalloc(*head(got), None))
    assert L.ms_query(_lib.MS_QUERY_LAST_SPLITS) == splits
    torch.cuda.synchronize()
    return got, want, splits


def test_no_alloc_entry_point_matches_the_workspace_entry_point():
    L = _lib.load()
    L.ms_set_variant(0)
    # first call: 2048 x 1536 x 12288 in four slices (64 tiles, contraction split); second call: a smaller product
    A = [_rand((2048, 3072), 1.0, 1 + s) for s in range(4)]; B = [_rand((3072, 1536), 0.02, 11 + s) for s in range(4)]
    got, want, splits = _both(L, A, B, 2048, 1536, 3072, 4)
    assert splits > 1 and torch.equal(got, want)
    A2 = [_rand((1024, 2048), 1.0, 21 + s) for s in range(2)]; B2 = [_rand((2048, 768), 0.02, 31 + s) for s in range(2)]
    got2, want2, splits2 = _both(L, A2, B2, 1024, 768, 2048, 2)
    assert splits2 > 1 and torch.equal(got2, want2)
    # and once more the large one, after the small one has used the same scratch
    got3, want3, _ = _both(L, A, B, 2048, 1536, 3072, 4)
    assert torch.equal(got3, want) and torch.equal(want3, want)
    # a product that does not split needs no scratch at all
    A3 = [_rand((4096, 512), 1.0, 41)]; B3 = [_rand((512, 4096), 0.02, 42)]
    got4, want4, splits4 = _both(L, A3, B3, 4096, 4096, 512, 1)
    assert splits4 == 1 and torch.equal(got4, want4)
    # fp32 operands take the fp32 kernel (no scratch)
    a32 = torch.randn((256, 128), device="cuda"); b32 = torch.randn((128, 256), device="cuda")
    c32 = torch.empty((256, 256), device="cuda")
    pa, _ka = _lib.ptr_array([a32.data_ptr()]); pb, _kb = _lib.ptr_array([b32.data_ptr()])
    _lib.check(L.ms_gemm_os_noalloc(pa, pb, 1, 256, 256, 128, 128, 256, ctypes.c_void_p(c32.data_ptr()), 256,
                                    _lib.MS_DTYPE_F32, _lib.MS_DTYPE_F32, None))
    assert torch.allclose(c32, a32 @ b32, rtol=1e-4, atol=1e-3)


def test_no_alloc_entry_point_refuses_what_its_scratch_cannot_hold():
    L = _lib.load()
    A = [_rand((1024, 4096), 1.0, 51)]; B = [_rand((4096, 1536), 0.02, 52)]
    C = torch.empty((1024, 1536), dtype=torch.bfloat16, device="cuda")
    pa, _ka = _lib.ptr_array([A[0].data_ptr()]); pb, _kb = _lib.ptr_array([B[0].data_ptr()])
    args = (pa, pb, 1, 1024, 1536, 4096, 4096, 1536, ctypes.c_void_p(C.data_ptr()), 1536, _lib.MS_DTYPE_BF16, _lib.MS_DTYPE_BF16, None)
    try:
        L.ms_set_variant(810)      # 256 x 384 tiles, contraction split 8 ways: 16 tiles x 8 x 384 KiB = 48 MiB + header: fits exactly
        assert L.ms_gemm_os_noalloc(*args) == 0
        A2 = [_rand((2048, 4096), 1.0, 53)]; C2 = torch.empty((2048, 1536), dtype=torch.bfloat16, device="cuda")
        pa2, _ka2 = _lib.ptr_array([A2[0].data_ptr()])
        args2 = (pa2, pb, 1, 2048, 1536, 4096, 4096, 1536, ctypes.c_void_p(C2.data_ptr()), 1536, _lib.MS_DTYPE_BF16, _lib.MS_DTYPE_BF16, None)
        assert L.ms_gemm_os_noalloc(*args2) == _lib.MS_ERR_UNSUPPORTED      # 32 tiles x 8: twice the scratch
        assert "built-in scratch" in _lib.last_error()
        L.ms_set_variant(0)
        assert L.ms_gemm_os_noalloc(*args2) == 0                            # the library's own choice fits
        assert L.ms_gemm_os_noalloc(pa2, pb, 1, 2048, 1536, -1, 4096, 1536, ctypes.c_void_p(C2.data_ptr()), 1536,
                                    _lib.MS_DTYPE_BF16, _lib.MS_DTYPE_BF16, None) == _lib.MS_ERR_ARG
    finally:
        L.ms_set_variant(0)
        torch.cuda.synchronize()
