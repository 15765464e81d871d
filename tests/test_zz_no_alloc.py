"""The entry point that allocates nothing (``ms_gemm_os_noalloc``) through the C ABI: against ``ms_gemm_os_ws`` bit for
bit on two calls in a row, the second with a smaller input, and against the float64 oracle (rel-Frobenius <= 1e-2,
bf16 in / fp32 accumulate; 1e-5 for the fp32 product); the device's free memory does not move across the calls; calls that alternate between two
streams, and replays of a captured call, give the same bits; an over-sized product is refused with a message."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import meshslice_oracle as orc
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
    free_before = torch.cuda.mem_get_info()[0]
    _lib.check(L.ms_gemm_os_noalloc(*head(got), None))
    assert L.ms_query(_lib.MS_QUERY_LAST_SPLITS) == splits
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before, "device memory was allocated or freed during the call"
    # and against the float64 oracle on sampled rows
    rows = np.random.default_rng(m + n).choice(m, min(m, 24), replace=False)
    f64 = lambda t: t.float().cpu().numpy().astype(np.float64)
    ref = sum(f64(a[rows]) @ f64(b) for a, b in zip(A, B))
    assert orc.rel_frobenius(f64(got[rows]), ref) <= 1e-2
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
    # fp32 operands take the fp32 kernel: a small product without the scratch ...
    a32 = torch.randn((256, 128), device="cuda"); b32 = torch.randn((128, 256), device="cuda")
    c32 = torch.empty((256, 256), device="cuda")
    pa, _ka = _lib.ptr_array([a32.data_ptr()]); pb, _kb = _lib.ptr_array([b32.data_ptr()])
    _lib.check(L.ms_gemm_os_noalloc(pa, pb, 1, 256, 256, 128, 128, 256, ctypes.c_void_p(c32.data_ptr()), 256,
                                    _lib.MS_DTYPE_F32, _lib.MS_DTYPE_F32, None))
    assert L.ms_query(_lib.MS_QUERY_LAST_SPLITS) == 1
    assert torch.allclose(c32, a32 @ b32, rtol=1e-4, atol=1e-3)
    # ... and one that splits its contraction through it (1536 x 1536 x 4096 in two slices), the bits of ms_gemm_os_ws
    g = torch.Generator(device="cuda").manual_seed(7)
    A5 = [torch.randn((1536, 2048), generator=g, device="cuda") for _ in range(2)]
    B5 = [torch.randn((2048, 1536), generator=g, device="cuda") * 0.02 for _ in range(2)]
    pa, _ka = _lib.ptr_array([t.data_ptr() for t in A5]); pb, _kb = _lib.ptr_array([t.data_ptr() for t in B5])
    ws = local_gemm.workspace("cuda")
    want5 = torch.empty((1536, 1536), device="cuda"); got5 = torch.zeros((1536, 1536), device="cuda")
    head5 = lambda C: (pa, pb, 2, 1536, 1536, 2048, 2048, 1536, ctypes.c_void_p(C.data_ptr()), 1536, _lib.MS_DTYPE_F32, _lib.MS_DTYPE_F32)
    _lib.check(L.ms_gemm_os_ws(*head5(want5), _lib.MS_ACT_NONE, None, 0, None, None, ctypes.c_void_p(ws.data_ptr()), ws.numel(), None))
    splits5, tile5 = L.ms_query(_lib.MS_QUERY_LAST_SPLITS), L.ms_query(_lib.MS_QUERY_LAST_VARIANT)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    _lib.check(L.ms_gemm_os_noalloc(*head5(got5), None))
    assert splits5 > 1 and L.ms_query(_lib.MS_QUERY_LAST_SPLITS) == splits5 and L.ms_query(_lib.MS_QUERY_LAST_VARIANT) == tile5
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    assert torch.equal(got5, want5)
    ref5 = sum(a[:48].double() @ b.double() for a, b in zip(A5, B5))
    assert ((got5[:48].double() - ref5).norm() / ref5.norm()).item() <= 1e-5


def _noalloc(L, A, B, C, stream):
    m, k = A[0].shape; n = B[0].shape[1]
    pa, _ka = _lib.ptr_array([t.data_ptr() for t in A]); pb, _kb = _lib.ptr_array([t.data_ptr() for t in B])
    _lib.check(L.ms_gemm_os_noalloc(pa, pb, len(A), m, n, k, A[0].stride(0), B[0].stride(0), ctypes.c_void_p(C.data_ptr()), n,
                                    _lib.MS_DTYPE_BF16, _lib.MS_DTYPE_BF16, ctypes.c_void_p(stream.cuda_stream)))


def test_no_alloc_calls_that_alternate_between_two_streams_do_not_meet_in_the_scratch():
    """Two different split products, issued alternately on two streams with no ordering of the caller's between them:
    the entry point itself keeps them apart (it waits for the device when the stream changes)."""
    L = _lib.load()
    L.ms_set_variant(0)
    A1 = [_rand((2048, 3072), 1.0, 61 + s) for s in range(4)]; B1 = [_rand((3072, 1536), 0.02, 71 + s) for s in range(4)]
    A2 = [_rand((1024, 4096), 1.0, 81 + s) for s in range(2)]; B2 = [_rand((4096, 768), 0.02, 91 + s) for s in range(2)]
    want1 = torch.empty((2048, 1536), dtype=torch.bfloat16, device="cuda"); want2 = torch.empty((1024, 768), dtype=torch.bfloat16, device="cuda")
    main = torch.cuda.current_stream()
    _noalloc(L, A1, B1, want1, main); assert L.ms_query(_lib.MS_QUERY_LAST_SPLITS) > 1
    _noalloc(L, A2, B2, want2, main); assert L.ms_query(_lib.MS_QUERY_LAST_SPLITS) > 1
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    outs1 = [torch.empty_like(want1) for _ in range(8)]; outs2 = [torch.empty_like(want2) for _ in range(8)]
    for r in range(8):
        _noalloc(L, A1, B1, outs1[r], s1)
        _noalloc(L, A2, B2, outs2[r], s2)
    torch.cuda.synchronize()
    for r in range(8):
        assert torch.equal(outs1[r], want1) and torch.equal(outs2[r], want2), r


def test_no_alloc_call_replays_from_a_hip_graph():
    """One warm call outside the capture (it looks the scratch's address up), then the call is captured and replayed
    with eager calls in between: every replay gives the eager bits."""
    L = _lib.load()
    L.ms_set_variant(0)
    A = [_rand((1024, 2048), 1.0, 101 + s) for s in range(2)]; B = [_rand((2048, 1536), 0.02, 111 + s) for s in range(2)]
    eager = torch.empty((1024, 1536), dtype=torch.bfloat16, device="cuda")
    out = torch.empty_like(eager)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        _noalloc(L, A, B, eager, side)
        assert L.ms_query(_lib.MS_QUERY_LAST_SPLITS) > 1
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            _noalloc(L, A, B, out, side)
        for _ in range(3):
            out.zero_()
            side.synchronize()
            graph.replay()
            side.synchronize()
            assert torch.equal(out, eager)
            again = torch.empty_like(eager)
            _noalloc(L, A, B, again, side)              # eager work between the replays, same stream
            side.synchronize()
            assert torch.equal(again, eager)
    torch.cuda.synchronize()


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
