"""Output-stationary products whose contraction is split over compute units (``ms_gemm_os_ws``): parity with the
float64 oracle and with the unsplit kernels, run-to-run bit-identity, the fused epilogue, HIP-graph capture, the
workspace rules of the C ABI.  Tolerance: rel-Frobenius <= 1e-2 against the oracle (bf16 in, fp32 accumulate)."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import meshslice_oracle as orc
import meshslice_amd as ms
from meshslice_amd import _lib, local_gemm

pytestmark = pytest.mark.gpu
TOL_BF16 = 1e-2
SPLIT_VARIANTS = (2, 3, 5, 6, 7, 8, 9, 10, 11)      # 1 and 4 (256x256 on four waves) have no split path


@pytest.fixture(autouse=True)
def _default_variant():
    _lib.load().ms_set_variant(0)
    yield
    _lib.load().ms_set_variant(0)
    torch.cuda.synchronize()


def _rand(shape, scale, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return (torch.randn(shape, generator=g, device="cuda") * scale).to(torch.bfloat16)


def _f64(t):
    return t.float().cpu().numpy().astype(np.float64)


def _counters():
    ws = local_gemm.workspace("cuda")
    return ws[:4096].view(torch.int32)


@pytest.mark.parametrize("variant", SPLIT_VARIANTS)
@pytest.mark.parametrize("splits", [2, 3, 8])
def test_forced_split_matches_oracle_and_is_bit_reproducible(variant, splits):
    """Ragged shapes (edge tiles, a K tail, K steps that do not divide by the split count, slices that a split's
    K range crosses) on every tile variant that can split."""
    L = _lib.load()
    m, n, ks, S = 200, 424, 712, 3             # 3 slices of 712 = 11.1 K steps of 64 each
    A = [_rand((m, ks), 1.0, 10 + s) for s in range(S)]
    B = [_rand((ks, n), 0.05, 20 + s) for s in range(S)]
    want = sum(_f64(a) @ _f64(b) for a, b in zip(A, B))
    L.ms_set_variant(variant)
    plain = ms.gemm_os(A, B, out_dtype=torch.float32)
    assert L.ms_query(_lib.MS_QUERY_LAST_SPLITS) == 1
    L.ms_set_variant(variant + 100 * splits)
    got = ms.gemm_os(A, B, out_dtype=torch.float32)
    assert L.ms_query(_lib.MS_QUERY_LAST_SPLITS) == splits and L.ms_query(_lib.MS_QUERY_LAST_VARIANT) == variant
    assert orc.rel_frobenius(_f64(got), want) <= 1e-5 * 50      # fp32 out of bf16 operands: accumulation error only
    assert orc.rel_frobenius(_f64(got), _f64(plain)) <= 1e-6
    for _ in range(3):                                          # the sum order is fixed: same bits every time
        assert torch.equal(ms.gemm_os(A, B, out_dtype=torch.float32), got)
    torch.cuda.synchronize()
    assert int(_counters().abs().sum()) == 0                    # the arrival counters are clear again
    out_bf16 = ms.gemm_os(A, B)
    assert torch.equal(out_bf16, got.to(torch.bfloat16))        # bf16 output = one rounding of the same sums


def _unsplit(A, B, out_dtype=torch.float32):
    """The same product through ms_gemm_os, which has no workspace and therefore never splits."""
    L = _lib.load()
    S, (m, ks), n = len(A), A[0].shape, B[0].shape[1]
    pa, _ka = _lib.ptr_array([t.data_ptr() for t in A]); pb, _kb = _lib.ptr_array([t.data_ptr() for t in B])
    C = torch.empty((m, n), dtype=out_dtype, device="cuda")
    dt = _lib.MS_DTYPE_BF16 if A[0].dtype == torch.bfloat16 else _lib.MS_DTYPE_F32
    rc = L.ms_gemm_os(pa, pb, S, m, n, ks, ks, n, ctypes.c_void_p(C.data_ptr()), n, dt,
                      _lib.MS_DTYPE_BF16 if out_dtype == torch.bfloat16 else _lib.MS_DTYPE_F32, None)
    assert rc == 0 and L.ms_query(_lib.MS_QUERY_LAST_SPLITS) == 1
    return C


@pytest.mark.parametrize("tile", [21, 22, 23, 24, 25])
@pytest.mark.parametrize("splits", [2, 3, 8])
def test_fp32_forced_split_matches_oracle_and_is_bit_reproducible(tile, splits):
    """The fp32 kernel's split contraction on each of its tiles: ragged edges, a K tail, K steps that do not divide by the
    split count, slices that a split's K range crosses.  Tolerance 1e-5 of the result's norm (fp32 in and out)."""
    L = _lib.load()
    m, n, ks, S = 200, 424, 708, 3             # 3 slices of 708 = 22.1 K steps of 32 each
    g = torch.Generator(device="cuda").manual_seed(100 * tile + splits)
    A = [torch.randn((m, ks), generator=g, device="cuda") for _ in range(S)]
    B = [torch.randn((ks, n), generator=g, device="cuda") * 0.05 for _ in range(S)]
    want = sum(_f64(a) @ _f64(b) for a, b in zip(A, B))
    L.ms_set_variant(tile)
    plain = _unsplit(A, B)
    assert L.ms_query(_lib.MS_QUERY_LAST_VARIANT) == tile
    L.ms_set_variant(tile + 100 * splits)
    got = ms.gemm_os(A, B)
    assert L.ms_query(_lib.MS_QUERY_LAST_SPLITS) == splits and L.ms_query(_lib.MS_QUERY_LAST_VARIANT) == tile
    assert orc.rel_frobenius(_f64(got), want) <= 1e-5
    assert orc.rel_frobenius(_f64(got), _f64(plain)) <= 1e-6
    for _ in range(3):
        assert torch.equal(ms.gemm_os(A, B), got)
    torch.cuda.synchronize()
    assert int(_counters().abs().sum()) == 0
    assert torch.equal(ms.gemm_os(A, B, out_dtype=torch.bfloat16), got.to(torch.bfloat16))


def test_fp32_product_of_well_under_one_round_is_split_by_default():
    """1536 x 1536 x 4096 in fp32: 72 tiles of 256x128 (or 576 of 64x64 in three rounds) for 256 compute units."""
    L = _lib.load()
    g = torch.Generator(device="cuda").manual_seed(5)
    A = [torch.randn((1536, 2048), generator=g, device="cuda") for _ in range(2)]
    B = [torch.randn((2048, 1536), generator=g, device="cuda") * 0.02 for _ in range(2)]
    C = ms.gemm_os(A, B)
    assert L.ms_query(_lib.MS_QUERY_LAST_SPLITS) > 1 and 21 <= L.ms_query(_lib.MS_QUERY_LAST_VARIANT) <= 25
    rows = np.random.default_rng(0).choice(1536, 64, replace=False)
    want = sum(_f64(a[rows]) @ _f64(b) for a, b in zip(A, B))
    assert orc.rel_frobenius(_f64(C[rows]), want) <= 1e-5
    assert torch.equal(ms.gemm_os(A, B), C)
    assert orc.rel_frobenius(_f64(_unsplit(A, B)), _f64(C)) <= 1e-6
    # LS / RS chunks and products with a tile per unit stay unsplit
    ms.gemm_ls(A[0], [B[0].t().contiguous()])
    assert L.ms_query(_lib.MS_QUERY_LAST_SPLITS) == 1
    ms.gemm_os([torch.randn((4096, 256), generator=g, device="cuda")], [torch.randn((256, 4096), generator=g, device="cuda")])
    assert L.ms_query(_lib.MS_QUERY_LAST_SPLITS) == 1
    # a forced split that cannot be: more items than compute units
    L.ms_set_variant(824)
    with pytest.raises(ValueError, match="cannot be split"):
        ms.gemm_os(A, B)


def test_small_output_long_contraction_is_split_by_default():
    """2048 x 1536 x 12288 (out_proj backward-data on an 8x8 mesh): 64 tiles for 256 compute units."""
    L = _lib.load()
    A = [_rand((2048, 3072), 1.0, 30 + s) for s in range(4)]
    B = [_rand((3072, 1536), 0.02, 40 + s) for s in range(4)]
    C = ms.gemm_os(A, B)
    splits = L.ms_query(_lib.MS_QUERY_LAST_SPLITS)
    assert splits > 1
    rows = np.random.default_rng(0).choice(2048, 64, replace=False)
    want = sum(_f64(a[rows]) @ _f64(b) for a, b in zip(A, B))
    assert orc.rel_frobenius(_f64(C[rows]), want) <= TOL_BF16
    assert torch.equal(ms.gemm_os(A, B), C)
    # the same product without a workspace is not split and agrees to output rounding
    pa, _ka = _lib.ptr_array([t.data_ptr() for t in A]); pb, _kb = _lib.ptr_array([t.data_ptr() for t in B])
    C1 = torch.empty_like(C)
    rc = L.ms_gemm_os(pa, pb, 4, 2048, 1536, 3072, 3072, 1536, ctypes.c_void_p(C1.data_ptr()), 1536,
                      _lib.MS_DTYPE_BF16, _lib.MS_DTYPE_BF16, None)
    assert rc == 0 and L.ms_query(_lib.MS_QUERY_LAST_SPLITS) == 1
    assert orc.rel_frobenius(_f64(C1), _f64(C)) <= 4e-3
    # a product with a tile per compute unit (or more) stays unsplit
    ms.gemm_os([_rand((4096, 1024), 1.0, 1)], [_rand((1024, 12288), 0.02, 2)])
    assert L.ms_query(_lib.MS_QUERY_LAST_SPLITS) == 1


def test_a_fused_epilogue_keeps_the_product_unsplit():
    """The fused-epilogue kernels carry no exchange of partial tiles: a product that would split runs unsplit when an
    epilogue is asked for, and a forced split is refused."""
    L = _lib.load()
    A = [_rand((2048, 3072), 1.0, 30 + s) for s in range(4)]
    B = [_rand((3072, 1536), 0.02, 40 + s) for s in range(4)]
    plain = ms.gemm_os(A, B, out_dtype=torch.float32)
    assert L.ms_query(_lib.MS_QUERY_LAST_SPLITS) > 1
    fused = ms.gemm_os(A, B, out_dtype=torch.float32, activation="gelu")
    assert L.ms_query(_lib.MS_QUERY_LAST_SPLITS) == 1
    assert orc.rel_frobenius(_f64(fused), orc.gelu_tanh(_f64(plain))) <= 1e-5
    L.ms_set_variant(408)
    with pytest.raises(ValueError, match="fused epilogue"):
        ms.gemm_os(A, B, activation="gelu")


def test_split_product_replays_from_a_hip_graph():
    A = [_rand((1024, 2048), 1.0, 60 + s) for s in range(2)]
    B = [_rand((2048, 1536), 0.02, 70 + s) for s in range(2)]
    out = torch.empty((1024, 1536), dtype=torch.bfloat16, device="cuda")
    eager = ms.gemm_os(A, B)
    assert _lib.load().ms_query(_lib.MS_QUERY_LAST_SPLITS) > 1
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        ms.gemm_os(A, B, out=out)
    for _ in range(3):
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager)
        assert torch.equal(ms.gemm_os(A, B), eager)     # eager work between the replays


def test_workspace_rules_of_the_c_abi():
    L = _lib.load()
    A = _rand((256, 2048), 1.0, 80); B = _rand((2048, 256), 0.05, 81)
    C = torch.empty((256, 256), dtype=torch.bfloat16, device="cuda")
    pa, _ka = _lib.ptr_array([A.data_ptr()]); pb, _kb = _lib.ptr_array([B.data_ptr()])
    head = (pa, pb, 1, 256, 256, 2048, 2048, 256, ctypes.c_void_p(C.data_ptr()), 256, _lib.MS_DTYPE_BF16, _lib.MS_DTYPE_BF16)
    epi = (_lib.MS_ACT_NONE, None, 0, None, None)
    ws = local_gemm.workspace("cuda")
    assert ws.numel() == L.ms_workspace_bytes() >= 4096 + 256 * 256 * 384 * 4 // 2
    # no workspace: the product runs unsplit; a forced split is refused
    assert L.ms_gemm_os_ws(*head, *epi, None, 0, None) == 0 and L.ms_query(_lib.MS_QUERY_LAST_SPLITS) == 1
    L.ms_set_variant(408)
    assert L.ms_gemm_os_ws(*head, *epi, None, 0, None) == _lib.MS_ERR_ARG
    assert "workspace" in _lib.last_error()
    # misaligned or undersized workspaces are argument errors
    assert L.ms_gemm_os_ws(*head, *epi, ctypes.c_void_p(ws.data_ptr() + 16), 1 << 20, None) == _lib.MS_ERR_ARG
    assert L.ms_gemm_os_ws(*head, *epi, ctypes.c_void_p(ws.data_ptr()), 1024, None) == _lib.MS_ERR_ARG
    # a workspace too small for the partial tiles of a forced split is refused with the reason
    assert L.ms_gemm_os_ws(*head, *epi, ctypes.c_void_p(ws.data_ptr()), 4096 + 1000, None) == _lib.MS_ERR_ARG
    assert "do not fit" in _lib.last_error()
    # ... and merely narrows the library's own choice
    L.ms_set_variant(0)
    assert L.ms_gemm_os_ws(*head, *epi, ctypes.c_void_p(ws.data_ptr()), 4096 + 1000, None) == 0
    assert L.ms_query(_lib.MS_QUERY_LAST_SPLITS) == 1
    # variants without a split path refuse (256x256 on four waves); bad split counts are unknown variants
    L.ms_set_variant(401)
    assert L.ms_gemm_os_ws(*head, *epi, ctypes.c_void_p(ws.data_ptr()), ws.numel(), None) == _lib.MS_ERR_ARG
    assert "no split path" in _lib.last_error()
    assert L.ms_set_variant(108) == _lib.MS_ERR_ARG and L.ms_set_variant(908) == _lib.MS_ERR_ARG and L.ms_set_variant(15) == _lib.MS_ERR_ARG
    L.ms_set_variant(0)
    assert L.ms_workspace_init(None, 4096, None) == _lib.MS_ERR_ARG
    assert L.ms_workspace_init(ctypes.c_void_p(ws.data_ptr()), 100, None) == _lib.MS_ERR_ARG
    torch.cuda.synchronize()
    got = ms.gemm_os([A], [B])
    assert orc.rel_frobenius(_f64(got), _f64(A) @ _f64(B)) <= TOL_BF16


def test_split_products_on_two_streams_and_threads_do_not_share_a_workspace():
    """Two host threads, each on a stream of its own, run products that DO split (64 tiles for 256 compute units),
    twenty rounds each, at the same time: every result equals the same product's single-stream result bit for bit and
    the float64 oracle to tolerance.  (One workspace shared by both streams would let their arrival counters and
    partial tiles meet.)"""
    import threading
    L = _lib.load()
    cases = []
    for t in range(2):
        A = [_rand((2048, 3072), 1.0, 200 + 10 * t + s) for s in range(4)]
        B = [_rand((3072, 1536), 0.02, 300 + 10 * t + s) for s in range(4)]
        alone = ms.gemm_os(A, B)
        assert L.ms_query(_lib.MS_QUERY_LAST_SPLITS) > 1
        rows = np.random.default_rng(t).choice(2048, 32, replace=False)
        want = sum(_f64(a[rows]) @ _f64(b) for a, b in zip(A, B))
        assert orc.rel_frobenius(_f64(alone[rows]), want) <= TOL_BF16
        cases.append((A, B, alone))
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    ready = threading.Barrier(2)
    bad, errors, split_counts = [], [], [None, None]

    def work(t):
        try:
            torch.cuda.set_device(0)
            A, B, alone = cases[t]
            outs = [torch.empty_like(alone) for _ in range(20)]
            with torch.cuda.stream(streams[t]):
                ms.gemm_os(A, B, out=outs[0])          # (this stream's workspace is made here, before the two meet)
                streams[t].synchronize()
                ready.wait()
                for r in range(20):
                    ms.gemm_os(A, B, out=outs[r])
                split_counts[t] = int(_lib.load().ms_query(_lib.MS_QUERY_LAST_SPLITS))
                streams[t].synchronize()
            bad.extend((t, r) for r in range(20) if not torch.equal(outs[r], alone))
        except Exception as e:  # pragma: no cover
            errors.append(e)
            ready.abort()

    threads = [threading.Thread(target=work, args=(t,)) for t in range(2)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    torch.cuda.synchronize()
    assert not errors, errors
    assert split_counts[0] > 1 and split_counts[1] > 1
    assert not bad, f"(thread, round) whose result differs from the single-stream result: {bad}"
    w0 = local_gemm.workspace("cuda", streams[0]); w1 = local_gemm.workspace("cuda", streams[1])
    assert w0.data_ptr() != w1.data_ptr() != local_gemm.workspace("cuda").data_ptr()
    # the same two products interleaved from ONE host thread on the two streams
    outs = [[torch.empty_like(cases[t][2]) for _ in range(10)] for t in range(2)]
    for r in range(10):
        for t in range(2):
            with torch.cuda.stream(streams[t]):
                ms.gemm_os(cases[t][0], cases[t][1], out=outs[t][r])
    torch.cuda.synchronize()
    for t in range(2):
        for r in range(10):
            assert torch.equal(outs[t][r], cases[t][2]), (t, r)


def test_workspace_cache_keeps_a_bounded_number_of_streams():
    keep = local_gemm._WORKSPACE_CACHE_MAX
    streams = [torch.cuda.Stream() for _ in range(3)]
    try:
        local_gemm._WORKSPACE_CACHE_MAX = 2
        first = local_gemm.workspace("cuda", streams[0])
        assert local_gemm.workspace("cuda", streams[0]) is first
        local_gemm.workspace("cuda", streams[1])
        local_gemm.workspace("cuda", streams[2])
        mine = [k for k in local_gemm._workspaces if k[0] == torch.cuda.current_device()]
        assert len(mine) == 2 and (torch.cuda.current_device(), streams[2].cuda_stream) in mine
    finally:
        local_gemm._WORKSPACE_CACHE_MAX = keep
    A = [_rand((1024, 2048), 1.0, 90)]; B = [_rand((2048, 768), 0.02, 91)]
    with torch.cuda.stream(streams[0]):
        got = ms.gemm_os(A, B)
    torch.cuda.synchronize()
    assert orc.rel_frobenius(_f64(got), _f64(A[0]) @ _f64(B[0])) <= TOL_BF16
