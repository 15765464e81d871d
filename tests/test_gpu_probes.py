"""The measurement aids (``meshslice_amd/probes.py``: ``ms_probe_os_parts``, ``ms_probe_l2_lds_stream``): the whole
kernel of the parts probe is the product kernel (same bits as ``gemm_os`` on the 16x16x32 variant, right against the
float64 oracle), the cut-down kernels run and end, the stream probe reports a rate inside the machine's limits, and bad
arguments come back as error codes."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import meshslice_oracle as orc
import meshslice_amd as ms
from meshslice_amd import _lib, probes

pytestmark = pytest.mark.gpu


def _rand(shape, scale, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return (torch.randn(shape, generator=g, device="cuda") * scale).to(torch.bfloat16)


def test_whole_kernel_of_the_parts_probe_is_the_product_kernel():
    L = _lib.load()
    S, m, n, ks = 3, 520, 776, 200          # ragged: edge tiles, a K tail in every slice
    A = [_rand((m, ks), 1.0, 1 + s) for s in range(S)]
    B = [_rand((ks, n), 0.05, 11 + s) for s in range(S)]
    got = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
    t = probes.os_parts_ms(0, A, B, got, warmup=1, reps=2)
    assert 0.0 < t < 10.0
    try:
        assert L.ms_set_variant(12) == 0
        want = ms.gemm_os(A, B)
    finally:
        L.ms_set_variant(0)
    assert torch.equal(got, want)
    f64 = lambda x: x.float().cpu().numpy().astype(np.float64)
    assert orc.rel_frobenius(f64(got), sum(f64(a) @ f64(b) for a, b in zip(A, B))) <= 1e-2


@pytest.mark.parametrize("skip", [1, 2, 3, 4, 8, 16, 24])
def test_cut_down_kernels_run_and_end(skip):
    A = [_rand((512, 256), 1.0, 21 + s) for s in range(2)]
    B = [_rand((256, 768), 0.05, 31 + s) for s in range(2)]
    C = torch.empty((512, 768), dtype=torch.bfloat16, device="cuda")
    t = probes.os_parts_ms(skip, A, B, C, warmup=1, reps=3)
    torch.cuda.synchronize()
    assert 0.0 < t < 10.0


def test_parts_probe_rejects_bad_arguments():
    L = _lib.load()
    A = [_rand((256, 64), 1.0, 41)]; B = [_rand((64, 384), 0.05, 42)]
    C = torch.empty((256, 384), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError, match="no kernel was built"):
        probes.os_parts_ms(5, A, B, C, warmup=1, reps=1)
    with pytest.raises(ValueError, match="bf16"):
        probes.os_parts_ms(0, [A[0].float()], [B[0].float()], C.float(), warmup=1, reps=1)
    pa, _ka = _lib.ptr_array([A[0].data_ptr()]); pb, _kb = _lib.ptr_array([B[0].data_ptr()])
    ms_out = ctypes.c_float(0.0)
    args = lambda **kw: [kw.get("skip", 0), pa, pb, kw.get("S", 1), 256, 384, kw.get("k", 64), 64, 384, ctypes.c_void_p(C.data_ptr()), 384,
                         1, kw.get("reps", 1), ctypes.byref(ms_out), None]
    assert L.ms_probe_os_parts(*args(S=0)) == _lib.MS_ERR_ARG
    assert L.ms_probe_os_parts(*args(k=60)) == _lib.MS_ERR_ARG
    assert L.ms_probe_os_parts(*args(reps=0)) == _lib.MS_ERR_ARG
    assert L.ms_probe_os_parts(*args()) == 0
    torch.cuda.synchronize()


def test_l2_lds_stream_probe_reports_a_rate_inside_the_machines_limits():
    r = probes.l2_lds_stream_rate(region_steps=8, in_flight_steps=2, steps=200, warmup=1, reps=3)
    # more than HBM could deliver (the data sits in the L2s), less than 64 B per clock and compute unit at 2.4 GHz
    assert 4e12 < r["bytes_per_s"] < 256 * 64 * 2.4e9 * 1.05
    L = _lib.load()
    buf = torch.ones(8 * 81920 // 2, dtype=torch.bfloat16, device="cuda"); sink = torch.zeros(1, device="cuda")
    ms_out, moved = ctypes.c_float(0.0), ctypes.c_double(0.0)
    call = lambda region, fl, nbytes: L.ms_probe_l2_lds_stream(ctypes.c_void_p(buf.data_ptr()), nbytes, region, fl, 10, 0, 1, ctypes.c_void_p(sink.data_ptr()),
                                                              ctypes.byref(ms_out), ctypes.byref(moved), None)
    assert call(1, 2, buf.numel() * 2) == 0 and moved.value == L.ms_query(_lib.MS_QUERY_CU_COUNT) * 10 * 81920
    assert call(2, 2, buf.numel() * 2) == _lib.MS_ERR_ARG          # the buffer holds one step per XCD
    assert call(1, 4, buf.numel() * 2) == _lib.MS_ERR_ARG
    torch.cuda.synchronize()
    assert float(sink[0]) == 0.0


def test_the_comparison_tool_times_a_small_product_both_ways():
    """``python3 -m meshslice_amd.compare``: one small product beside the vendor library's in all three layouts, and the
    default tile choice against the forced variants on one random shape per dataflow; the fp32 kernel's tiles on one small product."""
    from meshslice_amd import compare
    res = compare.vendor([(1024, 1024, 1024)])
    assert set(res) == {"nn", "nt", "tn"} and all(r["cases"] == 1 and 0.2 < r["geometric_mean"] < 5.0 for r in res.values())
    res = compare.chooser(1, 2, 3)
    assert set(res) == {"os", "ls", "rs"} and all(r["cases"] == 1 and 0.5 < r["max"] < 1.5 for r in res.values())
    assert _lib.load().ms_query(_lib.MS_QUERY_LAST_VARIANT) >= 1
    res = compare.fp32([(1024, 1024, 512)])
    assert res["cases"] == 1 and 0.2 < res["vendor_over_ours_geometric_mean"] < 5.0 and res["default_over_best_tile_max"] < 1.5
