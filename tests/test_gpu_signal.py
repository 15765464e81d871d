"""Completion counters of the chunk-producing calls (``ms_gemm_ls_signal`` / ``ms_gemm_rs_signal``): the counted
chunks equal the plain calls' bit for bit, every counter ends at the tile count the call reports, and a watcher on a
second stream that sees chunk s complete reads the finished chunk while the kernel is still running (the GEMM leaves
a few compute units free for the watcher's copies: its workgroups hold every register of the units they run on).

The watcher polls with a BOUNDED number of small device-to-host copies (never a spinning kernel): if the GEMM ends
before a poll sees a partial state the test still checks the final state, it just has nothing to say about overlap.
"""
import ctypes

import numpy as np
import pytest
import torch

import meshslice_amd as ms
from meshslice_amd import _lib

pytestmark = pytest.mark.gpu


def _rand(shape, seed, dtype, scale=1.0):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return (torch.randn(shape, generator=g, device="cuda") * scale).to(dtype)


def _operands(flow, m, n, k, S, dtype, seed=0):
    if flow == "ls":      # Y_s = A @ W_s^T
        return _rand((m, k), seed, dtype), [_rand((n, k), seed + 1 + s, dtype, 0.05) for s in range(S)]
    return [_rand((k, m), seed + 1 + s, dtype) for s in range(S)], _rand((k, n), seed, dtype, 0.05)   # Y_s = X_s^T @ W


def _plain(flow, ops, out_dtype):
    return ms.gemm_ls(ops[0], ops[1], out_dtype=out_dtype) if flow == "ls" else ms.gemm_rs(ops[0], ops[1], out_dtype=out_dtype)


def _signal(flow, ops, counters, out_dtype, out=None):
    fn = ms.gemm_ls_signal if flow == "ls" else ms.gemm_rs_signal
    return fn(ops[0], ops[1], counters, out=out, out_dtype=out_dtype)


@pytest.mark.parametrize("flow", ["ls", "rs"])
@pytest.mark.parametrize("variant", [0, 3, 8, 10, 11, 12])
def test_counted_chunks_equal_the_plain_call_and_every_counter_ends_at_the_tile_count(flow, variant):
    S, m, n, k = 5, 640, 776, 520      # ragged tiles, several tiles per chunk for the small variants
    lib = _lib.load()
    ops = _operands(flow, m, n, k, S, torch.bfloat16, seed=variant)
    try:
        assert lib.ms_set_variant(variant) == 0
        want = _plain(flow, ops, torch.float32)
        counters = torch.zeros(S + 3, dtype=torch.int32, device="cuda")
        got, tiles = _signal(flow, ops, counters, torch.float32)
        used = lib.ms_query(_lib.MS_QUERY_LAST_VARIANT)
    finally:
        lib.ms_set_variant(0)
    torch.cuda.synchronize()
    if variant:
        assert used == variant
    assert tiles >= 1
    assert counters.tolist() == [tiles] * S + [0, 0, 0]
    for s in range(S):
        assert torch.equal(got[s], want[s])


@pytest.mark.parametrize("flow", ["ls", "rs"])
def test_fp32_operands_count_too(flow):
    S, m, n, k = 3, 300, 260, 200
    ops = _operands(flow, m, n, k, S, torch.float32)
    want = _plain(flow, ops, torch.float32)
    counters = torch.zeros(S, dtype=torch.int32, device="cuda")
    got, tiles = _signal(flow, ops, counters, torch.float32)
    torch.cuda.synchronize()
    assert counters.tolist() == [tiles] * S and tiles == ((m + 63) // 64) * ((n + 63) // 64)     # so few tiles run as 64 x 64
    for s in range(S):
        assert torch.equal(got[s], want[s])


def test_counters_are_only_added_to():
    S, m, n, k = 2, 256, 384, 128
    ops = _operands("ls", m, n, k, S, torch.bfloat16)
    counters = torch.full((S,), 7, dtype=torch.int32, device="cuda")
    _, tiles = _signal("ls", ops, counters, torch.bfloat16)
    _, tiles2 = _signal("ls", ops, counters, torch.bfloat16)
    torch.cuda.synchronize()
    assert tiles == tiles2 and counters.tolist() == [7 + 2 * tiles] * S


def test_reserved_compute_units_change_the_grid_not_the_result():
    S, m, n, k = 4, 2048, 1536, 1024
    lib = _lib.load()
    ops = _operands("ls", m, n, k, S, torch.bfloat16)
    want = _plain("ls", ops, torch.bfloat16)
    a, b = _rand((4096, 2048), 5, torch.bfloat16), _rand((2048, 4096), 6, torch.bfloat16, 0.05)
    want_os = ms.gemm_os([a], [b])
    try:
        for reserve in (8, 16, 250, 1024):
            assert lib.ms_set_reserved_cus(reserve) == 0
            got = _plain("ls", ops, torch.bfloat16)
            for s in range(S):
                assert torch.equal(got[s], want[s])
            assert orc_close(ms.gemm_os([a], [b]), want_os)
        assert lib.ms_set_reserved_cus(-1) == _lib.MS_ERR_ARG and lib.ms_set_reserved_cus(1025) == _lib.MS_ERR_ARG
    finally:
        lib.ms_set_reserved_cus(0)
    torch.cuda.synchronize()


def orc_close(x, y):
    """Another tile shape or split of the contraction sums in another order: equal to bf16 rounding, not bit for bit."""
    d = (x.float() - y.float()).norm() / y.float().norm()
    return d.item() <= 1e-2


def test_argument_errors():
    S, m, n, k = 2, 256, 384, 128
    A, W = _operands("ls", m, n, k, S, torch.bfloat16)
    with pytest.raises(ValueError, match="chunk_done"):
        ms.gemm_ls_signal(A, W, torch.zeros(S, dtype=torch.int64, device="cuda"))
    with pytest.raises(ValueError, match="chunk_done"):
        ms.gemm_ls_signal(A, W, torch.zeros(S - 1, dtype=torch.int32, device="cuda"))
    with pytest.raises(ValueError, match="chunk_done"):
        ms.gemm_ls_signal(A, W, torch.zeros(S, dtype=torch.int32))
    # the C entry point refuses null counters
    lib = _lib.load()
    Y = [torch.empty((m, n), dtype=torch.float32, device="cuda") for _ in range(S)]
    wp = (ctypes.c_void_p * S)(*[w.data_ptr() for w in W])
    yp = (ctypes.c_void_p * S)(*[y.data_ptr() for y in Y])
    tiles = ctypes.c_int(-1)
    rc = lib.ms_gemm_ls_signal(ctypes.c_void_p(A.data_ptr()), k, wp, k, S, m, n, k, yp, n, _lib.MS_DTYPE_BF16, _lib.MS_DTYPE_F32,
                               None, ctypes.byref(tiles), None)
    assert rc == _lib.MS_ERR_ARG and b"chunk_done" in lib.ms_last_error() and tiles.value == -1
    torch.cuda.synchronize()


def _watch_once(flow, ops, out, S, m, n, BAND):
    """One counted call on its own stream with a watcher polling from another; returns what the watcher saw."""
    lib = _lib.load()
    counters = torch.zeros(S, dtype=torch.int32, device="cuda")
    seen = torch.zeros(S, dtype=torch.int32).pin_memory()
    bands = [torch.zeros((2, BAND, n), dtype=torch.bfloat16).pin_memory() for _ in range(S)]
    for o in out:
        o.zero_()
    compute, watch = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    try:
        assert lib.ms_set_reserved_cus(16) == 0
        with torch.cuda.stream(compute):
            _, tiles = _signal(flow, ops, counters, torch.bfloat16, out=out)
    finally:
        lib.ms_set_reserved_cus(0)
    history, copied = [], {}
    with torch.cuda.stream(watch):
        for poll in range(400):               # bounded: the watcher gives up, it never waits for the kernel
            seen.copy_(counters, non_blocking=True)
            watch.synchronize()
            now = seen.tolist()
            history.append(now)
            for s in range(S):
                if now[s] == tiles and s not in copied:
                    bands[s][0].copy_(out[s][:BAND], non_blocking=True)
                    bands[s][1].copy_(out[s][m - BAND:], non_blocking=True)
                    watch.synchronize()
                    copied[s] = not compute.query()     # True: the kernel had not ended when the chunk had been read
            if len(copied) == S:
                break
    torch.cuda.synchronize()
    return tiles, counters.tolist(), np.array(history), copied, bands


@pytest.mark.parametrize("flow", ["ls", "rs"])
def test_a_watcher_that_sees_a_chunk_complete_reads_the_finished_chunk(flow):
    S, m, n, k = 8, 8192, 1536, 8192          # about 1.3 ms of kernel: room for some tens of polls
    BAND = 48                                 # rows of a chunk the watcher copies out: its first and its last
    assert _lib.load().ms_query(_lib.MS_QUERY_CU_COUNT) > 16
    ops = _operands(flow, m, n, k, S, torch.bfloat16)
    out = [torch.zeros((m, n), dtype=torch.bfloat16, device="cuda") for _ in range(S)]
    want = _plain(flow, ops, torch.bfloat16)
    tiles, final, h, copied, bands = _watch_once(flow, ops, out, S, m, n, BAND)
    assert final == [tiles] * S
    # counts never decrease and never pass the tile count
    assert (np.diff(h, axis=0) >= 0).all() and h.max() <= tiles
    # whatever the watcher copied after seeing a chunk complete is the finished chunk
    assert len(copied) == S, "400 polls did not outlast the kernel"
    for s in range(S):
        assert torch.equal(out[s], want[s])
        assert torch.equal(bands[s][0], want[s][:BAND].cpu()), f"chunk {s}: first rows read before they were written"
        assert torch.equal(bands[s][1], want[s][m - BAND:].cpu()), f"chunk {s}: last rows read before they were written"
    # (whether any chunk was seen complete while the kernel still ran is a matter of timing: tests/test_zy_gpu_timing.py)
    early = sorted(s for s, r in copied.items() if r)
    print(f"\n{flow}: {len(h)} polls, chunks read while the kernel ran: {early}")
