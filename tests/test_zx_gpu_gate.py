"""Input gate of the sliced products (``ms_gemm_os_gated``, ``ms_gemm_ls_gated``, ``ms_gemm_rs_gated``): one launch that
reads gathered slice s only after the producer of that slice has raised ``slice_ready[s]``, as the reference's bodies
multiply slice k while slice k + 1 is still being gathered (TensorParallel.py:163-171, :176-189, :198-212).

With every flag set before the call the result equals the plain call's bit for bit; with the slices filled and flagged
by a second stream AFTER the launch the result is still the product of the filled data (the kernel waited); a flag that
is never raised makes the kernel give up after its time limit, end normally and say so in the status word (the limit is
a few milliseconds there: no test makes the GPU wait for long, and none can hang it).
"""
import time

import numpy as np
import pytest
import torch

import meshslice_amd as ms
from meshslice_amd import _lib
from oracle import meshslice_oracle as orc

pytestmark = pytest.mark.gpu


def _rand(shape, seed, dtype, scale=1.0):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return (torch.randn(shape, generator=g, device="cuda") * scale).to(dtype)


def _slices(m, n, k, S, dtype, seed):
    return [_rand((m, k), seed + s, dtype) for s in range(S)], [_rand((k, n), seed + 100 + s, dtype, 0.05) for s in range(S)]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("variant", [0, 3, 7, 8, 9, 10, 11, 12, 13, 14, 208, 21, 22, 23, 24, 25, 221, 322])
def test_with_every_flag_set_the_gated_call_equals_the_plain_one(variant, dtype):
    if variant and (dtype == torch.float32) != (variant % 100 >= 21):
        pytest.skip("variants 1-14 are tiles of the bf16 kernels, 21-25 of the fp32 kernel")
    S, m, n, k = 3, 520, 776, 136       # ragged tiles, a K tail in every slice
    A, B = _slices(m, n, k, S, dtype, seed=variant)
    lib = _lib.load()
    ready = torch.ones(S + 1, dtype=torch.int32, device="cuda")
    ready[S] = 0
    try:
        assert lib.ms_set_variant(variant) == 0
        want = ms.gemm_os(A, B)
        got = ms.gemm_os_gated(A, B, ready)
        used = lib.ms_query(_lib.MS_QUERY_LAST_VARIANT)
    finally:
        lib.ms_set_variant(0)
    torch.cuda.synchronize()
    if variant:
        assert used == variant % 100
    assert torch.equal(got, want)
    assert not ms.gate_timed_out(ready)
    tol = 1e-2 if dtype == torch.bfloat16 else 1e-5
    assert orc.rel_frobenius(got.float().cpu().numpy(), orc.oracle_os_block([a.float().cpu().numpy() for a in A], [b.float().cpu().numpy() for b in B])) <= tol


def test_slices_filled_and_flagged_by_another_stream_after_the_launch():
    """The operand buffers hold zeros when the product is launched; a second stream then fills slice after slice and
    raises its flag.  A kernel that read a slice before its flag would add zeros for it."""
    S, m, n, k = 4, 2048, 3072, 1024
    src_a, src_b = _slices(m, n, k, S, torch.bfloat16, seed=7)
    want = ms.gemm_os(src_a, src_b)
    A = [torch.zeros_like(t) for t in src_a]; B = [torch.zeros_like(t) for t in src_b]
    ready = torch.zeros(S + 1, dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()
    lib = _lib.load()
    producer = torch.cuda.Stream()
    try:
        assert lib.ms_set_reserved_cus(16) == 0      # the producer's copies need compute units beside the waiting product
        got = ms.gemm_os_gated(A, B, ready, timeout_ms=1500)
    finally:
        lib.ms_set_reserved_cus(0)
    time.sleep(0.003)                                # the product is on the device and waiting for slice 0
    with torch.cuda.stream(producer):
        for s in range(S):
            A[s].copy_(src_a[s]); B[s].copy_(src_b[s])
            ms.signal_set(ready, s)
    torch.cuda.synchronize()
    if ms.gate_timed_out(ready):
        # whether a second stream's kernels overtake a waiting launch is the runtime's to decide (its streams share a
        # few hardware queues); the kernel has ended by its time limit, which is what must always hold
        pytest.skip("the producer's copies did not run beside the waiting product on this machine")
    assert ready[:S].tolist() == [1] * S
    assert torch.equal(got, want)


def test_a_flag_that_is_never_raised_ends_the_kernel_after_its_time_limit():
    S, m, n, k = 3, 512, 768, 256
    A, B = _slices(m, n, k, S, torch.bfloat16, seed=11)
    ready = torch.tensor([1, 0, 1, 0], dtype=torch.int32, device="cuda")
    t0 = time.time()
    ms.gemm_os_gated(A, B, ready, timeout_ms=5)
    torch.cuda.synchronize()
    assert time.time() - t0 < 5.0
    assert ms.gate_timed_out(ready)
    assert ready[:S].tolist() == [1, 0, 1]           # the kernel only ever writes the status word
    # the same flags, cleared and complete, give the product
    ready.fill_(1); ready[S] = 0
    got = ms.gemm_os_gated(A, B, ready, timeout_ms=5)
    torch.cuda.synchronize()
    assert not ms.gate_timed_out(ready)
    assert torch.equal(got, ms.gemm_os(A, B))


def test_the_gated_call_checks_its_arguments():
    S, m, n, k = 2, 128, 128, 128
    A, B = _slices(m, n, k, S, torch.bfloat16, seed=3)
    good = torch.ones(S + 1, dtype=torch.int32, device="cuda"); good[S] = 0
    with pytest.raises(ValueError):
        ms.gemm_os_gated(A, B, torch.ones(S, dtype=torch.int32, device="cuda"))
    with pytest.raises(ValueError):
        ms.gemm_os_gated(A, B, torch.ones(S + 1, dtype=torch.int64, device="cuda"))
    with pytest.raises(ValueError):
        ms.gemm_os_gated(A, B, torch.ones(S + 1, dtype=torch.int32))
    with pytest.raises(ValueError):
        ms.gemm_os_gated(A, B, good, timeout_ms=0)
    lib = _lib.load()
    try:
        assert lib.ms_set_variant(1) == 0            # 256x256 on four waves of the ring kernel has no gate
        with pytest.raises(_lib.MeshSliceError):
            ms.gemm_os_gated(A, B, good)
    finally:
        lib.ms_set_variant(0)
    with pytest.raises(IndexError):
        ms.signal_set(good, S + 1)
    ms.signal_set(good, S, 5)
    torch.cuda.synchronize()
    assert good.tolist() == [1, 1, 5]


def _chunk_operands(flow, m, n, k, S, dtype, seed):
    """(operands of gemm_ls / gemm_rs with S chunks of m x n over contraction k, index of the gathered one)"""
    if flow == "ls":
        return [_rand((m, k), seed, dtype), [_rand((n, k), seed + 1 + s, dtype, 0.05) for s in range(S)]], 1
    return [[_rand((k, m), seed + 1 + s, dtype) for s in range(S)], _rand((k, n), seed, dtype, 0.05)], 0


def _plain(flow, ops, **kw):
    return (ms.gemm_ls if flow == "ls" else ms.gemm_rs)(*ops, **kw)


def _gated(flow, ops, ready, **kw):
    return (ms.gemm_ls_gated if flow == "ls" else ms.gemm_rs_gated)(*ops, ready, **kw)


@pytest.mark.parametrize("flow", ["ls", "rs"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("variant", [0, 3, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14])
def test_with_every_flag_set_the_gated_chunk_calls_equal_the_plain_ones(variant, dtype, flow):
    if dtype == torch.float32 and variant:
        pytest.skip("tile variants are those of the bf16 kernels")
    S, m, n, k = 3, 520, 392, 136       # ragged tiles, a K tail
    ops, _ = _chunk_operands(flow, m, n, k, S, dtype, seed=variant)
    lib = _lib.load()
    ready = torch.ones(S + 1, dtype=torch.int32, device="cuda")
    ready[S] = 0
    done = torch.zeros(S, dtype=torch.int32, device="cuda")
    try:
        assert lib.ms_set_variant(variant) == 0
        want = _plain(flow, ops)
        got = _gated(flow, ops, ready)
        used = lib.ms_query(_lib.MS_QUERY_LAST_VARIANT)
        counted, tiles = _gated(flow, ops, ready, chunk_done=done, out_dtype=torch.bfloat16)
        want_bf16 = _plain(flow, ops, out_dtype=torch.bfloat16)
    finally:
        lib.ms_set_variant(0)
    torch.cuda.synchronize()
    if variant and dtype == torch.bfloat16:
        assert used == variant
    assert not ms.gate_timed_out(ready)
    assert done.tolist() == [tiles] * S and tiles > 0
    for s in range(S):
        assert torch.equal(got[s], want[s]), f"chunk {s}"
        assert torch.equal(counted[s], want_bf16[s]), f"chunk {s} with counters"
    host = [[t.float().cpu().numpy() for t in o] if isinstance(o, list) else o.float().cpu().numpy() for o in ops]
    ref = orc.oracle_ls_chunks(*host) if flow == "ls" else orc.oracle_rs_chunks(*host)
    tol = 1e-2 if dtype == torch.bfloat16 else 1e-5
    for s in range(S):
        assert orc.rel_frobenius(got[s].float().cpu().numpy(), ref[s]) <= tol


@pytest.mark.parametrize("flow", ["ls", "rs"])
def test_chunk_slices_flagged_in_reverse_order_by_another_stream_after_the_launch(flow):
    """The gathered operand's buffers hold zeros at the launch; a second stream fills them LAST SLICE FIRST and raises
    each flag, and the completion counters are watched: every chunk is the product of the filled data, so each
    workgroup waited for its own chunk's flag and for no other."""
    S, m, n, k = 4, 1024, 768, 1024
    src, which = _chunk_operands(flow, m, n, k, S, torch.bfloat16, seed=31)
    lib = _lib.load()
    ops = list(src)
    ops[which] = [torch.zeros_like(t) for t in src[which]]
    ready = torch.zeros(S + 1, dtype=torch.int32, device="cuda")
    done = torch.zeros(S, dtype=torch.int32, device="cuda")
    producer = torch.cuda.Stream()
    try:
        assert lib.ms_set_reserved_cus(32) == 0      # the producer's copies need compute units beside the waiting product
        want = _plain(flow, src)
        torch.cuda.synchronize()
        got, tiles = _gated(flow, ops, ready, chunk_done=done, timeout_ms=1500)
    finally:
        lib.ms_set_reserved_cus(0)
    time.sleep(0.003)                                # the product is on the device and waiting
    with torch.cuda.stream(producer):
        for s in reversed(range(S)):
            ops[which][s].copy_(src[which][s])
            ms.signal_set(ready, s)
    torch.cuda.synchronize()
    if ms.gate_timed_out(ready):
        pytest.skip("the producer's copies did not run beside the waiting product on this machine")
    assert done.tolist() == [tiles] * S
    for s in range(S):
        assert torch.equal(got[s], want[s]), f"chunk {s}"


@pytest.mark.parametrize("flow", ["ls", "rs"])
def test_a_chunk_whose_flag_is_never_raised_leaves_the_other_chunks_intact(flow):
    S, m, n, k = 3, 512, 384, 256
    ops, _ = _chunk_operands(flow, m, n, k, S, torch.bfloat16, seed=41)
    want = _plain(flow, ops)
    ready = torch.tensor([1, 0, 1, 0], dtype=torch.int32, device="cuda")
    t0 = time.time()
    got = _gated(flow, ops, ready, timeout_ms=5)
    torch.cuda.synchronize()
    assert time.time() - t0 < 5.0
    assert ms.gate_timed_out(ready)
    assert ready[:S].tolist() == [1, 0, 1]
    assert torch.equal(got[0], want[0]) and torch.equal(got[2], want[2])      # chunks are independent products


def test_the_gated_chunk_calls_check_their_arguments():
    S, m, n, k = 2, 128, 128, 128
    ops, _ = _chunk_operands("ls", m, n, k, S, torch.bfloat16, seed=5)
    good = torch.ones(S + 1, dtype=torch.int32, device="cuda"); good[S] = 0
    with pytest.raises(ValueError):
        ms.gemm_ls_gated(*ops, torch.ones(S, dtype=torch.int32, device="cuda"))
    with pytest.raises(ValueError):
        ms.gemm_ls_gated(*ops, good, timeout_ms=60001)
    with pytest.raises(ValueError):
        ms.gemm_ls_gated(*ops, good, chunk_done=torch.zeros(S - 1, dtype=torch.int32, device="cuda"))
    # through the C ABI: counters without a place for the tile count
    import ctypes
    lib = _lib.load()
    A, W = ops
    Y = [torch.empty((m, n), dtype=torch.float32, device="cuda") for _ in range(S)]
    pw = (ctypes.c_void_p * S)(*[w.data_ptr() for w in W]); py = (ctypes.c_void_p * S)(*[y.data_ptr() for y in Y])
    done = torch.zeros(S, dtype=torch.int32, device="cuda")
    rc = lib.ms_gemm_ls_gated(ctypes.c_void_p(A.data_ptr()), k, pw, k, S, m, n, k, py, n, _lib.MS_DTYPE_BF16, _lib.MS_DTYPE_F32,
                              ctypes.c_void_p(done.data_ptr()), None, ctypes.c_void_p(good.data_ptr()), 100, None)
    assert rc == _lib.MS_ERR_ARG and "come together" in lib.ms_last_error().decode()
    rc = lib.ms_gemm_ls_gated(ctypes.c_void_p(A.data_ptr()), k, pw, k, S, m, n, k, py, n, _lib.MS_DTYPE_BF16, _lib.MS_DTYPE_F32,
                              None, None, None, 100, None)
    assert rc == _lib.MS_ERR_ARG and "slice_ready" in lib.ms_last_error().decode()
    torch.cuda.synchronize()


def test_the_mesh_body_that_launches_the_product_ahead_of_its_gathers_equals_meshflow():
    """SPMD(mesh, 'meshflow_overlap').OS(K): every device launches its gated product first and fills the gathered slices
    afterwards on a second stream, slice by slice; the global result equals MeshFlow's bit for bit."""
    from meshslice_amd import TensorParallel as TP
    from meshslice_amd.mesh import Mesh, create_device_mesh
    mesh = Mesh(create_device_mesh((2, 2)), ("x", "y"))
    X = _rand((512, 1024), 21, torch.bfloat16); W = _rand((1024, 768), 22, torch.bfloat16, 0.05)
    lib = _lib.load()
    try:
        # (the overlapped body leaves compute units to its gathers; the tile choice, and with it the order of the
        # additions, follows the units a product may use)
        assert lib.ms_set_reserved_cus(TP.OVERLAP_RESERVED_CUS) == 0
        want = TP.SPMD(mesh, "meshflow").OS(4)(X, W)
    finally:
        lib.ms_set_reserved_cus(0)
    try:
        got = TP.SPMD(mesh, "meshflow_overlap").OS(4)(X, W)
    except _lib.MeshSliceError as e:
        if "gave up waiting" in str(e):
            pytest.skip("the gather stream did not run beside the waiting product on this machine")
        raise
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    plain = TP.SPMD(mesh, "meshflow").OS(4)(X, W)
    assert orc.rel_frobenius(got.float().cpu().numpy(), plain.float().cpu().numpy()) <= 1e-2


@pytest.mark.parametrize("flow", ["ls", "rs"])
def test_the_chunk_producing_mesh_bodies_launched_ahead_of_their_gathers_equal_meshflow(flow):
    from meshslice_amd import TensorParallel as TP
    from meshslice_amd.mesh import Mesh, create_device_mesh
    mesh = Mesh(create_device_mesh((2, 2)), ("x", "y"))
    if flow == "ls":
        X = _rand((512, 1024), 23, torch.bfloat16); W = _rand((768, 1024), 24, torch.bfloat16, 0.05)
    else:
        X = _rand((1024, 512), 25, torch.bfloat16); W = _rand((1024, 768), 26, torch.bfloat16, 0.05)
    lib = _lib.load()
    try:
        assert lib.ms_set_reserved_cus(TP.OVERLAP_RESERVED_CUS) == 0
        want = getattr(TP.SPMD(mesh, "meshflow"), flow.upper())(4)(X, W)
    finally:
        lib.ms_set_reserved_cus(0)
    try:
        got = getattr(TP.SPMD(mesh, "meshflow_overlap"), flow.upper())(4)(X, W)
    except _lib.MeshSliceError as e:
        if "gave up waiting" in str(e):
            pytest.skip("the gather stream did not run beside the waiting product on this machine")
        raise
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    dense = (X.float() @ W.float().T) if flow == "ls" else (X.float().T @ W.float())
    assert orc.rel_frobenius(got.float().cpu().numpy(), dense.cpu().numpy()) <= 1e-2
