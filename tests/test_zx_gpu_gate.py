"""Input gate of the output-stationary product (``ms_gemm_os_gated``): one launch that reads slice s only after the
producer of that slice has raised ``slice_ready[s]``, as the reference's OS body multiplies slice k while slice k + 1 is
still being gathered (TensorParallel.py:163-171).

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
@pytest.mark.parametrize("variant", [0, 3, 7, 8, 9, 10, 11, 12, 13, 14, 208])
def test_with_every_flag_set_the_gated_call_equals_the_plain_one(variant, dtype):
    if dtype == torch.float32 and variant:
        pytest.skip("tile variants are those of the bf16 kernels")
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
    if variant and dtype == torch.bfloat16:
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
