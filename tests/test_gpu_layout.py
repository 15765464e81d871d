"""The block-cyclic layout kernels (ms_pack_slices, ms_unpack_chunks) against the oracle, through the C ABI,
on the GPU.  Pure placement is compared bit for bit; the peer sum runs in fp32 in peer order on both sides
and is compared bit for bit too; bf16 results equal one round-to-nearest-even of that fp32 sum."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import meshslice_oracle as orc
from meshslice_amd import _lib, slice_layout as sl
from meshslice_amd import TensorParallel as TP

pytestmark = pytest.mark.gpu


def _bits(t):
    """Raw element bits of a device tensor as a numpy array."""
    t = t.contiguous()
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).cpu().numpy().view(np.uint16)
    return t.view(torch.int32).cpu().numpy().view(np.uint32)


def _rand(shape, dtype, seed):
    """Random bit patterns of finite values (every exponent, both zeros)."""
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal(shape) * np.exp2(rng.integers(-20, 20, size=shape))).astype(np.float32)
    x[rng.random(shape) < 0.02] = -0.0
    if dtype == torch.bfloat16:
        x = orc.bf16_round(x)
    return x


def _dev(x, dtype):
    return torch.from_numpy(np.ascontiguousarray(x)).cuda().to(dtype)


PACK_CASES = [
    # rows, cols, S, B
    (64, 256, 4, 8), (37, 512, 8, 8), (8, 64, 1, 8), (100, 96, 3, 8), (5, 4096, 16, 8), (1031, 1536, 4, 8),
    (16, 32, 2, 2), (9, 120, 5, 4), (24, 48, 3, 16),
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("r,c,S,B", PACK_CASES)
def test_pack_cols_equals_the_oracle_bit_for_bit(r, c, S, B, dtype):
    x = _rand((r, c), dtype, r + c + S)
    d = _dev(x, dtype)
    got = sl.pack_slices(d, S, B, 1)
    want = orc.pack_slices(x, S, B, 1)
    for g, w in zip(got, want):
        assert tuple(g.shape) == w.shape
        assert np.array_equal(_bits(g), _bits(_dev(w, dtype)))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("c,r,S,B", PACK_CASES)
def test_pack_rows_equals_the_oracle_bit_for_bit(r, c, S, B, dtype):
    x = _rand((r, c), dtype, r + c + S + 1)
    d = _dev(x, dtype)
    got = sl.pack_slices(d, S, B, 0)
    want = orc.pack_slices(x, S, B, 0)
    for g, w in zip(got, want):
        assert np.array_equal(_bits(g), _bits(_dev(w, dtype)))


def test_pack_reads_a_strided_shard_and_writes_into_a_gathered_buffer():
    """The shard is a view of the global matrix (ld > cols); every peer's slices go straight to their place in
    the row-major gathered slices [S][rows, C * cols / S]; nothing else in the buffer is touched."""
    R, C, S, B = 2, 4, 4, 8
    X = _rand((256, 1024), torch.bfloat16, 3)
    dX = _dev(X, torch.bfloat16)
    h, w = 256 // R, 1024 // C
    ws = w // S
    for i in range(R):
        buf = torch.full((S, h, C * ws + 8), 7.0, dtype=torch.bfloat16, device="cuda")
        for jj in range(C):
            sl.pack_slices(dX[i * h:(i + 1) * h, jj * w:(jj + 1) * w], S, B, 1,
                           out=[buf[s][:, jj * ws:(jj + 1) * ws] for s in range(S)])
        for s in range(S):
            want = np.concatenate([orc.pack_slices(orc.shard(X, R, C, i, jj), S, B, 1)[s] for jj in range(C)], axis=1)
            assert np.array_equal(_bits(buf[s][:, :C * ws]), _bits(_dev(want, torch.bfloat16)))
        assert bool((buf[:, :, C * ws:] == 7.0).all())
    # the gathered slices are exactly the operands the closed-form oracle derives for device (i, j)
    As, _ = orc.device_operands_os(X, _rand((1024, 64), torch.bfloat16, 4), R, C, 1, 0, S, B)
    assert np.array_equal(_bits(buf[2][:, :C * ws]), _bits(_dev(As[2], torch.bfloat16)))


UNPACK_CASES = [
    # chunk rows, chunk cols, S, B, parts, P
    (64, 256, 4, 8, 2, 2), (37, 512, 8, 8, 4, 4), (16, 64, 1, 8, 1, 1), (100, 96, 3, 8, 2, 2), (1031, 384, 4, 8, 1, 1),
    (24, 1536, 8, 8, 8, 8), (16, 32, 2, 2, 2, 2), (9, 120, 5, 4, 3, 3), (8, 96, 3, 16, 2, 1),
]


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("axis", [0, 1])
@pytest.mark.parametrize("cr,cc,S,B,parts,P", UNPACK_CASES)
def test_unpack_equals_the_oracle_bit_for_bit(cr, cc, S, B, parts, P, axis, in_dtype, out_dtype):
    if axis == 0:
        cr, cc = cc, cr
    peers = [[_rand((cr, cc), in_dtype, 1000 * p + 10 * s + axis) for s in range(S)] for p in range(P)]
    dpeers = [[_dev(x, in_dtype) for x in peer] for peer in peers]
    for w in sorted({0, parts - 1}):
        got = sl.unpack_chunks(dpeers, B, axis, window=w, parts=parts, out_dtype=out_dtype)
        want = orc.unpack_chunks(peers, B, axis, window=w, parts=parts, out_dtype="bf16" if out_dtype == torch.bfloat16 else np.float32)
        assert tuple(got.shape) == want.shape and got.dtype == out_dtype
        assert np.array_equal(_bits(got), _bits(_dev(want, out_dtype)))


@pytest.mark.parametrize("axis", [0, 1])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_unpack_inverts_pack_at_full_size(axis, dtype):
    """The shard of the large configuration ([4096, 12288], S = 8, B = 8): pack then unpack returns the
    shard bit for bit, the slices hold every element exactly once (sum of element bits), and a padded
    destination stays untouched outside the shard."""
    g = torch.Generator(device="cuda").manual_seed(5 + axis)
    x = torch.randn((4096, 12288), generator=g, device="cuda").to(dtype)
    slices = sl.pack_slices(x, 8, 8, axis)
    as_int = (lambda t: t.contiguous().view(torch.int16 if dtype == torch.bfloat16 else torch.int32).to(torch.int64))
    assert int(sum(as_int(s).sum() for s in slices)) == int(as_int(x).sum())
    k = 5
    idx = torch.from_numpy(orc.sel(x.shape[axis], 8, 8, k)).cuda()
    assert torch.equal(slices[k], x[:, idx] if axis == 1 else x[idx, :])
    pad = torch.full((4096, 12288 + 8), 3.0, dtype=dtype, device="cuda")
    back = sl.unpack_chunks([slices], 8, axis, out=pad[:, :12288])
    assert torch.equal(back, x)
    assert bool((pad[:, 12288:] == 3.0).all())


# ---------------------------------------------------------------- the mesh plumbing built on the kernels
@pytest.mark.parametrize("R,C,K,B", [(2, 2, 2, 2), (4, 2, 8, 8), (2, 4, 4, 8)])
def test_gathered_slices_match_the_closed_form(R, C, K, B):
    """Slice k gathered over the peers == the global matrix indexed with the closed-form rule."""
    L = R * C * K * B * 2
    G = torch.arange(24 * L, dtype=torch.float32).reshape(24, L)
    Xs = TP._shards(G.cuda(), 4, C)
    got = TP._gather_col_slices([Xs[1][jj] for jj in range(C)], K, B)
    for k in range(K):
        assert torch.equal(got[k].cpu(), G[6:12][:, torch.from_numpy(orc.sel(L, K, B, k))])
    Gt = G.t().contiguous()
    Ws = TP._shards(Gt.cuda(), R, 4)
    got = TP._gather_row_slices([Ws[ii][2] for ii in range(R)], K, B)
    for k in range(K):
        assert torch.equal(got[k].cpu(), Gt[:, 12:18][torch.from_numpy(orc.sel(L, K, B, k)), :])


@pytest.mark.parametrize("R,C,S,B", [(2, 2, 2, 2), (4, 2, 4, 8), (2, 4, 2, 8), (8, 2, 16, 8)])
def test_chunk_assembly_matches_the_oracle(R, C, S, B):
    """psum_scatter + interleave of integer-valued chunks (exact in fp32) == the closed-form assembly; the last
    case has more chunk pointers than one launch takes and sums the peers first."""
    rng = np.random.default_rng(11)
    O = R * C * S * B * 2
    m = 6
    chunks = [[rng.integers(-5, 6, (m, O // S)).astype(np.float32) for _ in range(S)] for _ in range(C)]
    tch = [[torch.from_numpy(c).cuda() for c in row] for row in chunks]
    for j in range(C):
        got = TP._finish(tch, j, 1, B, torch.float32).cpu().numpy()
        assert np.array_equal(got, orc.assemble_ls(chunks, R, C, j, S, B))
    n = 5
    chunks = [[rng.integers(-5, 6, (O // S, n)).astype(np.float32) for _ in range(S)] for _ in range(R)]
    tch = [[torch.from_numpy(c).cuda() for c in row] for row in chunks]
    for i in range(R):
        got = TP._finish(tch, i, 0, B, torch.bfloat16).float().cpu().numpy()
        assert np.array_equal(got, orc.assemble_rs(chunks, R, C, i, S, B))


def test_peer_major_gathered_slices_are_ingested_without_a_repack():
    """A library all-gather along the columns leaves slice k peer-major, [C][m, k_slice / C].  The
    output-stationary call takes that as S * C slice pairs (the weights' slice k is cut at the same k
    offsets by pointer arithmetic alone), so no transposing copy is needed; the result equals the one from
    the row-major gathered slices and the oracle's."""
    import meshslice_amd as ms
    R, C, S, B = 2, 4, 4, 8
    rng = np.random.default_rng(21)
    X = orc.bf16_round(rng.standard_normal((512, 4096)).astype(np.float32))
    W = orc.bf16_round(rng.standard_normal((4096, 768)).astype(np.float32) * 0.05)
    dX, dW = _dev(X, torch.bfloat16), _dev(W, torch.bfloat16)
    Xs, Ws = TP._shards(dX, R, C), TP._shards(dW, R, C)
    i, j = 1, 2
    A_rm = TP._gather_col_slices([Xs[i][jj] for jj in range(C)], S, B)       # S x [256, 1024]
    B_rm = TP._gather_row_slices([Ws[ii][j] for ii in range(R)], S, B)       # S x [1024, 192]
    c_rm = ms.gemm_os(A_rm, B_rm, out_dtype=torch.float32)
    ks = 4096 // C // S
    A_pm = [p for k in range(S) for p in [sl.pack_slices(Xs[i][jj], S, B, 1)[k] for jj in range(C)]]
    B_pm = [B_rm[k][jj * ks:(jj + 1) * ks] for k in range(S) for jj in range(C)]
    assert len(A_pm) == S * C and tuple(A_pm[0].shape) == (256, ks) and tuple(B_pm[0].shape) == (ks, 192)
    c_pm = ms.gemm_os(A_pm, B_pm, out_dtype=torch.float32)
    want = orc.oracle_os_block(*orc.device_operands_os(X, W, R, C, i, j, S, B))
    assert orc.rel_frobenius(c_pm.cpu().numpy().astype(np.float64), want) <= 1e-2
    assert orc.rel_frobenius(c_pm.cpu().numpy().astype(np.float64), c_rm.cpu().numpy().astype(np.float64)) <= 1e-6


def test_device_step_is_capturable_in_a_hip_graph():
    """One device's step of the LHS-stationary dataflow — cut the weight shard into slices, multiply, reduce and
    interleave the chunks — captured once and replayed with new operand values each time; every replay equals
    the eager result bit for bit (kernel launches only: no allocation, no memset inside the calls)."""
    import meshslice_amd as ms
    S, B = 4, 8
    g = torch.Generator(device="cuda").manual_seed(31)
    x = torch.randn((256, 512), generator=g, device="cuda").to(torch.bfloat16)
    w = (torch.randn((768, 512), generator=g, device="cuda") * 0.05).to(torch.bfloat16)          # [out, in] shard
    wsl = [torch.empty((768 // S, 512), dtype=torch.bfloat16, device="cuda") for _ in range(S)]
    chunks = [torch.empty((256, 768 // S), dtype=torch.float32, device="cuda") for _ in range(S)]
    y = torch.empty((256, 768), dtype=torch.bfloat16, device="cuda")

    def step():
        sl.pack_slices(w, S, B, 0, out=wsl)
        ms.gemm_ls(x, wsl, out=chunks)
        sl.unpack_chunks([chunks], B, 1, out=y)
    step()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for rep in range(3):
        x.copy_(torch.randn((256, 512), generator=g, device="cuda").to(torch.bfloat16))
        w.mul_(-1.5)
        step()
        want = y.clone()
        y.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, want), f"replay {rep} differs from the eager step"
        ref = x.double() @ w.double().t()
        assert orc.rel_frobenius(y.double().cpu().numpy(), ref.cpu().numpy()) <= 1e-2


def test_layout_calls_reject_bad_arguments():
    L = _lib.load()
    x = torch.zeros((64, 64), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError):
        sl.pack_slices(x, 3, 8, 1)                      # 64 is not a multiple of 3 * 8
    with pytest.raises(ValueError):
        sl.pack_slices(x, 2, 8, 2)
    with pytest.raises(ValueError):
        sl.pack_slices(x, 2, 8, 1, out=[torch.zeros((64, 16), dtype=torch.bfloat16, device="cuda")] * 2)
    with pytest.raises(_lib.MeshSliceError):
        sl.pack_slices(x.cpu(), 2, 8, 1)
    with pytest.raises(ValueError):
        sl.unpack_chunks([[x, x]], 8, 1, window=2, parts=2)
    with pytest.raises(ValueError):
        sl.unpack_chunks([[x, x]], 8, 1, parts=16)      # windows of 4 columns are not whole blocks of 8
    # straight through the C ABI: too many pointers, unknown dtype, null table
    ptrs, _keep = _lib.ptr_array([x.data_ptr()] * 72)
    null = ctypes.c_void_p(None)
    assert L.ms_unpack_chunks(ptrs, 9, 8, 64, 0, 0, 64, 512, 1, 8, ctypes.c_void_p(x.data_ptr()), 512, 1, 1, null) == _lib.MS_ERR_ARG
    assert "P*S" in _lib.last_error()
    assert L.ms_pack_slices(ctypes.c_void_p(x.data_ptr()), 64, 64, 64, 1, 2, 8, ptrs, 32, 7, null) == _lib.MS_ERR_UNSUPPORTED
    assert L.ms_pack_slices(ctypes.c_void_p(x.data_ptr()), 64, 64, 64, 1, 2, 8, None, 32, 1, null) == _lib.MS_ERR_ARG
    assert L.ms_pack_slices(ctypes.c_void_p(x.data_ptr()), 32, 64, 64, 1, 2, 8, ptrs, 32, 1, null) == _lib.MS_ERR_ARG
