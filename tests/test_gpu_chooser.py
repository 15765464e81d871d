"""The library's default tile choice against every forced variant on products OUTSIDE the GPT-3 family the chooser's
constants were first tuned on (Llama-like 4096 x 11008, cubes, tall / wide / short-contraction shapes): the default
must be within 15 % of the best variant's time, and right (float64 oracle on sampled rows).

Times are sustained wall-clock means (warm-up, then a loop between two synchronisations), the best of two rounds per
candidate, so that one host hiccup does not decide the comparison."""
import time

import numpy as np
import pytest
import torch

from oracle import meshslice_oracle as orc
import meshslice_amd as ms
from meshslice_amd import _lib

pytestmark = pytest.mark.gpu
SHAPES = [(4096, 11008, 4096), (5120, 5120, 5120), (3008, 7040, 4992), (1024, 8192, 8192), (6144, 6144, 2048),
          (12288, 1024, 4096), (16384, 4096, 1024)]
SLACK = 1.15


def _rand(shape, seed, scale):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return (torch.randn(shape, generator=g, device="cuda") * scale).to(torch.bfloat16)


def _sustained(f, warm=10, steps=25):
    for _ in range(warm):
        f()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        f()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


@pytest.mark.parametrize("flow", ["os", "ls", "rs"])
@pytest.mark.parametrize("shape", SHAPES, ids=["x".join(map(str, s)) for s in SHAPES])
def test_default_choice_is_close_to_the_best_variant(flow, shape):
    m, n, k = shape
    S = 2
    lib = _lib.load()
    if flow == "os":
        A = [_rand((m, k // S), s, 1.0) for s in range(S)]
        B = [_rand((k // S, n), 10 + s, 0.02) for s in range(S)]
        C = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
        run = lambda: ms.gemm_os(A, B, out=C)
    elif flow == "ls":
        A = _rand((m, k), 1, 1.0)
        W = [_rand((n // S, k), 10 + s, 0.02) for s in range(S)]
        Y = [torch.empty((m, n // S), dtype=torch.bfloat16, device="cuda") for _ in range(S)]
        run = lambda: ms.gemm_ls(A, W, out=Y)
    else:
        X = [_rand((k, m // S), s, 1.0) for s in range(S)]
        W = _rand((k, n), 9, 0.02)
        Y = [torch.empty((m // S, n), dtype=torch.bfloat16, device="cuda") for _ in range(S)]
        run = lambda: ms.gemm_rs(X, W, out=Y)
    times = {}
    try:
        for rnd in range(2):
            for v in range(0, 13):
                assert lib.ms_set_variant(v) == 0
                t = _sustained(run)
                times[v] = min(times.get(v, t), t)
                if v == 0:
                    picked = (int(lib.ms_query(_lib.MS_QUERY_LAST_VARIANT)), int(lib.ms_query(_lib.MS_QUERY_LAST_SPLITS)),
                              int(lib.ms_query(_lib.MS_QUERY_LAST_LAUNCHES)))
    finally:
        lib.ms_set_variant(0)
    best_v = min(range(1, 13), key=lambda v: times[v])
    if times[0] > SLACK * times[best_v]:
        # a host hiccup during the default's loops reads like a bad choice: time the two again before judging
        try:
            for v in (0, best_v, 0, best_v):
                assert lib.ms_set_variant(v) == 0
                times[v] = min(times[v], _sustained(run))
        finally:
            lib.ms_set_variant(0)
    assert times[0] <= SLACK * times[best_v], (
        f"default (variant {picked[0]}, {picked[1]} split(s), {picked[2]} launch(es)) {times[0] * 1e6:.0f} us; "
        f"variant {best_v} {times[best_v] * 1e6:.0f} us; all: " + " ".join(f"{v}:{t * 1e6:.0f}" for v, t in times.items()))
    # and the default's result is right
    run()
    rows = np.random.default_rng(0).choice(m if flow != "rs" else m // S, 8, replace=False)
    f64 = lambda t: t.float().cpu().numpy().astype(np.float64)
    if flow == "os":
        want = sum(f64(a[rows]) @ f64(b) for a, b in zip(A, B))
        got = f64(C[rows])
    elif flow == "ls":
        want, got = f64(A[rows]) @ f64(W[1]).T, f64(Y[1][rows])
    else:
        want, got = f64(X[1][:, rows]).T @ f64(W), f64(Y[1][rows])
    assert orc.rel_frobenius(got, want) <= 1e-2


def test_a_partly_filled_last_round_becomes_whole_rounds_on_fewer_units():
    """400 tiles of 256x256 on a device of 256 units are two rounds: the launch uses 200 workgroups (a multiple of 8),
    not 256 and then 144; the units it reserves come off first; a launch that fits one round uses one workgroup per tile."""
    lib = _lib.load()
    cus = int(lib.ms_query(_lib.MS_QUERY_CU_COUNT))
    A = [_rand((5120, 256), 1, 1.0)]; B = [_rand((256, 5120), 2, 0.02)]
    C = torch.empty((5120, 5120), dtype=torch.bfloat16, device="cuda")

    def balanced(items, units):
        if items <= units:
            return items
        rounds = -(-items // units)
        return min(units, -(-(-(-items // rounds)) // 8) * 8)

    try:
        for variant, tiles in ((7, 400), (12, 20 * 14), (11, 14 * 27), (8, 20 * 27), (3, 1600)):
            for reserve in (0, 16):
                assert lib.ms_set_variant(variant) == 0 and lib.ms_set_reserved_cus(reserve) == 0
                ms.gemm_os(A, B, out=C)
                per_unit = 2 if variant == 3 and reserve == 0 else 1      # two 128 x 128 workgroups share a unit unless units are reserved
                assert lib.ms_query(_lib.MS_QUERY_LAST_GRID) == balanced(tiles, per_unit * (cus - reserve)), (variant, reserve)
        assert lib.ms_set_variant(7) == 0 and lib.ms_set_reserved_cus(0) == 0
        ms.gemm_os([A[0][:1024]], B, out=C[:1024])
        assert lib.ms_query(_lib.MS_QUERY_LAST_GRID) == min(cus, 4 * 20)
    finally:
        lib.ms_set_variant(0); lib.ms_set_reserved_cus(0)
    torch.cuda.synchronize()
