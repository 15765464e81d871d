"""The library's default tile choice on products OUTSIDE the GPT-3 family the chooser's constants were first tuned on
(Llama-like 4096 x 11008, cubes, tall / wide / short-contraction shapes): right against the float64 oracle on sampled
rows, and the grid sizes the launches use.  (How FAST the default is against every forced variant is a wall-clock
question: tests/test_zy_gpu_timing.py, collected after every parity file.)"""

import numpy as np
import pytest
import torch

from oracle import meshslice_oracle as orc
import meshslice_amd as ms
from meshslice_amd import _lib

pytestmark = pytest.mark.gpu
SHAPES = [(4096, 11008, 4096), (5120, 5120, 5120), (3008, 7040, 4992), (1024, 8192, 8192), (6144, 6144, 2048),
          (12288, 1024, 4096), (16384, 4096, 1024)]


def _rand(shape, seed, scale):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return (torch.randn(shape, generator=g, device="cuda") * scale).to(torch.bfloat16)


def operands(flow, shape, S=2):
    """(run, check) for one product of ``shape`` in dataflow ``flow`` with S slices: ``run()`` launches it with the
    library's current variant, ``check()`` compares sampled rows of its output with the float64 oracle."""
    m, n, k = shape
    f64 = lambda t: t.float().cpu().numpy().astype(np.float64)
    rows = np.random.default_rng(0).choice(m if flow != "rs" else m // S, 8, replace=False)
    if flow == "os":
        A = [_rand((m, k // S), s, 1.0) for s in range(S)]
        B = [_rand((k // S, n), 10 + s, 0.02) for s in range(S)]
        C = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
        run = lambda: ms.gemm_os(A, B, out=C)
        check = lambda: orc.rel_frobenius(f64(C[rows]), sum(f64(a[rows]) @ f64(b) for a, b in zip(A, B)))
    elif flow == "ls":
        A = _rand((m, k), 1, 1.0)
        W = [_rand((n // S, k), 10 + s, 0.02) for s in range(S)]
        Y = [torch.empty((m, n // S), dtype=torch.bfloat16, device="cuda") for _ in range(S)]
        run = lambda: ms.gemm_ls(A, W, out=Y)
        check = lambda: orc.rel_frobenius(f64(Y[1][rows]), f64(A[rows]) @ f64(W[1]).T)
    else:
        X = [_rand((k, m // S), s, 1.0) for s in range(S)]
        W = _rand((k, n), 9, 0.02)
        Y = [torch.empty((m // S, n), dtype=torch.bfloat16, device="cuda") for _ in range(S)]
        run = lambda: ms.gemm_rs(X, W, out=Y)
        check = lambda: orc.rel_frobenius(f64(Y[1][rows]), f64(X[1][:, rows]).T @ f64(W))
    return run, check


@pytest.mark.parametrize("flow", ["os", "ls", "rs"])
@pytest.mark.parametrize("shape", SHAPES, ids=["x".join(map(str, s)) for s in SHAPES])
def test_default_choice_is_right_on_products_outside_the_gpt3_family(flow, shape):
    """Whatever tile shape, launch count and split the library picks for these products, the result is the oracle's."""
    lib = _lib.load()
    assert lib.ms_set_variant(0) == 0
    run, check = operands(flow, shape)
    run()
    assert 1 <= lib.ms_query(_lib.MS_QUERY_LAST_VARIANT) <= 14
    assert check() <= 1e-2


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
        for variant, tiles in ((7, 400), (13, 400), (12, 20 * 14), (11, 14 * 27), (8, 20 * 27), (3, 1600)):
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
