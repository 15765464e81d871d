"""Seeded random cases through the C ABI: dataflow x tile variant x operand dtype x output dtype x slice count x
row pitch, drawn together (the fixed lists of test_gpu_parity.py vary one of them at a time).  The expected values
are the oracle's float64 products of the same (dtype-rounded) operands; tolerances: 1e-5 of the result's Frobenius norm for fp32 outputs
(fp32 accumulation of at most 3200 terms), 6e-3 for outputs rounded to bf16."""
import random

import numpy as np
import pytest
import torch

from oracle import meshslice_oracle as orc
import meshslice_amd as ms
from meshslice_amd import _lib

pytestmark = pytest.mark.gpu


def _operand(g, rows, cols, dtype, pad):
    return torch.randn((rows, cols + pad), generator=g, device="cuda").to(dtype)[:, :cols]


def _host(t):
    return t.detach().float().cpu().numpy().astype(np.float64)


@pytest.mark.parametrize("seed", [0, 1, 2, 3])
def test_random_cases(seed):
    lib = _lib.load()
    rnd = random.Random(seed)
    g = torch.Generator(device="cuda").manual_seed(seed)
    try:
        for it in range(60):
            flow = rnd.choice(["os", "ls", "rs"])
            dtype = rnd.choice([torch.bfloat16, torch.bfloat16, torch.float32])
            q = 8 if dtype == torch.bfloat16 else 4
            variant = rnd.choice([0, 0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14]) if dtype == torch.bfloat16 else rnd.choice([0, 0, 21, 22, 23, 24, 25])
            top = 400 if rnd.random() < 0.15 else 120
            m, n, k = q * rnd.randint(1, top), 8 * rnd.randint(1, top), q * rnd.randint(1, 80)
            S = rnd.randint(1, 5)
            out_dtype = rnd.choice([torch.float32, torch.bfloat16])
            pa, pb = q * rnd.randint(0, 3), q * rnd.randint(0, 3)
            case = f"seed {seed} case {it}: {flow} variant {variant} {dtype} -> {out_dtype} m {m} n {n} k {k} S {S} pads {pa}, {pb}"
            assert lib.ms_set_variant(variant) == 0
            if flow == "os":
                A = [_operand(g, m, k, dtype, pa) for _ in range(S)]
                B = [_operand(g, k, n, dtype, pb) for _ in range(S)]
                got = [ms.gemm_os(A, B, out_dtype=out_dtype)]
                want = [orc.oracle_os_block([_host(a) for a in A], [_host(b) for b in B])]
            elif flow == "ls":
                A = _operand(g, m, k, dtype, pa)
                W = [_operand(g, n, k, dtype, pb) for _ in range(S)]
                got = ms.gemm_ls(A, W, out_dtype=out_dtype)
                want = orc.oracle_ls_chunks(_host(A), [_host(w) for w in W])
            else:
                X = [_operand(g, k, m, dtype, pa) for _ in range(S)]
                W = _operand(g, k, n, dtype, pb)
                got = ms.gemm_rs(X, W, out_dtype=out_dtype)
                want = orc.oracle_rs_chunks([_host(x) for x in X], _host(W))
            tol = 1e-5 if out_dtype == torch.float32 else 6e-3
            for y, ref in zip(got, want):
                assert y.dtype == out_dtype, case
                err = orc.rel_frobenius(_host(y), ref)
                assert err <= tol, f"{case}: {err:.3e}"
    finally:
        lib.ms_set_variant(0)
        torch.cuda.synchronize()
