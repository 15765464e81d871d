"""Pins the C restatement (oracle/ms_oracle.c) against exact closed forms and the numpy oracle."""
import ctypes
import os
import subprocess

import numpy as np
import pytest

from oracle import meshslice_oracle as orc

HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_DIR = os.path.join(os.path.dirname(HERE), "oracle")


@pytest.fixture(scope="module")
def lib():
    so = os.path.join(ORACLE_DIR, "libms_oracle.so")
    if not os.path.exists(so):
        subprocess.check_call(["make", "-C", ORACLE_DIR, "libms_oracle.so"])
    L = ctypes.CDLL(so)
    fp = ctypes.POINTER(ctypes.c_float); dp = ctypes.POINTER(ctypes.c_double)
    for name in ("ms_oracle_meshflow_os", "ms_oracle_meshflow_ls", "ms_oracle_meshflow_rs"):
        f = getattr(L, name)
        f.argtypes = [fp, fp, ctypes.c_long, ctypes.c_long, ctypes.c_long,
                      ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, dp]
        f.restype = ctypes.c_int
    L.ms_oracle_bf16_round.argtypes = [fp, fp, ctypes.c_long]
    L.ms_oracle_bf16_round.restype = None
    return L


def _run(lib, dataflow, X, W, R, C, S, B):
    X = np.ascontiguousarray(X, np.float32); W = np.ascontiguousarray(W, np.float32)
    fp = ctypes.POINTER(ctypes.c_float); dp = ctypes.POINTER(ctypes.c_double)
    if dataflow == "os":
        Y = np.empty((X.shape[0], W.shape[1]), np.float64); dims = (X.shape[0], X.shape[1], W.shape[1])
    elif dataflow == "ls":
        Y = np.empty((X.shape[0], W.shape[0]), np.float64); dims = (X.shape[0], X.shape[1], W.shape[0])
    else:
        Y = np.empty((X.shape[1], W.shape[1]), np.float64); dims = (X.shape[0], X.shape[1], W.shape[1])
    rc = getattr(lib, "ms_oracle_meshflow_" + dataflow)(
        X.ctypes.data_as(fp), W.ctypes.data_as(fp), *dims, R, C, S, B, Y.ctypes.data_as(dp))
    return rc, Y


@pytest.mark.parametrize("dataflow", ["os", "ls", "rs"])
def test_c_oracle_notebook_exact(lib, dataflow):
    d = orc.notebook_inputs(np.float32)
    R, C = d["mesh"]
    X, W = {"os": (d["X"], d["W"]), "ls": (d["dY"], d["W"]), "rs": (d["X"], d["dY"])}[dataflow]
    rc, Y = _run(lib, dataflow, X, W, R, C, d["K"], d["blocksize"])
    assert rc == 0
    # all values are integers over powers of two: the double sums are exact in any order
    assert np.array_equal(Y, orc.dense(dataflow, X, W))


@pytest.mark.parametrize("R,C,S,B", [(2, 2, 2, 2), (4, 2, 4, 8), (2, 4, 8, 8), (1, 1, 1, 8), (2, 2, 3, 4)])
@pytest.mark.parametrize("dataflow", ["os", "ls", "rs"])
def test_c_oracle_random_integer_cases(lib, dataflow, R, C, S, B):
    rng = np.random.default_rng(7 + R * 100 + C * 10 + S)
    u = R * C * S * B
    a, b, c = 2 * u, u, 3 * u
    if dataflow == "os":
        X = rng.integers(-4, 5, (2 * R * 4, b)); W = rng.integers(-4, 5, (b, c))
    elif dataflow == "ls":
        X = rng.integers(-4, 5, (2 * R * 4, C * 8)); W = rng.integers(-4, 5, (c, C * 8))
    else:
        X = rng.integers(-4, 5, (R * 8, a)); W = rng.integers(-4, 5, (R * 8, C * 8))
    X = X.astype(np.float32); W = W.astype(np.float32)
    orc.check_divisibility(dataflow, X.shape, W.shape, R, C, S, B)
    rc, Y = _run(lib, dataflow, X, W, R, C, S, B)
    assert rc == 0
    assert np.array_equal(Y, orc.dense(dataflow, X, W))
    if not (dataflow == "os" and S == 1):
        assert np.array_equal(Y, orc.literal_meshflow(dataflow, X.astype(np.float64), W.astype(np.float64), R, C, S, B))


def test_c_oracle_rejects_inadmissible_shapes(lib):
    X = np.zeros((8, 24), np.float32); W = np.zeros((24, 8), np.float32)
    rc, _ = _run(lib, "os", X, W, 2, 2, 4, 8)
    assert rc == -1


def test_c_bf16_round_matches_numpy(lib):
    rng = np.random.default_rng(2)
    x = np.concatenate([rng.standard_normal(5000).astype(np.float32) * 3,
                        np.float32([1.00390625, 1.01171875, 0.0, -0.0, np.inf, -np.inf, 1e-41])])
    out = np.empty_like(x)
    fp = ctypes.POINTER(ctypes.c_float)
    lib.ms_oracle_bf16_round(x.ctypes.data_as(fp), out.ctypes.data_as(fp), len(x))
    assert np.array_equal(out.view(np.uint32), orc.bf16_round(x).view(np.uint32))
