"""Committed fixtures (tests/golden/*.npz, written by tests/golden/make_fixtures.py).

CPU part: the oracle still reproduces the committed vectors (so a change of
the oracle is visible as a diff of data).  GPU part: the HIP path meets the
parity bar against the committed vectors, without calling the oracle."""
import os

import numpy as np
import pytest

from oracle import vectorised as vo

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
TOL = 1e-5


def load(name):
    return np.load(os.path.join(GOLDEN, name + ".npz"), allow_pickle=False)


def test_oracle_reproduces_fixtures():
    g = load("vec_add")
    assert np.array_equal(vo.vec_add(g["a"], g["b"]), g["c"])
    g = load("reductions")
    assert vo.vector_sum(g["A"]) == (float(g["vector_sum"]), float(g["vector_sum_budget"]))
    assert vo.masked_sum(g["A"], g["M"]) == (float(g["masked_sum"]), float(g["masked_sum_budget"]))
    g = load("gemv")
    assert np.array_equal(vo.gemv(g["A"], g["x"])[0], g["y"])
    g = load("spmv")
    assert np.array_equal(vo.spmv_csr(g["data"], g["indptr"], g["indices"], g["x"], (257, 300))[0], g["y"])
    g = load("spmm")
    assert np.array_equal(vo.spmm_csr(g["data"], g["indptr"], g["indices"], g["B"], (129, 140))[0], g["C"])


@pytest.mark.gpu
def test_hip_path_against_fixtures(gpu):
    from appy_amd.backends.hip import selfcheck

    k = selfcheck.kernels()
    g = load("vec_add")
    assert np.array_equal(k.vec_add(g["a"], g["b"]), g["c"])
    g = load("reductions")
    assert abs(k.vector_sum(g["A"]) - float(g["vector_sum"])) <= TOL * float(g["vector_sum_budget"])
    assert abs(k.masked_sum(g["A"], g["M"]) - float(g["masked_sum"])) <= TOL * float(g["masked_sum_budget"])
    g = load("gemv")
    assert np.all(np.abs(k.gemv(g["A"], g["x"]) - g["y"]) <= TOL * g["budget"])
    g = load("spmv")
    y = k.spmv(g["data"], g["indptr"], g["indices"], g["x"], 257, 300)
    assert np.all(np.abs(y - g["y"]) <= TOL * g["budget"])
    g = load("spmm")
    Y = np.empty((129, 128), dtype=np.float32)
    k.spmm(g["data"], g["indptr"], g["indices"], g["B"], Y, 129)
    assert np.all(np.abs(Y - g["C"]) <= TOL * g["budget"])
