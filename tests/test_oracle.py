"""Pins the CPU oracle (oracle/) before anything is compared with it.

The reference holds no golden vectors for this path, so every oracle function
is pinned by independent facts: the reference's literal loop bodies run by the
interpreter, closed forms, exact special cases, library routines that do not
share code with the oracle (math.fsum, dense matmul), and invariants chosen so
that a dropped term, a wrong index or a transposed operand fails."""
import math

import numpy as np
import pytest

from oracle import loops as lo
from oracle import vectorised as vo
from oracle import workloads as wl


def test_vec_add_is_ieee_addition():
    a, b = wl.vec_add(1001)
    c = vo.vec_add(a, b)
    assert c.dtype == np.float32
    assert np.array_equal(c, lo.vec_add(a, b))                      # literal loop
    assert np.array_equal(c, vo.vec_add(b, a))                      # commutative
    assert np.array_equal(vo.vec_add(a, np.zeros_like(a)), a)       # a + 0 = a
    # against exact rational arithmetic rounded once
    exact = (a.astype(np.float64) + b.astype(np.float64)).astype(np.float32)
    assert np.array_equal(c, exact)


def test_vector_sum_closed_form_and_fsum():
    n = 4096
    a = np.arange(1, n + 1, dtype=np.float32)
    val, budget = vo.vector_sum(a)
    assert val == n * (n + 1) / 2 == budget
    A, _ = wl.reduce_inputs(20_011)
    val, budget = vo.vector_sum(A)
    assert val == pytest.approx(math.fsum(float(x) for x in A), rel=1e-15)
    assert budget == pytest.approx(math.fsum(abs(float(x)) for x in A), rel=1e-15)
    assert val == pytest.approx(lo.vector_sum(A), rel=1e-13)       # sequential float64 loop
    assert vo.vector_sum(-A)[0] == -val


def test_masked_sum_masks_and_complement():
    A, M = wl.reduce_inputs(10_007)
    val, budget = vo.masked_sum(A, M)
    assert val == pytest.approx(lo.masked_sum_ternary(A, M), rel=1e-13)
    assert val == pytest.approx(lo.masked_sum_if(A, M), rel=1e-13)
    assert vo.masked_sum(A, np.zeros_like(M)) == (0.0, 0.0)
    assert vo.masked_sum(A, np.ones_like(M))[0] == vo.vector_sum(A)[0]
    comp = vo.masked_sum(A, ~M)[0]
    assert val + comp == pytest.approx(vo.vector_sum(A)[0], rel=1e-14)
    assert 0.4 < M.mean() < 0.6                                     # Bernoulli(0.5), independent of A
    assert abs(np.corrcoef(A, M)[0, 1]) < 0.05


def test_gather_dot_is_a_one_row_spmv():
    rng = np.random.default_rng(31)
    v = rng.standard_normal(501).astype(np.float32)
    x = rng.standard_normal(64).astype(np.float32)
    idx = rng.integers(0, 64, 501).astype(np.int32)
    val, budget = vo.gather_dot(v, idx, x)
    assert val == pytest.approx(math.fsum(float(v[i]) * float(x[idx[i]]) for i in range(501)), rel=1e-13)
    assert budget == pytest.approx(math.fsum(abs(float(v[i]) * float(x[idx[i]])) for i in range(501)), rel=1e-13)
    # identity permutation: a plain dot product; a constant index picks one element of x
    assert vo.gather_dot(x, np.arange(64), x)[0] == pytest.approx(float(x.astype(np.float64) @ x.astype(np.float64)), rel=1e-14)
    assert vo.gather_dot(v, np.full(501, 7), x)[0] == pytest.approx(float(x[7]) * vo.vector_sum(v)[0], rel=1e-12)


def test_gemv_unit_vectors_identity_linearity_loop():
    A, x = wl.gemv(37, 53)
    val, budget = vo.gemv(A, x)
    ref = lo.gemv(1.0, A.astype(np.float64), x.astype(np.float64))
    assert np.allclose(val, ref, rtol=1e-13, atol=0)
    for col in (0, 17, 52):
        e = np.zeros(53, dtype=np.float32)
        e[col] = 1.0
        assert np.array_equal(vo.gemv(A, e)[0], A[:, col].astype(np.float64))   # selects a column, not a row
    eye = np.eye(53, dtype=np.float32)
    assert np.array_equal(vo.gemv(eye, x)[0], x.astype(np.float64))
    assert np.allclose(vo.gemv(A, x, alpha=-2.5)[0], -2.5 * val, rtol=1e-15)
    assert np.allclose(vo.gemv(A, 2 * x)[0], 2 * val, rtol=1e-15)
    assert np.all(budget >= np.abs(val) - 1e-12)
    brute = np.array([math.fsum(abs(float(A[i, j])) * abs(float(x[j])) for j in range(53)) for i in range(37)])
    assert np.allclose(budget, brute, rtol=1e-13)


def _dense(data, indptr, indices, shape):
    D = np.zeros(shape, dtype=np.float64)
    for i in range(shape[0]):
        for p in range(indptr[i], indptr[i + 1]):
            D[i, indices[p]] += float(data[p])
    return D


def test_spmv_against_dense_loop_and_special_cases():
    data, indptr, indices, x = wl.spmv_powerlaw(300, 300, clip=64)
    val, budget = vo.spmv_csr(data, indptr, indices, x, (300, 300))
    D = _dense(data, indptr, indices, (300, 300))
    assert np.allclose(val, D @ x.astype(np.float64), rtol=1e-12, atol=1e-12)
    assert np.allclose(budget, np.abs(D) @ np.abs(x.astype(np.float64)), rtol=1e-12, atol=1e-12)
    ref = lo.spmv_csr(data.astype(np.float64), indptr, indices, x.astype(np.float64), 300, 300)
    assert np.allclose(val, ref, rtol=1e-12, atol=1e-12)
    # empty rows give 0; identity returns x
    ptr = np.array([0, 0, 2, 2, 3], dtype=np.int32)
    idx = np.array([1, 3, 0], dtype=np.int32)
    dat = np.array([2.0, -1.0, 0.5], dtype=np.float32)
    xx = np.array([4.0, 3.0, 2.0, 1.0], dtype=np.float32)
    assert np.array_equal(vo.spmv_csr(dat, ptr, idx, xx, (4, 4))[0], [0.0, 5.0, 0.0, 2.0])
    n = 50
    assert np.array_equal(
        vo.spmv_csr(np.ones(n, np.float32), np.arange(n + 1, dtype=np.int32), np.arange(n, dtype=np.int32), x[:n], (n, n))[0],
        x[:n].astype(np.float64))


def test_spmm_columns_are_spmvs_and_dense():
    data, indptr, indices, B = wl.spmm(120, 150, 16, mean_row=8)
    val, budget = vo.spmm_csr(data, indptr, indices, B, (120, 150))
    D = _dense(data, indptr, indices, (120, 150))
    assert np.allclose(val, D @ B.astype(np.float64), rtol=1e-12, atol=1e-12)
    for col in (0, 7, 15):
        v1, b1 = vo.spmv_csr(data, indptr, indices, np.ascontiguousarray(B[:, col]), (120, 150))
        assert np.allclose(val[:, col], v1, rtol=1e-13, atol=1e-13)
        assert np.allclose(budget[:, col], b1, rtol=1e-13, atol=1e-13)
    Y = np.full((120, 16), np.nan)
    lo.spmm_csr(data.astype(np.float64), indptr, indices, B.astype(np.float64), Y, 120)
    assert np.allclose(val, Y, rtol=1e-12, atol=1e-12)


def test_generators_meet_the_workload_definitions():
    data, indptr, indices, x = wl.spmv_uniform(500, 4000, 16)
    lens = np.diff(indptr)
    assert np.all(lens == 16) and indptr.dtype == np.int32 and indices.dtype == np.int32
    for i in range(0, 500, 37):
        row = indices[indptr[i]:indptr[i + 1]]
        assert np.all(np.diff(row) > 0) and row.min() >= 0 and row.max() < 4000     # sorted, distinct, in range
    data, indptr, indices, x = wl.spmv_powerlaw(5000, 5000, clip=128)
    lens = np.diff(indptr)
    assert lens.min() >= 1 and lens.max() <= 128
    for i in range(0, 5000, 331):
        row = indices[indptr[i]:indptr[i + 1]]
        assert np.all(np.diff(row) > 0)
    a1, _ = wl.vec_add(100)
    a2, _ = wl.vec_add(100)
    assert np.array_equal(a1, a2) and a1.min() >= -1 and a1.max() < 1                # seeded, uniform[-1,1)


def test_within_budget_helper():
    ok, worst = vo.within_budget([1.0, 2.0], [1.0, 2.0], [1.0, 1.0])
    assert ok and worst == 0.0
    ok, worst = vo.within_budget([1.0 + 2e-5], [1.0], [1.0])
    assert not ok and worst == pytest.approx(2.0, rel=1e-6)
    assert vo.within_budget([0.0], [0.0], [0.0])[0]
    assert not vo.within_budget([1e-300], [0.0], [0.0])[0]
