"""Seeded random shapes around the tile, vector and team boundaries of the
generated kernels (BLOCK x U x V tiles, V-wide vectors, W-lane teams, row
accumulators), each against the oracle.  Deterministic: the seeds are fixed."""
import numpy as np
import pytest

from appy_amd.backends.hip import selfcheck
from oracle import vectorised as vo
from oracle import workloads as wl

pytestmark = pytest.mark.gpu
TOL = 1e-5


@pytest.fixture(scope="module")
def k(gpu):
    return selfcheck.kernels()


def sizes(seed, count, hi):
    rng = np.random.default_rng(seed)
    special = [1, 2, 3, 4, 5, 255, 256, 257, 1023, 1024, 1025, 2047, 2048, 2049, 4095, 4096, 4097, 8191, 8193]
    return sorted(set(special + [int(v) for v in rng.integers(1, hi, count)]))


def test_flat_kernels_over_many_lengths(k):
    for n in sizes(1, 40, 70_000):
        a, b = wl.vec_add(n, seed=n)
        assert np.array_equal(k.vec_add(a, b), a + b), n
        A, M = wl.reduce_inputs(n, seed=n)
        ref, budget = vo.vector_sum(A)
        assert abs(k.vector_sum(A) - ref) <= TOL * budget, n
        ref, budget = vo.masked_sum(A, M)
        assert abs(k.masked_sum(A, M) - ref) <= TOL * budget, n


def test_gemv_over_many_shapes(k):
    rng = np.random.default_rng(2)
    shapes = [(1, 1), (1, 5000), (5000, 1), (2, 3), (7, 4), (8, 127), (9, 128), (33, 129), (65, 4097)]
    shapes += [(int(r), int(c)) for r, c in zip(rng.integers(1, 600, 25), rng.integers(1, 3000, 25))]
    for r, c in shapes:
        A, x = wl.gemv(r, c, seed=r * 7919 + c)
        ref, budget = vo.gemv(A, x)
        ok, worst = vo.within_budget(k.gemv(A, x), ref, budget, TOL)
        assert ok, (r, c, worst)


def test_csr_kernels_over_many_structures(k):
    rng = np.random.default_rng(3)
    for case in range(25):
        m = int(rng.integers(1, 3000))
        n = int(rng.integers(1, 3000))
        kind = case % 4
        if kind == 0:
            lengths = rng.integers(0, min(n, 40) + 1, m)                      # short rows, some empty
        elif kind == 1:
            lengths = np.minimum(rng.zipf(1.5, m), n)                         # power law up to full rows
        elif kind == 2:
            lengths = np.where(rng.random(m) < 0.7, 0, min(n, 300))           # mostly empty, a few long rows
        else:
            lengths = np.full(m, min(n, int(rng.integers(1, 70))))            # uniform
        data, indptr, indices = wl.csr_matrix(lengths, n, rng)
        x = rng.standard_normal(n, dtype=np.float32)
        ref, budget = vo.spmv_csr(data, indptr, indices, x, (m, n))
        y = k.spmv(data, indptr, indices, x, m, n)
        ok, worst = vo.within_budget(y, ref, budget, TOL)
        assert ok, ("spmv", case, m, n, worst)
        ncol = [128, 1, 4, 60, 200][case % 5]
        B = rng.standard_normal((n, ncol), dtype=np.float32)
        ref, budget = vo.spmm_csr(data, indptr, indices, B, (m, n))
        Y = np.full((m, ncol), np.nan, dtype=np.float32)
        k.spmm(data, indptr, indices, B, Y, m)
        ok, worst = vo.within_budget(Y, ref, budget, TOL)
        assert ok, ("spmm", case, m, n, ncol, worst)
