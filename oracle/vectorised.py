"""Float64 restatements of the loop patterns for full sizes.  TEST INFRASTRUCTURE.

Every function returns ``(value, budget)``: the result in float64 (computed
from the inputs converted to float64, so that the only rounding left is
float64's) and ``budget = sum(|terms|)`` per output, the quantity the parity
bar is stated in: ``|out - value| <= 1e-5 * budget``.  ``vec_add`` is
elementwise and bit-exact, so it returns the float32 result only.
"""
import numpy as np
import scipy.sparse as sp

TOL = 1e-5


def vec_add(a, b):
    """c[i] = a[i] + b[i] (examples/01-vec_add.py:11-12): one IEEE-754
    addition per element in the arrays' dtype."""
    return np.add(a, b)


def vector_sum(a):
    """s += a[i] (examples/02-vec_sum.py:9-10)."""
    a64 = np.asarray(a, dtype=np.float64)
    return float(a64.sum()), float(np.abs(a64).sum())


def masked_sum(a, mask):
    """s += a[i] if mask[i] else 0.0 (examples/04-masked_sum.py:21-22)."""
    a64 = np.where(mask, np.asarray(a, dtype=np.float64), 0.0)
    return float(a64.sum()), float(np.abs(a64).sum())


def gemv(A, x, alpha=1.0):
    """y[i] = sum_j alpha * A[i, j] * x[j] (examples/05-gemv.py:11-16)."""
    A64 = np.asarray(A, dtype=np.float64)
    x64 = np.asarray(x, dtype=np.float64)
    return alpha * (A64 @ x64), abs(alpha) * (np.abs(A64) @ np.abs(x64))


def _csr(data, indptr, indices, shape, absolute=False):
    d = np.asarray(data, dtype=np.float64)
    if absolute:
        d = np.abs(d)
    return sp.csr_matrix((d, np.asarray(indices), np.asarray(indptr)), shape=shape)


def spmv_csr(data, indptr, indices, x, shape):
    """y[i] = sum_{j in row i} data[j] * x[indices[j]] (examples/03-spmv.py:9-15)."""
    x64 = np.asarray(x, dtype=np.float64)
    y = _csr(data, indptr, indices, shape) @ x64
    budget = _csr(data, indptr, indices, shape, absolute=True) @ np.abs(x64)
    return np.asarray(y), np.asarray(budget)


def spmm_csr(data, indptr, indices, B, shape):
    """C[i, :] = sum_k data[k] * B[indices[k], :] (examples/06-spmm.py:6-10)."""
    B64 = np.asarray(B, dtype=np.float64)
    C = _csr(data, indptr, indices, shape) @ B64
    budget = _csr(data, indptr, indices, shape, absolute=True) @ np.abs(B64)
    return np.asarray(C), np.asarray(budget)


def gather_dot(v, idx, x):
    """s += v[i] * x[idx[i]]: the inner loop of examples/03-spmv.py:12-13 over one flat
    stream of (value, index) pairs (used to calibrate the gather rate)."""
    terms = np.asarray(v, dtype=np.float64) * np.asarray(x, dtype=np.float64)[np.asarray(idx)]
    return float(terms.sum()), float(np.abs(terms).sum())


def within_budget(out, value, budget, tol=TOL):
    """max over outputs of |out - value| / (tol * budget) <= 1 (outputs whose
    budget is zero must be exact)."""
    out = np.asarray(out, dtype=np.float64)
    value = np.asarray(value, dtype=np.float64)
    budget = np.asarray(budget, dtype=np.float64)
    err = np.abs(out - value)
    return bool(np.all(err <= tol * budget + 0.0)), float(np.max(err / np.maximum(tol * budget, np.finfo(np.float64).tiny)))
