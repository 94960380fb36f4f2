"""The reference's loop bodies, run by the interpreter.  TEST INFRASTRUCTURE.

Each function is the body of the corresponding example of the reference with
the decorator removed and the pragmas left as comments, i.e. the reference's
CPU path.  Arrays are NumPy arrays; sizes must be small (CPython speed).
"""
import numpy as np


def vec_add(a, b):
    """examples/01-vec_add.py:7-13"""
    c = np.empty_like(a)
    #pragma parallel for simd
    for i in range(a.shape[0]):
        c[i] = a[i] + b[i]
    return c


def vector_sum(a):
    """examples/02-vec_sum.py:5-11, after the shared() rewrite
    (appy/frontend/process_shared.py:27-53): the accumulator is a float64
    one-element array."""
    b = 0.0
    b = np.array([b])
    #pragma parallel for simd shared(b)
    for i in range(a.shape[0]):
        b[0] += a[i]
    b = b.item()
    return b


def masked_sum_if(a, mask):
    """examples/04-masked_sum.py:7-14"""
    b = np.array([0.0])
    #pragma parallel for shared(b)
    for i in range(a.shape[0]):
        if mask[i]:
            b[0] += a[i]
    return b.item()


def masked_sum_ternary(a, mask):
    """examples/04-masked_sum.py:17-23"""
    b = np.array([0.0])
    #pragma parallel for simd shared(b)
    for i in range(a.shape[0]):
        b[0] += a[i] if mask[i] else 0.0
    return b.item()


def gemv(alpha, A, x):
    """examples/05-gemv.py:7-17"""
    y = np.empty(A.shape[0], dtype=x.dtype)
    #pragma parallel for
    for i in range(A.shape[0]):
        yi = 0.0
        #pragma simd
        for j in range(A.shape[1]):
            yi += alpha * A[i, j] * x[j]
        y[i] = yi
    return y


def spmv_csr(A_data, A_indptr, A_indices, x, M, N):
    """examples/03-spmv.py:5-16"""
    y = np.empty(M, dtype=x.dtype)
    #pragma parallel for
    for i in range(M):
        start, end = A_indptr[i], A_indptr[i + 1]
        s = 0.0
        #pragma simd
        for j in range(start, end):
            s += A_data[j] * x[A_indices[j]]
        y[i] = s
    return y


def spmm_csr(A_data, A_indptr, A_indices, B, y, M):
    """examples/06-spmm.py:4-11"""
    #pragma parallel for
    for i in range(M):
        start, end = A_indptr[i], A_indptr[i + 1]
        y[i, :] = 0
        for k in range(start, end):
            y[i, :] += A_data[k] * B[A_indices[k], :]
    return y
