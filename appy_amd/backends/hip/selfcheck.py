"""The five workload loops written with the public annotations, used by the
build check, the smoke run and the benchmark.

These are the loop shapes of the reference's examples (reference tree:
examples/01-vec_add.py:7-13, 02-vec_sum.py:5-11, 04-masked_sum.py:17-23,
05-gemv.py:7-17 without ``alpha``, 03-spmv.py:5-16, 06-spmm.py:4-11), decorated
with :func:`appy_amd.jit`; they run through the same path as user code.
"""
from __future__ import annotations

import types

import numpy as np

import appy_amd as appy


def _empty_like(a):
    if isinstance(a, np.ndarray):
        return np.empty_like(a)
    import torch

    return torch.empty_like(a)


def _empty(n, like):
    if isinstance(like, np.ndarray):
        return np.empty(n, dtype=like.dtype)
    import torch

    return torch.empty(n, dtype=like.dtype, device=like.device)


def vec_add(a, b):
    c = _empty_like(a)
    #pragma parallel for simd
    for i in range(a.shape[0]):
        c[i] = a[i] + b[i]
    return c


def copy(a, c):
    #pragma parallel for simd
    for i in range(a.shape[0]):
        c[i] = a[i]


def vector_sum(A):
    s = 0.0
    #pragma parallel for simd shared(s)
    for i in range(A.shape[0]):
        s += A[i]
    return s


def masked_sum(A, M):
    s = 0.0
    #pragma parallel for simd shared(s)
    for i in range(A.shape[0]):
        s += A[i] if M[i] else 0.0
    return s


def gemv(A, x):
    y = _empty(A.shape[0], x)
    #pragma parallel for
    for i in range(A.shape[0]):
        yi = 0.0
        #pragma simd
        for j in range(A.shape[1]):
            yi += A[i, j] * x[j]
        y[i] = yi
    return y


def gemv_columns(A, y):
    x = _empty(A.shape[1], y)
    #pragma parallel for
    for j in range(A.shape[1]):
        s = 0.0
        #pragma simd
        for i in range(A.shape[0]):
            s += A[i, j] * y[i]
        x[j] = s
    return x


def spmv(A_data, A_indptr, A_indices, x, M, N):
    y = _empty(M, x)
    #pragma parallel for
    for i in range(M):
        start, end = A_indptr[i], A_indptr[i+1]
        s = 0.0
        #pragma simd
        for j in range(start, end):
            s += A_data[j] * x[A_indices[j]]
        y[i] = s
    return y


def gather_dot(v, idx, x):
    """Calibration loop: one coalesced stream of (value, index) pairs and one 4-byte
    gather per pair, i.e. the memory behaviour of CSR SpMV without its row structure."""
    s = 0.0
    #pragma parallel for simd shared(s)
    for i in range(v.shape[0]):
        s += v[i] * x[idx[i]]
    return s


def spmm(A_data, A_indptr, A_indices, B, y, M):
    #pragma parallel for
    for i in range(M):
        start, end = A_indptr[i], A_indptr[i+1]
        y[i, :] = 0
        for k in range(start, end):
            y[i, :] += A_data[k] * B[A_indices[k], :]


_RAW = (vec_add, copy, vector_sum, masked_sum, gemv, gemv_columns, spmv, spmm, gather_dot)
_cache = {}


def kernels(**options):
    """Namespace with the six loops compiled by :func:`appy_amd.jit` under
    ``options`` (cached per option set)."""
    key = repr(sorted(options.items()))
    ns = _cache.get(key)
    if ns is None:
        ns = types.SimpleNamespace(**{f.__name__: appy.jit(f, **options) if options else appy.jit(f) for f in _RAW})
        _cache[key] = ns
    return ns


def compile_all_patterns() -> int:
    """Generate and hiprtc-compile the kernels of all six loops for small
    float32/int32 inputs (no GPU needed: the loops themselves are then run by
    the interpreter, ``dry_run``).  Returns the number of kernel variants."""
    from . import codegen as cg
    from .kernelgen import Spec

    k = kernels(dry_run=True)
    rng = np.random.default_rng(0)
    a = rng.random(64, dtype=np.float32)
    m = rng.random(64) < 0.5
    A = rng.random((8, 16), dtype=np.float32)
    x = rng.random(16, dtype=np.float32)
    indptr = np.arange(0, 17, 2, dtype=np.int32)
    indices = (np.arange(16, dtype=np.int32) * 3) % 8
    data = rng.random(16, dtype=np.float32)
    B = rng.random((8, 128), dtype=np.float32)
    Y = np.empty((8, 128), dtype=np.float32)
    before = set(cg.code_cache)
    k.vec_add(a, a)
    k.copy(a, np.empty_like(a))
    k.vector_sum(a)
    k.masked_sum(a, m)
    k.gemv(A, x)
    k.gemv_columns(A, x[:8].copy())
    k.spmv(data, indptr, indices, x[:8].copy(), 8, 8)
    k.spmm(data, indptr, indices, B, Y, 8)
    k.gather_dot(data, indices, x[:8].copy())
    count = 0
    names = {f.__name__ for f in _RAW}
    for key in [k for k in cg.code_cache if k not in before or k[-1] in names]:
        loop, _src = cg.code_cache[key]
        count += len(loop.kernels)
        if loop.analysis.strip is not None:
            loop.kernel_for(Spec("strip", block=1024, vec=1, unroll=8, stream_loads=True)).code
            count += 1
        if loop.analysis.kind == "team":
            for w in (1, 4, 16, 64):
                loop.kernel_for(Spec("team", block=256, vec=loop.default_spec.vec, width=w)).code
                count += 1
        v = loop.default_spec.vec
        more = []
        if loop.analysis.ragged is not None and v > 1:
            # rows sorted by the length of their simd loop; long rows in planned parts
            more += [Spec("team", block=1024, vec=1, width=1, aux="bins"), Spec("team", block=256, vec=v, width=64, rows="mixed")]
            if loop.analysis.ragged[1] is not None:
                more += [Spec("team", block=256, vec=1, width=8, rows="list", parts=8, aux="plan"),
                         Spec("team", block=256, vec=v, width=16, phase=1, rows="list", parts=8),
                         Spec("team", block=256, vec=v, width=1, phase=2, rows="list", parts=8)]
            if loop.analysis.grouping is not None:
                # elements grouped by the stripe of the gathered operand
                more += [Spec("team", block=256, vec=1, width=64, parts=8, aux="group", block_rows=256),
                         Spec("team", block=256, vec=1, width=64, parts=8, aux="group", block_rows=512, skip_long=True),
                         Spec("team", block=256, vec=1, width=64, parts=8, aux="cells", block_rows=1024, guard=1),
                         Spec("team", block=256, vec=v, width=1, phase=2, guard=1, skip_long=True),
                         Spec("team", block=256, vec=v, width=16, phase=1, rows="list", parts=8, guard=1),
                         Spec("team", block=256, vec=1, width=64, parts=16, aux="cells", block_rows=256, guard=1),
                         Spec("team", block=256, vec=v, width=1, phase=2, guard=1),
                         Spec("team", block=256, vec=v, width=4, guard=2),
                         # the order of the elements worked out once and kept: the kernel that writes the pairs to
                         # sort, the kernel that runs the plan
                         Spec("team", block=256, vec=1, width=64, aux="rkeys", block_rows=256),
                         Spec("team", block=1024, vec=1, width=1024, unroll=6, parts=8, aux="xcells"),
                         Spec("team", block=1024, vec=1, width=1024, unroll=4, parts=8, aux="xcells")]
        for spec in more:
            loop.kernel_for(spec).code
            count += 1
    return count
