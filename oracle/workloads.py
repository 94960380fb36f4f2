"""Seeded synthetic inputs for the five workload configurations.  TEST
INFRASTRUCTURE (also used by bench.py to build its inputs).

All generators use ``numpy.random.default_rng(seed)`` so that the GPU path and
the oracle see identical arrays.  Sizes are parameters; the full sizes are the
defaults of bench.py.
"""
import numpy as np

SEEDS = {"vec_add": 1, "reduce": 2, "gemv": 3, "spmv": 4, "spmm": 5}


def vec_add(n, seed=SEEDS["vec_add"]):
    rng = np.random.default_rng(seed)
    a = rng.uniform(-1.0, 1.0, n).astype(np.float32)
    b = rng.uniform(-1.0, 1.0, n).astype(np.float32)
    return a, b


def reduce_inputs(n, seed=SEEDS["reduce"]):
    """A uniform[0,1) float32; M Bernoulli(0.5) bool from an independent stream."""
    rng = np.random.default_rng(seed)
    A = rng.random(n, dtype=np.float32)
    rng_m = np.random.default_rng(seed + 1000)
    M = rng_m.random(n, dtype=np.float32) < 0.5
    return A, M


def gemv(rows, cols, seed=SEEDS["gemv"]):
    rng = np.random.default_rng(seed)
    A = rng.standard_normal((rows, cols), dtype=np.float32)
    x = rng.standard_normal(cols, dtype=np.float32)
    return A, x


def _sorted_unique_columns(rng, lengths, ncols):
    """Per row: ``len`` distinct column indices, uniform over [0, ncols),
    sorted.  Drawn as uniform samples with duplicates inside a row redrawn
    (row lengths are far below ncols, so few rounds are needed)."""
    lengths = np.asarray(lengths, dtype=np.int64)
    indptr = np.zeros(len(lengths) + 1, dtype=np.int64)
    np.cumsum(lengths, out=indptr[1:])
    nnz = int(indptr[-1])
    if len(lengths) and int(lengths.max()) * 4 > ncols:
        # dense rows: rejection would not terminate, draw each row without replacement
        cols = np.concatenate([np.sort(rng.permutation(ncols)[: int(n)]) for n in lengths] or [np.empty(0, np.int64)])
        return indptr, cols.astype(np.int64)
    if len(lengths) and np.all(lengths == lengths[0]) and 0 < lengths[0] and 4 * int(lengths[0]) ** 2 < ncols:
        # equal rows: sort each row on its own, redraw the rows that hold a duplicate
        L = int(lengths[0])
        cols = np.sort(rng.integers(0, ncols, size=(len(lengths), L), dtype=np.int64), axis=1)
        for _ in range(64):
            bad = np.flatnonzero((cols[:, 1:] == cols[:, :-1]).any(axis=1)) if L > 1 else np.empty(0, dtype=np.int64)
            if bad.size == 0:
                return indptr, cols.reshape(-1)
            cols[bad] = np.sort(rng.integers(0, ncols, size=(bad.size, L), dtype=np.int64), axis=1)
        raise RuntimeError("could not draw distinct columns")
    row_of = np.repeat(np.arange(len(lengths), dtype=np.int64), lengths)
    cols = rng.integers(0, ncols, size=nnz, dtype=np.int64)
    for _ in range(64):
        key = row_of * ncols + cols
        order = np.argsort(key, kind="stable")
        sk = key[order]
        dup = np.zeros(nnz, dtype=bool)
        dup[order[1:]] = sk[1:] == sk[:-1]
        ndup = int(dup.sum())
        if ndup == 0:
            cols = (sk % ncols)
            break
        cols[dup] = rng.integers(0, ncols, size=ndup, dtype=np.int64)
    else:
        raise RuntimeError("could not draw distinct columns")
    return indptr, cols


def csr_matrix(lengths, ncols, rng):
    indptr, cols = _sorted_unique_columns(rng, lengths, ncols)
    nnz = int(indptr[-1])
    if nnz >= 2**31:
        raise ValueError("nnz does not fit int32 row pointers")
    data = rng.standard_normal(nnz, dtype=np.float32)
    return data, indptr.astype(np.int32), cols.astype(np.int32)


def spmv_uniform(m, n, per_row=16, seed=SEEDS["spmv"]):
    rng = np.random.default_rng(seed)
    lengths = np.full(m, per_row, dtype=np.int64)
    data, indptr, indices = csr_matrix(lengths, n, rng)
    x = rng.standard_normal(n, dtype=np.float32)
    return data, indptr, indices, x


def spmv_powerlaw(m, n, exponent=1.5, clip=4096, seed=SEEDS["spmv"] + 100):
    """Row lengths Zipf(exponent) clipped to [1, clip]."""
    rng = np.random.default_rng(seed)
    lengths = np.clip(rng.zipf(exponent, m), 1, min(clip, n)).astype(np.int64)
    data, indptr, indices = csr_matrix(lengths, n, rng)
    x = rng.standard_normal(n, dtype=np.float32)
    return data, indptr, indices, x


def spmm(m, n, ncols_b=128, mean_row=32, seed=SEEDS["spmm"]):
    rng = np.random.default_rng(seed)
    lengths = np.minimum(rng.poisson(mean_row, m), n).astype(np.int64)
    data, indptr, indices = csr_matrix(lengths, n, rng)
    B = rng.standard_normal((n, ncols_b), dtype=np.float32)
    return data, indptr, indices, B
