"""Wider loop shapes on the GPU, each against NumPy on seeded inputs: the kernel
families of the reference's NPBench / DPBench integration tests
(tests/integration/triton/npbench/*.py, dpbench/test_black_scholes.py) -
triangular ``simd`` loops, stencils with neighbour offsets, in-place row
updates, strided (column) accesses, several reductions in one ``simd`` loop,
slices of the first dimension, ``@`` of slices, maths functions, loops nested
in host-side Python loops.  Tolerances are those of the reference's tests."""
import math
from math import erf

import numpy as np
import pytest

import appy

pytestmark = pytest.mark.gpu


@appy.jit
def syrk_loops(alpha, beta, C, A):
    #pragma parallel for
    for i in range(A.shape[0]):
        #pragma simd
        for j in range(i + 1):
            C[i, j] *= beta
        for k in range(A.shape[1]):
            #pragma simd
            for j in range(i + 1):
                C[i, j] += alpha * A[i, k] * A[j, k]
    return C


@appy.jit
def syrk_slices(alpha, beta, C, A):
    #pragma parallel for
    for i in range(A.shape[0]):
        C[i, :i + 1] *= beta
        for k in range(A.shape[1]):
            C[i, :i + 1] += alpha * A[i, k] * A[:i + 1, k]
    return C


def test_syrk(gpu):
    rng = np.random.default_rng(0)
    n, m = 70, 50
    A = rng.standard_normal((n, m))
    C = rng.standard_normal((n, n))
    alpha, beta = 1.5, 1.2
    ref = C.copy()
    for i in range(n):
        ref[i, :i + 1] = beta * ref[i, :i + 1] + alpha * (A[:i + 1] @ A[i])
    assert np.allclose(syrk_loops(alpha, beta, C.copy(), A), ref)
    assert np.allclose(syrk_slices(alpha, beta, C.copy(), A), ref)


@appy.jit
def jacobi_1d(TSTEPS, A, B):
    for t in range(1, TSTEPS):
        #pragma parallel for simd
        for i in range(1, A.shape[0] - 1):
            B[i] = 0.33333 * (A[i - 1] + A[i] + A[i + 1])

        #pragma parallel for simd
        for i in range(1, B.shape[0] - 1):
            A[i] = 0.33333 * (B[i - 1] + B[i] + B[i + 1])
    return A, B


def test_jacobi_1d(gpu):
    n = 10_007
    A = np.fromfunction(lambda i: (i + 2) / n, (n,), dtype=np.float64)
    B = np.fromfunction(lambda i: (i + 3) / n, (n,), dtype=np.float64)
    A1, B1 = A.copy(), B.copy()
    for _ in range(1, 10):
        B1[1:-1] = 0.33333 * (A1[:-2] + A1[1:-1] + A1[2:])
        A1[1:-1] = 0.33333 * (B1[:-2] + B1[1:-1] + B1[2:])
    A2, B2 = jacobi_1d(10, A.copy(), B.copy())
    assert np.array_equal(A2, A1) and np.array_equal(B2, B1)      # same operations in the same order


@appy.jit
def jacobi_2d(TSTEPS, A, B):
    for t in range(1, TSTEPS):
        #pragma parallel for
        for i in range(1, A.shape[0] - 1):
            #pragma simd
            for j in range(1, A.shape[1] - 1):
                B[i, j] = 0.2 * (A[i, j] + A[i, j - 1] + A[i, j + 1] + A[i - 1, j] + A[i + 1, j])

        #pragma parallel for
        for i in range(1, B.shape[0] - 1):
            #pragma simd
            for j in range(1, B.shape[1] - 1):
                A[i, j] = 0.2 * (B[i, j] + B[i, j - 1] + B[i, j + 1] + B[i - 1, j] + B[i + 1, j])
    return A, B


def test_jacobi_2d(gpu):
    n = 131
    rng = np.random.default_rng(1)
    A, B = rng.random((n, n)), rng.random((n, n))
    A1, B1 = A.copy(), B.copy()
    for _ in range(1, 6):
        B1[1:-1, 1:-1] = 0.2 * (A1[1:-1, 1:-1] + A1[1:-1, :-2] + A1[1:-1, 2:] + A1[:-2, 1:-1] + A1[2:, 1:-1])
        A1[1:-1, 1:-1] = 0.2 * (B1[1:-1, 1:-1] + B1[1:-1, :-2] + B1[1:-1, 2:] + B1[:-2, 1:-1] + B1[2:, 1:-1])
    A2, B2 = jacobi_2d(6, A.copy(), B.copy())
    assert np.allclose(A2, A1) and np.allclose(B2, B1)


@appy.jit
def floyd_warshall(path):
    for k in range(path.shape[0]):
        #pragma parallel for
        for i in range(path.shape[0]):
            #pragma simd
            for j in range(path.shape[1]):
                path[i, j] = min(path[i, j], path[i, k] + path[k, j])
    return path


def test_floyd_warshall(gpu):
    n = 90
    path = np.fromfunction(lambda i, j: i * j % 7 + 1, (n, n), dtype=np.int32)
    for i in range(n):
        for j in range(n):
            if (i + j) % 13 == 0 or (i + j) % 7 == 0 or (i + j) % 11 == 0:
                path[i, j] = 999
    ref = path.copy()
    for k in range(n):
        ref[:] = np.minimum(ref, np.add.outer(ref[:, k], ref[k, :]))
    out = floyd_warshall(path.copy())
    assert out.dtype == np.int32 and np.array_equal(out, ref)


@appy.jit
def go_fast(a):
    trace = 0.0
    #pragma parallel for simd shared(trace)
    for i in range(a.shape[0]):
        trace += np.tanh(a[i, i])
    return a + trace


def test_go_fast_diagonal_and_tanh(gpu):
    a = np.random.default_rng(2).random((300, 300))
    assert np.allclose(go_fast(a), a + np.tanh(np.diagonal(a)).sum(), atol=1e-6)


@appy.jit
def azimint(data, radius, npt):
    rmax = radius.max()
    res = np.zeros(npt, dtype=np.float64)
    #pragma parallel for
    for i in range(npt):
        r1 = rmax * i / npt
        r2 = rmax * (i + 1) / npt
        s, count = 0.0, 0
        #pragma simd
        for j in range(radius.shape[0]):
            mask_r12 = (r1 <= radius[j]) & (radius[j] < r2)
            s += data[j] if mask_r12 else 0.0
            count += 1 if mask_r12 else 0
        res[i] = s / count
    return res


def test_azimint_two_reductions_in_one_loop(gpu):
    rng = np.random.default_rng(3)
    n, npt = 4000, 50
    data, radius = rng.random(n), rng.random(n)
    rmax = radius.max()
    ref = np.zeros(npt)
    for i in range(npt):
        m = (rmax * i / npt <= radius) & (radius < rmax * (i + 1) / npt)
        ref[i] = data[m].mean()
    assert np.allclose(azimint(data, radius, npt), ref)


@appy.jit
def gemver(alpha, beta, A, u1, v1, u2, v2, w, x, y, z):
    M, N = A.shape
    #pragma parallel for
    for i in range(M):
        #pragma simd
        for j in range(N):
            A[i, j] += u1[i] * v1[j] + u2[i] * v2[j]

    #pragma parallel for
    for j in range(N):
        s = 0.0
        #pragma simd
        for i in range(M):
            s += beta * y[i] * A[i, j]
        x[j] += s + z[j]

    #pragma parallel for
    for i in range(M):
        s = 0.0
        #pragma simd
        for j in range(N):
            s += alpha * A[i, j] * x[j]
        w[i] += s
    return A, x, w


def test_gemver_three_loops_column_access(gpu):
    rng = np.random.default_rng(4)
    n = 120
    A = rng.random((n, n))
    u1, v1, u2, v2, w, x, y, z = (rng.random(n) for _ in range(8))
    alpha, beta = 1.5, 1.2
    A1 = A + np.outer(u1, v1) + np.outer(u2, v2)
    x1 = x + beta * y @ A1 + z
    w1 = w + alpha * A1 @ x1
    A2, x2, w2 = gemver(alpha, beta, A.copy(), u1, v1, u2, v2, w.copy(), x.copy(), y, z)
    assert np.allclose(A2, A1) and np.allclose(x2, x1) and np.allclose(w2, w1)


@appy.jit
def symm_loops(alpha, beta, C, A, B):
    temp2 = np.empty((C.shape[1], ), dtype=C.dtype)
    C *= beta
    for i in range(C.shape[0]):
        #pragma parallel for
        for j in range(C.shape[1]):
            s = 0.0
            #pragma simd
            for k in range(i):
                C[k, j] += alpha * B[i, j] * A[i, k]
                s += B[k, j] * A[i, k]
            temp2[j] = s
        C[i, :] += alpha * B[i, :] * A[i, i] + alpha * temp2
    return C


@appy.jit
def symm_slices(alpha, beta, C, A, B):
    temp2 = np.empty((C.shape[1], ), dtype=C.dtype)
    C *= beta
    for i in range(C.shape[0]):
        #pragma parallel for
        for j in range(C.shape[1]):
            C[:i, j] += alpha * B[i, j] * A[i, :i]
            temp2[j] = B[:i, j] @ A[i, :i]
        C[i, :] += alpha * B[i, :] * A[i, i] + alpha * temp2
    return C


def test_symm_store_and_reduction_in_one_simd_loop(gpu):
    rng = np.random.default_rng(5)
    m, n = 40, 45
    A, B, C = rng.random((m, m)), rng.random((m, n)), rng.random((m, n))
    alpha, beta = 1.5, 1.2
    ref = beta * C
    for i in range(m):
        for j in range(n):
            ref[:i, j] += alpha * B[i, j] * A[i, :i]
        ref[i, :] += alpha * B[i, :] * A[i, i] + alpha * (B[:i, :].T @ A[i, :i])
    assert np.allclose(symm_loops(alpha, beta, C.copy(), A, B), ref)
    assert np.allclose(symm_slices(alpha, beta, C.copy(), A, B), ref)


@appy.jit
def gramschmidt(A):
    Q = np.zeros_like(A)
    R = np.zeros((A.shape[1], A.shape[1]), dtype=A.dtype)
    for k in range(A.shape[1]):
        nrm = np.dot(A[:, k], A[:, k])
        R[k, k] = np.sqrt(nrm)
        Q[:, k] = A[:, k] / R[k, k]
        #pragma parallel for
        for j in range(k + 1, A.shape[1]):
            s = 0.0
            #pragma simd
            for i in range(A.shape[0]):
                s += Q[i, k] * A[i, j]

            #pragma simd
            for i in range(A.shape[0]):
                A[i, j] -= Q[i, k] * s
            R[k, j] = s
    return Q, R


def test_gramschmidt_two_simd_loops_per_iteration(gpu):
    rng = np.random.default_rng(6)
    A = rng.random((60, 40))
    Q, R = gramschmidt(A.copy())
    assert np.allclose(Q @ R, A) and np.allclose(Q.T @ Q, np.eye(40), atol=1e-8)
    assert np.allclose(R, np.triu(R))


@appy.jit
def fdtd_2d(TMAX, ex, ey, hz, _fict_):
    for t in range(TMAX):
        ey[0, :] = _fict_[t]
        #pragma parallel for
        for i in range(1, ey.shape[0]):
            #pragma simd
            for j in range(ey.shape[1]):
                ey[i, j] -= 0.5 * (hz[i, j] - hz[i - 1, j])
        #pragma parallel for
        for i in range(ex.shape[0]):
            #pragma simd
            for j in range(1, ex.shape[1]):
                ex[i, j] -= 0.5 * (hz[i, j] - hz[i, j - 1])
        #pragma parallel for
        for i in range(hz.shape[0] - 1):
            #pragma simd
            for j in range(hz.shape[1] - 1):
                hz[i, j] -= 0.7 * (ex[i, j + 1] - ex[i, j] + ey[i + 1, j] - ey[i, j])
    return ey, ex, hz


def test_fdtd_2d(gpu):
    rng = np.random.default_rng(7)
    nx, ny, tmax = 50, 60, 8
    ex, ey, hz = rng.random((nx, ny)), rng.random((nx, ny)), rng.random((nx, ny))
    fict = np.arange(tmax, dtype=np.float64)
    ex1, ey1, hz1 = ex.copy(), ey.copy(), hz.copy()
    for t in range(tmax):
        ey1[0, :] = fict[t]
        ey1[1:, :] -= 0.5 * (hz1[1:, :] - hz1[:-1, :])
        ex1[:, 1:] -= 0.5 * (hz1[:, 1:] - hz1[:, :-1])
        hz1[:-1, :-1] -= 0.7 * (ex1[:-1, 1:] - ex1[:-1, :-1] + ey1[1:, :-1] - ey1[:-1, :-1])
    ey2, ex2, hz2 = fdtd_2d(tmax, ex.copy(), ey.copy(), hz.copy(), fict)
    assert np.allclose(ey2, ey1) and np.allclose(ex2, ex1) and np.allclose(hz2, hz1)


@appy.jit
def black_scholes(nopt, price, strike, t, rate, volatility, call, put):
    mr = -rate
    sig_sig_two = volatility * volatility * 2
    #pragma parallel for simd
    for i in range(nopt):
        P = price[i]
        S = strike[i]
        T = t[i]
        a = np.log(P / S)
        b = T * mr
        z = T * sig_sig_two
        c = 0.25 * z
        y = 1.0 / np.sqrt(z)
        w1 = (a - b + c) * y
        w2 = (a - b - c) * y
        d1 = 0.5 + 0.5 * erf(w1)
        d2 = 0.5 + 0.5 * erf(w2)
        Se = np.exp(b) * S
        r = P * d1 - Se * d2
        call[i] = r
        put[i] = r - P + Se


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_black_scholes_maths_functions(gpu, dtype):
    rng = np.random.default_rng(8)
    n = 100_003
    price = rng.uniform(10, 50, n).astype(dtype)
    strike = rng.uniform(10, 50, n).astype(dtype)
    t = rng.uniform(1, 2, n).astype(dtype)
    rate, vol = dtype(0.1), dtype(0.2)
    call, put = np.zeros(n, dtype), -np.ones(n, dtype)
    black_scholes(n, price, strike, t, rate, vol, call, put)
    P, S, T = (v.astype(np.float64) for v in (price, strike, t))
    a = np.log(P / S)
    b = T * -0.1
    z = T * (0.2 * 0.2 * 2)
    c = 0.25 * z
    y = 1.0 / np.sqrt(z)
    verf = np.vectorize(math.erf)
    d1 = 0.5 + 0.5 * verf((a - b + c) * y)
    d2 = 0.5 + 0.5 * verf((a - b - c) * y)
    Se = np.exp(b) * S
    r = P * d1 - Se * d2
    tol = 1e-10 if dtype is np.float64 else 2e-4
    assert call.dtype == dtype
    assert np.allclose(call, r, rtol=tol, atol=tol * 50) and np.allclose(put, r - P + Se, rtol=tol, atol=tol * 50)


@appy.jit
def column_stats(A, y, x, lo, beta):
    #pragma parallel for
    for i in range(A.shape[1]):
        s = 0.0
        m = -1e300
        for j in range(A.shape[0]):
            s += A[j, i] * y[j]
            m = max(m, A[j, i])
        x[i] += beta * s
        lo[i] = m


@appy.jit
def upper_column_sums(A, out):
    #pragma parallel for
    for i in range(A.shape[1]):
        s = 0.0
        for j in range(i + 1):
            s += A[j, i]
        out[i] = s


@pytest.mark.parametrize("shape", [(700, 1000), (64, 64), (5000, 37), (100, 129), (3, 500)])
def test_column_reductions_run_as_strips(gpu, shape):
    """``A[j, i]`` under a parallel ``i`` and a sequential ``j``: lanes side by
    side along ``i``, the inner loop shared out between wavefronts (second loop of
    tests/integration/triton/npbench/test_gemver.py:50-56 written as a column loop)."""
    from appy_amd.backends.hip import codegen as cg

    rng = np.random.default_rng(shape[0])
    r, c = shape
    A = rng.standard_normal((r, c))
    y = rng.standard_normal(r)
    x0 = rng.standard_normal(c)
    x, lo = x0.copy(), np.zeros(c)
    column_stats(A, y, x, lo, 1.2)
    assert np.allclose(x, x0 + 1.2 * (y @ A), rtol=1e-11, atol=1e-11)
    assert np.array_equal(lo, A.max(axis=0))
    loop = [v[0] for kk, v in cg.code_cache.items() if kk[-1] == "column_stats"][-1]
    assert loop.last_launch.spec.kind == ("strip" if r >= 64 else "flat")
    if r == c or r > c:
        S = rng.standard_normal((c, c))
        out = np.zeros(c)
        upper_column_sums(S, out)
        assert np.allclose(out, np.triu(S).sum(axis=0), rtol=1e-11, atol=1e-11)


@appy.jit
def column_dots_simd(A, y, x, beta):
    #pragma parallel for
    for j in range(A.shape[1]):
        s = 0.0
        #pragma simd
        for i in range(A.shape[0]):
            s += beta * y[i] * A[i, j]
        x[j] += s


@appy.jit
def column_dots_slices(A, y, x, beta):
    #pragma parallel for
    for j in range(A.shape[1]):
        x[j] += beta * (y[:] @ A[:, j])


def test_simd_loops_down_a_column_run_as_strips_too(gpu):
    from appy_amd.backends.hip import codegen as cg

    rng = np.random.default_rng(77)
    A = rng.standard_normal((900, 333))
    y = rng.standard_normal(900)
    x0 = rng.standard_normal(333)
    for fn in (column_dots_simd, column_dots_slices):
        x = x0.copy()
        fn(A, y, x, 0.7)
        assert np.allclose(x, x0 + 0.7 * (y @ A), rtol=1e-11, atol=1e-11), fn.__name__
        loop = [v[0] for kk, v in cg.code_cache.items() if kk[-1] == fn.__name__][-1]
        assert loop.last_launch.spec.kind == "strip", fn.__name__


@appy.jit
def scale_columns(A, f, colmax):
    #pragma parallel for
    for j in range(A.shape[1]):
        m = 0.0
        #pragma simd
        for c in range(A.shape[0]):
            if A[c, j] < 0.0:
                continue
            A[c, j] = A[c, j] * f[j]
            m = max(m, A[c, j])
        colmax[j] = m


@appy.jit
def subtract_from_columns(A, q, s):
    #pragma parallel for
    for j in range(A.shape[1]):
        A[:, j] -= q[:] * s[j]


def test_column_updates_run_as_strips(gpu):
    from appy_amd.backends.hip import codegen as cg

    rng = np.random.default_rng(5)
    A = rng.standard_normal((777, 203))
    f = rng.uniform(1.0, 2.0, 203)
    ref = np.where(A < 0, A, A * f)
    colmax = np.zeros(203)
    scale_columns(A, f, colmax)
    assert np.array_equal(A, ref)
    assert np.array_equal(colmax, np.where(ref < 0, 0.0, ref).max(axis=0))
    q, s = rng.standard_normal(777), rng.standard_normal(203)
    B = ref.copy()
    subtract_from_columns(B, q, s)
    assert np.allclose(B, ref - np.outer(q, s), rtol=1e-13, atol=1e-13)
    for name in ("scale_columns", "subtract_from_columns"):
        loop = [v[0] for kk, v in cg.code_cache.items() if kk[-1] == name][-1]
        assert loop.last_launch.spec.kind == "strip", name


def test_gramschmidt_columns_run_as_strips_with_two_shared_out_loops(gpu):
    """Tall matrix: both column loops of the Gram-Schmidt step are dealt to the
    wavefronts of a strip (a reduction, then an update that uses its result)."""
    from appy_amd.backends.hip import codegen as cg

    rng = np.random.default_rng(9)
    A = rng.random((700, 130)) + np.eye(700, 130)
    Q, R = gramschmidt(A.copy())
    assert np.allclose(Q @ R, A, atol=1e-10)
    assert np.allclose(Q.T @ Q, np.eye(130), atol=1e-9)
    loop = [v[0] for kk, v in cg.code_cache.items() if kk[-1] == "gramschmidt"][-1]
    assert loop.last_launch.spec.kind == "strip" and len(loop.analysis.strip) == 2


@appy.jit
def repeated_column_smoothing(A, rounds):
    #pragma parallel for
    for j in range(A.shape[1]):
        for t in range(rounds):
            m = 0.0
            #pragma simd
            for i in range(A.shape[0]):
                m += A[i, j]
            m = m / A.shape[0]
            #pragma simd
            for i in range(A.shape[0]):
                A[i, j] = 0.5 * (A[i, j] + m)


def test_strip_loops_inside_a_sequential_loop_with_uniform_bounds(gpu):
    from appy_amd.backends.hip import codegen as cg

    rng = np.random.default_rng(10)
    A = rng.standard_normal((333, 201))
    ref = A.copy()
    for _ in range(3):
        ref = 0.5 * (ref + ref.mean(axis=0))
    repeated_column_smoothing(A, 3)
    assert np.allclose(A, ref, rtol=1e-12, atol=1e-12)
    loop = [v[0] for kk, v in cg.code_cache.items() if kk[-1] == "repeated_column_smoothing"][-1]
    assert loop.last_launch.spec.kind == "strip"


@appy.jit
def rows_into_elements(A, x, y, z, w):
    #pragma parallel for
    for i in range(A.shape[0]):
        y[i] = 0.5
        #pragma simd
        for j in range(A.shape[1]):
            y[i] += A[i, j] * x[j]
            z[i] = max(z[i], A[i, j])
            w[i] -= x[j]


@appy.jit
def running_differences(a, A, y):
    s = 10.0
    #pragma parallel for simd shared(s)
    for i in range(a.shape[0]):
        s -= a[i]
    #pragma parallel for
    for i in range(A.shape[0]):
        t = 1.0
        #pragma simd
        for j in range(A.shape[1]):
            t -= A[i, j]
        y[i] = t
    return s


@pytest.mark.parametrize("shape", [(37, 83), (300, 1000), (5, 20000)])
def test_simd_loops_that_accumulate_into_an_array_element(gpu, shape):
    """`y[i] += ...` inside a simd loop: one element is updated by every iteration of the
    loop, so it is accumulated in a register and stored once (a lane-parallel
    read-modify-write of `y[i]` would lose updates)."""
    rng = np.random.default_rng(11)
    A, x = rng.standard_normal(shape), rng.standard_normal(shape[1])
    y, z, w = np.zeros(shape[0]), np.full(shape[0], 0.25), rng.standard_normal(shape[0])
    w0 = w.copy()
    rows_into_elements(A, x, y, z, w)
    assert np.allclose(y, 0.5 + A @ x)
    assert np.array_equal(z, np.maximum(0.25, A.max(axis=1)))
    assert np.allclose(w, w0 - x.sum())
    a = rng.standard_normal(100_003)
    s = running_differences(a, A, y)
    assert s == pytest.approx(10.0 - a.sum(), rel=1e-12)
    assert np.allclose(y, 1.0 - A.sum(axis=1))


@appy.jit
def trmm_row_by_row(alpha, A, B):
    for i in range(B.shape[0]):
        #pragma parallel for simd
        for j in range(B.shape[1]):
            s = 0.0
            for k in range(i + 1, A.shape[0]):
                s += A[k, i] * B[k, j]
            B[i, j] = alpha * (B[i, j] + s)
    return B


@appy.jit
def trmm_column_by_column(alpha, A, B):
    #pragma parallel for
    for j in range(B.shape[1]):
        for i in range(B.shape[0]):
            s = 0.0
            #pragma simd
            for k in range(i + 1, A.shape[0]):
                s += A[k, i] * B[k, j]
            B[i, j] = alpha * (B[i, j] + s)
    return B


def test_trmm_in_place_updates(gpu):
    """The triangular product of the reference's NPBench tests
    (tests/integration/triton/npbench/test_trmm.py:20-38), in the two race-free orders:
    one launch per row with the columns in parallel (an in-place update whose loads all
    precede its store: runs as a strip), and one launch with the columns in parallel around
    the row loop (a stored row is read by later rows: single-wavefront teams)."""
    from appy_amd.backends.hip import codegen as cg

    M, N = 150, 200
    A = np.fromfunction(lambda i, j: ((i * j) % M) / M, (M, M), dtype=np.float64)
    np.fill_diagonal(A, 1.0)
    B = np.fromfunction(lambda i, j: ((N + i - j) % N) / N, (M, N), dtype=np.float64)
    want = B.copy()
    for i in range(M):
        want[i, :] += A[i + 1:, i] @ want[i + 1:, :]
    want *= 1.5
    got = trmm_row_by_row(1.5, A, B.copy())
    assert np.allclose(got, want, atol=1e-6)
    loop = next(v[0] for k, v in cg.code_cache.items() if k[-1] == "trmm_row_by_row")
    assert loop.analysis.strip is not None and loop.analysis.multi_wave_ok
    assert loop.choose_spec(N, dict(i=0, A_shape_0=M, alpha=1.5), dict(A=A, B=B)).kind == "strip"
    got = trmm_column_by_column(1.5, A, B.copy())
    assert np.allclose(got, want, atol=1e-6)
    loop = next(v[0] for k, v in cg.code_cache.items() if k[-1] == "trmm_column_by_column")
    assert not loop.analysis.multi_wave_ok


# ---- further NPBench kernels in the reference's loop style (polybench covariance / correlation /
# heat-3d / doitgen, deep-learning softmax): column walks under triangular loops, 3-D stencils,
# 4-D arrays addressed through a flattened parallel index, slices of 3-D arrays -------------------
@appy.jit
def covariance(data, cov, mean):
    #pragma parallel for
    for j in range(data.shape[1]):
        s = 0.0
        for k in range(data.shape[0]):
            s += data[k, j]
        mean[j] = s / data.shape[0]
    #pragma parallel for
    for k in range(data.shape[0]):
        data[k, :] -= mean[:]
    #pragma parallel for
    for i in range(data.shape[1]):
        for j in range(i, data.shape[1]):
            s = 0.0
            #pragma simd
            for k in range(data.shape[0]):
                s += data[k, i] * data[k, j]
            cov[i, j] = cov[j, i] = s / (data.shape[0] - 1.0)
def covariance_ref(data, cov, mean):
    mean[:] = data.mean(axis=0); data -= mean
    cov[:] = data.T @ data / (data.shape[0] - 1.0)

@appy.jit
def heat_3d(T, A, B):
    for t in range(1, T):
        #pragma parallel for
        for i in range(1, A.shape[0] - 1):
            for j in range(1, A.shape[1] - 1):
                #pragma simd
                for k in range(1, A.shape[2] - 1):
                    B[i, j, k] = (0.125 * (A[i + 1, j, k] - 2.0 * A[i, j, k] + A[i - 1, j, k]) + 0.125 * (A[i, j + 1, k] - 2.0 * A[i, j, k] + A[i, j - 1, k])
                                  + 0.125 * (A[i, j, k + 1] - 2.0 * A[i, j, k] + A[i, j, k - 1]) + A[i, j, k])
        #pragma parallel for
        for i in range(1, A.shape[0] - 1):
            for j in range(1, A.shape[1] - 1):
                #pragma simd
                for k in range(1, A.shape[2] - 1):
                    A[i, j, k] = (0.125 * (B[i + 1, j, k] - 2.0 * B[i, j, k] + B[i - 1, j, k]) + 0.125 * (B[i, j + 1, k] - 2.0 * B[i, j, k] + B[i, j - 1, k])
                                  + 0.125 * (B[i, j, k + 1] - 2.0 * B[i, j, k] + B[i, j, k - 1]) + B[i, j, k])
def heat_3d_ref(T, A, B):
    for t in range(1, T):
        B[1:-1, 1:-1, 1:-1] = (0.125 * (A[2:, 1:-1, 1:-1] - 2.0 * A[1:-1, 1:-1, 1:-1] + A[:-2, 1:-1, 1:-1]) + 0.125 * (A[1:-1, 2:, 1:-1] - 2.0 * A[1:-1, 1:-1, 1:-1] + A[1:-1, :-2, 1:-1]) + 0.125 * (A[1:-1, 1:-1, 2:] - 2.0 * A[1:-1, 1:-1, 1:-1] + A[1:-1, 1:-1, 0:-2]) + A[1:-1, 1:-1, 1:-1])
        A[1:-1, 1:-1, 1:-1] = (0.125 * (B[2:, 1:-1, 1:-1] - 2.0 * B[1:-1, 1:-1, 1:-1] + B[:-2, 1:-1, 1:-1]) + 0.125 * (B[1:-1, 2:, 1:-1] - 2.0 * B[1:-1, 1:-1, 1:-1] + B[1:-1, :-2, 1:-1]) + 0.125 * (B[1:-1, 1:-1, 2:] - 2.0 * B[1:-1, 1:-1, 1:-1] + B[1:-1, 1:-1, 0:-2]) + B[1:-1, 1:-1, 1:-1])

@appy.jit
def softmax4(x, out):
    #pragma parallel for
    for n in range(x.shape[0] * x.shape[1] * x.shape[2]):
        a = n // (x.shape[1] * x.shape[2])
        b = (n // x.shape[2]) % x.shape[1]
        c = n % x.shape[2]
        m = -1e30
        #pragma simd
        for k in range(x.shape[3]):
            m = max(m, x[a, b, c, k])
        s = 0.0
        #pragma simd
        for k in range(x.shape[3]):
            s += np.exp(x[a, b, c, k] - m)
        #pragma simd
        for k in range(x.shape[3]):
            out[a, b, c, k] = np.exp(x[a, b, c, k] - m) / s
def softmax4_ref(x, out):
    e = np.exp(x - x.max(axis=-1, keepdims=True)); out[:] = e / e.sum(axis=-1, keepdims=True)

@appy.jit
def softmax_slices(x, out):
    #pragma parallel for
    for i in range(x.shape[0]):
        for j in range(x.shape[1]):
            m = np.max(x[i, j, :])
            s = np.sum(np.exp(x[i, j, :] - m))
            out[i, j, :] = np.exp(x[i, j, :] - m) / s
def softmax_slices_ref(x, out):
    e = np.exp(x - x.max(axis=-1, keepdims=True)); out[:] = e / e.sum(axis=-1, keepdims=True)

@appy.jit
def correlation(data, corr, mean, std):
    #pragma parallel for
    for j in range(data.shape[1]):
        s = 0.0
        q = 0.0
        for k in range(data.shape[0]):
            s += data[k, j]
        mu = s / data.shape[0]
        for k in range(data.shape[0]):
            q += (data[k, j] - mu) ** 2
        sd = math.sqrt(q / data.shape[0])
        mean[j] = mu
        std[j] = 1.0 if sd <= 0.1 else sd
    #pragma parallel for
    for k in range(data.shape[0]):
        data[k, :] = (data[k, :] - mean[:]) / (math.sqrt(data.shape[0]) * std[:])
    #pragma parallel for
    for i in range(data.shape[1]):
        corr[i, i] = 1.0
        for j in range(i + 1, data.shape[1]):
            s = 0.0
            #pragma simd
            for k in range(data.shape[0]):
                s += data[k, i] * data[k, j]
            corr[i, j] = s
            corr[j, i] = s
def correlation_ref(data, corr, mean, std):
    mean[:] = data.mean(axis=0); sd = data.std(axis=0); sd[sd <= 0.1] = 1.0; std[:] = sd
    data -= mean; data /= math.sqrt(data.shape[0]) * std
    corr[:] = data.T @ data; np.fill_diagonal(corr, 1.0)

@appy.jit
def doitgen(A, C4, tmp):
    #pragma parallel for
    for n in range(A.shape[0] * A.shape[1]):
        r = n // A.shape[1]
        q = n % A.shape[1]
        for p in range(A.shape[2]):
            s = 0.0
            #pragma simd
            for k in range(A.shape[2]):
                s += A[r, q, k] * C4[k, p]
            tmp[r, q, p] = s
        #pragma simd
        for p in range(A.shape[2]):
            A[r, q, p] = tmp[r, q, p]
def doitgen_ref(A, C4, tmp):
    tmp[:] = A @ C4; A[:] = tmp


def test_more_npbench_kernels(gpu):
    rng = np.random.default_rng(0)

    def check(fn, ref, *args, tol=1e-9):
        mine = [a.copy() if hasattr(a, "copy") else a for a in args]
        ref(*args)
        fn(*mine)
        for got, want in zip(mine, args):
            if hasattr(got, "shape"):
                assert np.allclose(got, want, rtol=tol, atol=tol), fn.__name__

    N, M = 130, 90
    check(covariance, covariance_ref, rng.random((N, M)), np.zeros((M, M)), np.zeros(M))
    check(correlation, correlation_ref, rng.random((N, M)), np.zeros((M, M)), np.zeros(M), np.zeros(M))
    check(heat_3d, heat_3d_ref, 5, rng.random((20, 22, 70)), rng.random((20, 22, 70)))
    x = rng.standard_normal((3, 4, 17, 65))
    check(softmax4, softmax4_ref, x, np.zeros_like(x))
    x3 = rng.standard_normal((7, 17, 65))
    check(softmax_slices, softmax_slices_ref, x3, np.zeros_like(x3))
    check(doitgen, doitgen_ref, rng.random((6, 5, 40)), rng.random((40, 40)), np.zeros((6, 5, 40)))


@appy.jit
def shift_planes(A, B):
    #pragma parallel for
    for i in range(A.shape[0]):
        for j in range(1, A.shape[1]):
            #pragma simd
            for k in range(A.shape[2]):
                B[i, j, k] = A[i, j - 1, k] + 1.0


def test_collapsed_nests_keep_sequential_meaning_when_arguments_alias(gpu):
    """`B[i, j] = A[i, j - 1] + 1` is independent across j for two arrays and a running sum
    along j when both names are one array: the collapsed shape is only taken when the
    arguments do not share memory."""
    from appy_amd.backends.hip import codegen as cg

    rng = np.random.default_rng(12)
    A = rng.random((6, 40, 50))
    B = np.zeros_like(A)
    shift_planes(A, B)
    assert np.array_equal(B[:, 1:], A[:, :-1] + 1.0) and not B[:, 0].any()
    loop = next(v[0] for k, v in cg.code_cache.items() if k[-1] == "shift_planes")
    assert loop.last_launch.spec.collapse
    C = A.copy()
    shift_planes(C, C)                          # one array under both names
    assert not loop.last_launch.spec.collapse
    want = A.copy()
    for j in range(1, 40):
        want[:, j] = want[:, j - 1] + 1.0
    assert np.allclose(C, want)
    # degenerate trip counts of the inner loop
    one = rng.random((5, 1, 8))
    out = np.full_like(one, -1.0)
    shift_planes(one, out)
    assert np.all(out == -1.0)
    two = rng.random((5, 2, 8))
    out = np.zeros_like(two)
    shift_planes(two, out)
    assert np.array_equal(out[:, 1], two[:, 0] + 1.0)


@appy.jit
def tall_column_stats(A, total, top, scaled, w):
    #pragma parallel for
    for j in range(A.shape[1]):
        bias = w * 2.0
        s = 0.0
        m = -1e30
        for i in range(A.shape[0]):
            s += A[i, j]
            m = max(m, A[i, j])
        total[j] = s
        top[j] = m
        scaled[j] = (s + bias) / A.shape[0]


@appy.jit
def tall_column_dot(A, y, x):
    #pragma parallel for
    for j in range(A.shape[1]):
        s = 0.0
        #pragma simd
        for i in range(A.shape[0]):
            s += A[i, j] * y[i]
        x[j] = s


@pytest.mark.parametrize("shape,dtype", [((200_003, 20), np.float64), ((100_000, 64), np.float32),
                                         ((50_001, 257), np.float32), ((70_000, 3), np.int32)])
def test_tall_matrices_with_few_columns_run_as_two_phase_strips(gpu, shape, dtype):
    """Few columns, many rows: several workgroups share the rows of a strip (partial sums
    and maxima in a scratch buffer), a second small kernel runs the rest of the body."""
    from appy_amd.backends.hip import codegen as cg

    rng = np.random.default_rng(21)
    A = (rng.standard_normal(shape) * 10).astype(dtype)
    n, m = shape
    total, top, scaled = np.zeros(m, dtype), np.zeros(m, dtype), np.zeros(m, np.float64)
    tall_column_stats(A, total, top, scaled, 0.25)
    loop = next(v[0] for k, v in cg.code_cache.items() if k[-1] == "tall_column_stats"
                and v[0].analysis.arrays["A"].ty.name == np.dtype(dtype).name)
    assert loop.last_launch.spec.phase == 1 and loop.last_launch.second is not None
    want = A.sum(axis=0, dtype=np.float64)
    if np.dtype(dtype).kind == "f":
        assert np.allclose(total, want, rtol=1e-4 if dtype == np.float32 else 1e-11, atol=1e-2 if dtype == np.float32 else 1e-7)
        assert np.allclose(scaled, (want + 0.5) / n, rtol=1e-4 if dtype == np.float32 else 1e-11, atol=1e-6)
    else:
        assert np.array_equal(total, want.astype(dtype))
    assert np.array_equal(top, A.max(axis=0))
    # twice in a row (the scratch buffer is reused), then on a smaller matrix
    tall_column_stats(A, total, top, scaled, 0.25)
    assert np.array_equal(top, A.max(axis=0))
    B = A[: n // 3].copy()
    tall_column_stats(B, total, top, scaled, 0.25)
    assert np.array_equal(top, B.max(axis=0))
    if np.dtype(dtype).kind == "f":
        y = rng.standard_normal(n).astype(dtype)
        x = np.zeros(m, dtype)
        tall_column_dot(A, y, x)
        ref = A.astype(np.float64).T @ y.astype(np.float64)
        budget = np.abs(A.astype(np.float64)).T @ np.abs(y.astype(np.float64))
        assert np.all(np.abs(x - ref) <= (1e-5 if dtype == np.float32 else 1e-12) * budget + 1e-30)


@appy.jit
def few_long_rows(A, B, C, y, z, scale):
    #pragma parallel for
    for i in range(A.shape[0]):
        #pragma simd
        for j in range(A.shape[1]):
            C[i, j] = A[i, j] + B[i, j]
    #pragma parallel for
    for i in range(A.shape[0]):
        f = scale[i] * 2.0
        s = 0.0
        m = -1e30
        #pragma simd
        for j in range(A.shape[1]):
            s += A[i, j] * f
            m = max(m, B[i, j])
        y[i] = s + 1.0
        z[i] = m


@appy.jit
def csr_rows(data, indptr, indices, x, y):
    #pragma parallel for
    for i in range(y.shape[0]):
        start, end = indptr[i], indptr[i + 1]
        s = 0.0
        #pragma simd
        for k in range(start, end):
            s += data[k] * x[indices[k]]
        y[i] = s


@pytest.mark.parametrize("shape", [(1, 1_000_003), (3, 400_001), (40, 70_000)])
def test_few_very_long_rows_are_shared_by_several_workgroups(gpu, shape):
    """Fewer rows than half the CUs, each very long: several workgroups take parts of a row;
    elementwise loops need nothing more, reductions meet in a finishing kernel."""
    from appy_amd.backends.hip import codegen as cg

    rng = np.random.default_rng(31)
    A, B = rng.standard_normal(shape), rng.standard_normal(shape)
    C = np.zeros(shape)
    y, z, scale = np.zeros(shape[0]), np.zeros(shape[0]), rng.random(shape[0])
    few_long_rows(A, B, C, y, z, scale)
    loops = [v[0] for k, v in cg.code_cache.items() if k[-1] == "few_long_rows"]
    assert all(lp.last_launch.spec.phase == 1 for lp in loops)
    assert sorted(lp.last_launch.second is not None for lp in loops) == [False, True]
    assert np.array_equal(C, A + B)
    assert np.allclose(y, (A * (scale[:, None] * 2.0)).sum(axis=1) + 1.0, rtol=1e-11, atol=1e-8)
    assert np.array_equal(z, B.max(axis=1))
    # CSR rows whose bounds are read per row: two long rows and an empty one
    n = 300_000
    data, x = rng.standard_normal(2 * n), rng.standard_normal(1000)
    indices = rng.integers(0, 1000, 2 * n).astype(np.int32)
    indptr = np.array([0, n, n, 2 * n], dtype=np.int64)
    out = np.zeros(3)
    csr_rows(data, indptr, indices, x, out)
    want = [np.dot(data[:n], x[indices[:n]]), 0.0, np.dot(data[n:], x[indices[n:]])]
    assert np.allclose(out, want, rtol=1e-10, atol=1e-7)
    loop = next(v[0] for k, v in cg.code_cache.items() if k[-1] == "csr_rows")
    assert loop.last_launch.spec.phase == 1


@appy.jit
def shifted_column_updates(A, f, C, D):
    #pragma parallel for
    for j in range(A.shape[1]):
        w = f[j] * 2.0
        for i in range(1, A.shape[0]):
            C[i, j] = A[i, j] * w + A[i - 1, j]
            D[i - 1, j] = A[i, j] - w


@pytest.mark.parametrize("shape", [(3, 5000), (700, 300), (100_000, 48), (300_000, 5)])
def test_column_updates_written_without_simd(gpu, shape):
    """A sequential loop down the columns that only stores, each iteration to its own row of
    the arrays it stores to: shared out between the wavefronts of a strip like a reduction
    loop (and between workgroups when the matrix is tall and narrow); with few rows one lane
    per column walks them."""
    from appy_amd.backends.hip import codegen as cg

    rng = np.random.default_rng(41)
    A, f = rng.standard_normal(shape), rng.standard_normal(shape[1])
    C, D = np.zeros(shape), np.zeros(shape)
    shifted_column_updates(A, f, C, D)
    assert np.array_equal(C[1:], A[1:] * (f * 2.0) + A[:-1]) and not C[0].any()
    assert np.array_equal(D[:-1], A[1:] - f * 2.0) and not D[-1].any()
    loop = next(v[0] for k, v in cg.code_cache.items() if k[-1] == "shifted_column_updates")
    spec = loop.last_launch.spec
    assert loop.analysis.strip is not None
    assert spec.kind == ("flat" if shape[0] < 64 else "strip")
    assert spec.phase == (1 if shape[0] >= 100_000 else 0) and loop.last_launch.second is None


@appy.jit
def shape_rowstats(A, y, z):
    #pragma parallel for
    for i in range(A.shape[0]):
        s = 0.0
        m = -1e30
        #pragma simd
        for j in range(A.shape[1]):
            s += A[i, j]
            m = max(m, A[i, j])
        y[i] = s
        z[i] = m


@appy.jit
def shape_colstats(A, y, z):
    #pragma parallel for
    for j in range(A.shape[1]):
        s = 0.0
        m = -1e30
        for i in range(A.shape[0]):
            s += A[i, j]
            m = max(m, A[i, j])
        y[j] = s
        z[j] = m


@appy.jit
def shape_rowscale(A, f, C):
    #pragma parallel for
    for i in range(A.shape[0]):
        #pragma simd
        for j in range(A.shape[1]):
            C[i, j] = A[i, j] * f[i] + 1.0


@appy.jit
def shape_colscale(A, f, C):
    #pragma parallel for
    for j in range(A.shape[1]):
        for i in range(A.shape[0]):
            C[i, j] = A[i, j] * f[j] + 1.0


_EDGE_SHAPES = [(1, 200_000), (2, 65_537), (127, 8193), (128, 8192), (129, 4095), (1023, 1025), (4096, 257),
                (8193, 63), (32_769, 64), (65_536, 3), (200_000, 1), (63, 32_768), (64, 32_767), (3, 3)]


@pytest.mark.parametrize("shape", _EDGE_SHAPES)
def test_row_and_column_loops_over_shapes_at_the_edges_of_the_launch_heuristics(gpu, shape):
    """The same four loops (row and column reductions, row and column updates) over matrices of
    every aspect ratio, with extents at and next to the thresholds where the launch picks another
    kernel shape (teams of a wavefront or a workgroup, strips, one or two phases, flat)."""
    n, m = shape
    for dt in (np.float32, np.float64):
        rng = np.random.default_rng(n * 31 + m)
        A = rng.standard_normal(shape).astype(dt)
        tol = dict(rtol=1e-3, atol=1e-2) if dt == np.float32 else dict(rtol=1e-9, atol=1e-9)
        y, z = np.zeros(n, dt), np.zeros(n, dt)
        shape_rowstats(A, y, z)
        assert np.allclose(y, A.sum(axis=1, dtype=np.float64), **tol) and np.array_equal(z, A.max(axis=1))
        y, z = np.zeros(m, dt), np.zeros(m, dt)
        shape_colstats(A, y, z)
        assert np.allclose(y, A.sum(axis=0, dtype=np.float64), **tol) and np.array_equal(z, A.max(axis=0))
        f, C = rng.standard_normal(n).astype(dt), np.zeros_like(A)
        shape_rowscale(A, f, C)
        assert np.array_equal(C, A * f[:, None] + dt(1.0))
        f, C = rng.standard_normal(m).astype(dt), np.zeros_like(A)
        shape_colscale(A, f, C)
        assert np.array_equal(C, A * f[None, :] + dt(1.0))


# rows that several simd loops of an iteration read (layer norm, RMS norm, soft-max over 2-D
# rows): kept in registers when a row is a whole, small number of vector steps per lane, read
# again from memory otherwise - both against NumPy in float64
@appy.jit
def layer_norm_rows(x, g, b, out, eps):
    #pragma parallel for
    for i in range(x.shape[0]):
        s = 0.0
        #pragma simd
        for j in range(x.shape[1]):
            s += x[i, j]
        mu = s / x.shape[1]
        v = 0.0
        #pragma simd
        for j in range(x.shape[1]):
            v += (x[i, j] - mu) * (x[i, j] - mu)
        r = 1.0 / np.sqrt(v / x.shape[1] + eps)
        #pragma simd
        for j in range(x.shape[1]):
            out[i, j] = (x[i, j] - mu) * r * g[j] + b[j]


@appy.jit
def rms_norm_rows(x, g, out, eps):
    for i in appy.prange(x.shape[0]):
        r = 1.0 / np.sqrt(np.mean(x[i] * x[i]) + eps)
        out[i] = x[i] * r * g


@appy.jit
def softmax_rows(x, out):
    for i in appy.prange(x.shape[0]):
        m = np.max(x[i])
        out[i] = np.exp(x[i] - m) / np.sum(np.exp(x[i] - m))


@pytest.mark.parametrize("n,d", [(300, 512), (1000, 1024), (257, 4096), (600, 8192), (3, 32768), (40, 16384),
                                 (300, 1000), (33, 4100), (5000, 256), (7, 1024)])
def test_rows_read_by_several_simd_loops(gpu, n, d):
    from appy_amd.backends.hip import codegen as cg

    rng = np.random.default_rng(n * 7 + d)
    x = (rng.standard_normal((n, d)) * 3 + 1).astype(np.float32)
    g, b = rng.random(d, dtype=np.float32) + 0.5, rng.random(d, dtype=np.float32)
    x64 = x.astype(np.float64)
    mu, var = x64.mean(axis=1, keepdims=True), x64.var(axis=1, keepdims=True)
    out = np.zeros_like(x)
    layer_norm_rows(x, g, b, out, 1e-5)
    np.testing.assert_allclose(out, (x64 - mu) / np.sqrt(var + 1e-5) * g + b, rtol=2e-4, atol=2e-4)
    loop = next(v[0] for k, v in cg.code_cache.items() if k[-1] == "layer_norm_rows")
    spec = loop.last_launch.spec
    if (n, d) in ((300, 512), (1000, 1024), (257, 4096), (600, 8192), (5000, 256)):
        assert spec.row_steps == d // (spec.width * spec.vec) > 0, spec.tag()
    if d in (1000, 4100):
        assert spec.row_steps == 0, spec.tag()
    out = np.zeros_like(x)
    rms_norm_rows(x, g, out, 1e-5)
    np.testing.assert_allclose(out, x64 / np.sqrt((x64 * x64).mean(axis=1, keepdims=True) + 1e-5) * g, rtol=2e-4, atol=2e-4)
    out = np.zeros_like(x)
    softmax_rows(x, out)
    e = np.exp(x64 - x64.max(axis=1, keepdims=True))
    np.testing.assert_allclose(out, e / e.sum(axis=1, keepdims=True), rtol=2e-4, atol=1e-7)
    # the result written over the input: every lane has read its part of the row before it stores
    y = x.copy()
    layer_norm_rows(y, g, b, y, 1e-5)
    np.testing.assert_allclose(y, (x64 - mu) / np.sqrt(var + 1e-5) * g + b, rtol=2e-4, atol=2e-4)


@appy.jit
def softmax_planes(x, out):
    #pragma parallel for
    for i in range(x.shape[0]):
        for j in range(x.shape[1]):
            m = np.max(x[i, j, :])
            s = np.sum(np.exp(x[i, j, :] - m))
            out[i, j, :] = np.exp(x[i, j, :] - m) / s


def test_collapsed_nests_keep_rows_in_registers_too(gpu):
    """`parallel i / for j / three simd loops over x[i, j, :]`: the pairs (i, j) are the
    iterations, and each keeps its row in registers when the row length allows."""
    from appy_amd.backends.hip import codegen as cg

    rng = np.random.default_rng(77)
    for shape in ((6, 50, 512), (3, 7, 2048), (5, 9, 500)):
        x = (rng.standard_normal(shape) * 4).astype(np.float32)
        out = np.zeros_like(x)
        softmax_planes(x, out)
        x64 = x.astype(np.float64)
        e = np.exp(x64 - x64.max(axis=-1, keepdims=True))
        np.testing.assert_allclose(out, e / e.sum(axis=-1, keepdims=True), rtol=2e-4, atol=1e-7)
        spec = next(v[0] for k, v in cg.code_cache.items() if k[-1] == "softmax_planes").last_launch.spec
        assert spec.collapse and bool(spec.row_steps) == (shape[2] % 512 == 0), spec.tag()


@appy.jit
def normalise_then_sum(x, out, t):
    #pragma parallel for
    for i in range(x.shape[0]):
        s = 0.0
        #pragma simd
        for j in range(x.shape[1]):
            s += x[i, j]
        #pragma simd
        for j in range(x.shape[1]):
            out[i, j] = x[i, j] / s
        u = 0.0
        #pragma simd
        for j in range(x.shape[1]):
            u += x[i, j]
        t[i] = u


def test_rows_are_not_kept_in_registers_when_arguments_share_memory(gpu):
    """`out` and `x` the same array: the third loop must see what the second stored."""
    import torch

    rng = np.random.default_rng(3)
    x = rng.random((200, 1024), dtype=np.float32) + 0.5
    sep_out, t = np.zeros_like(x), np.zeros(200, np.float32)
    normalise_then_sum(x, sep_out, t)
    np.testing.assert_allclose(t, x.sum(axis=1), rtol=1e-5)
    y, t = x.copy(), np.zeros(200, np.float32)
    normalise_then_sum(y, y, t)
    np.testing.assert_allclose(y, sep_out, rtol=1e-6)
    np.testing.assert_allclose(t, np.ones(200), rtol=1e-5)
    yd, td = torch.tensor(x, device="cuda"), torch.zeros(200, device="cuda")
    normalise_then_sum(yd, yd, td)
    np.testing.assert_allclose(td.cpu().numpy(), np.ones(200), rtol=1e-5)


@appy.jit
def weighted_rows(x, w, out):
    #pragma parallel for
    for i in range(x.shape[0]):
        s = 0.0
        #pragma simd
        for j in range(x.shape[1]):
            s += x[i, j] * w[i, j]
        #pragma simd
        for j in range(x.shape[1]):
            out[i, j] = x[i, j] * s - w[i, j]


@pytest.mark.parametrize("dtype,n,d", [("float64", 100, 512), ("float64", 7, 16384), ("float64", 1000, 3072),
                                       ("float32", 20000, 128), ("float32", 2, 32768), ("float32", 64, 12288),
                                       ("float16", 300, 256), ("float16", 50, 1024)])
def test_two_rows_kept_in_registers_over_element_types(gpu, dtype, n, d):
    """Two arrays cached per iteration (x and w), 2, 4 and 8 elements per vector step, teams
    from two lanes to a whole workgroup."""
    from appy_amd.backends.hip import codegen as cg

    rng = np.random.default_rng(d + n)
    x = (rng.standard_normal((n, d)) * 0.25).astype(dtype)
    w = (rng.standard_normal((n, d)) * 0.25).astype(dtype)
    out = np.zeros_like(x)
    weighted_rows(x, w, out)
    x64, w64 = x.astype(np.float64), w.astype(np.float64)
    ref = x64 * (x64 * w64).sum(axis=1, keepdims=True) - w64
    tol = {"float64": 1e-11, "float32": 2e-4, "float16": 3e-2}[dtype]
    np.testing.assert_allclose(out, ref, rtol=tol, atol=tol)
    loop = next(v[0] for k, v in cg.code_cache.items()
                if k[-1] == "weighted_rows" and v[0].analysis.arrays["x"].ty.name == dtype)
    spec = loop.last_launch.spec
    assert spec.row_steps == d // (spec.width * spec.vec) > 0, spec.tag()
    text = loop.kernel_for(spec).src.text
    assert "__rc0[" in text and "__rc1[" in text
