"""Array statements inside parallel loops on the GPU: the slice forms of the
reference's Metal NPBench tests (tests/integration/metal/npbench/test_gemver.py,
test_symm.py, test_gramschmidt.py, test_fdtd_2d.py, test_floyd_warshall.py,
test_jacobi_2d.py, test_syr2k.py, test_jacobi_1d.py): whole-row and column
slices, slices with negative and open bounds, ``@`` of two slices, ``np.minimum``
of slices, in-place column updates.  The expected values are the same statements
executed by NumPy (the un-jitted function) on the same inputs."""
import numpy as np
import pytest

import appy

pytestmark = pytest.mark.gpu


def both(fn, *args):
    """Run ``fn`` jitted and un-jitted on copies of the arguments."""
    cp = lambda a: a.copy() if isinstance(a, np.ndarray) else a
    got = appy.jit(fn)(*[cp(a) for a in args])
    ref = fn(*[cp(a) for a in args])
    return got, ref


def close(got, ref, **kw):
    if isinstance(ref, tuple):
        return all(np.allclose(g, r, **kw) for g, r in zip(got, ref))
    return np.allclose(got, ref, **kw)


def gemver(alpha, beta, A, u1, u2, v1, v2, w, x, yv, z):
    M, N = A.shape
    #pragma parallel for
    for i in range(M):
        A[i, :] += u1[i] * v1[:] + u2[i] * v2[:]
    #pragma parallel for
    for j in range(N):
        x[j] += beta * (yv[:] @ A[:, j]) + z[j]
    #pragma parallel for
    for i in range(M):
        w[i] += alpha * (A[i, :] @ x[:])
    return A, x, w


def test_gemver_row_updates_and_dots_of_slices(gpu):
    rng = np.random.default_rng(0)
    n = 150
    A = rng.random((n, n))
    vecs = [rng.random(n) for _ in range(8)]
    got, ref = both(gemver, 1.5, 1.2, A, *vecs)
    assert close(got, ref, atol=1e-6)


def symm(alpha, beta, C, A, B):
    temp2 = np.empty((C.shape[1],), dtype=C.dtype)
    C *= beta
    for i in range(C.shape[0]):
        #pragma parallel for
        for j in range(C.shape[1]):
            C[:i, j] += alpha * B[i, j] * A[i, :i]
            temp2[j] = B[:i, j] @ A[i, :i]
        C[i, :] += alpha * B[i, :] * A[i, i] + alpha * temp2
    return C


def test_symm_column_slices(gpu):
    rng = np.random.default_rng(1)
    m, n = 40, 50
    got, ref = both(symm, 1.5, 1.2, rng.random((m, n)), rng.random((m, m)), rng.random((m, n)))
    assert close(got, ref, atol=1e-6)


def gramschmidt(A):
    M, N = A.shape
    Q = np.zeros((M, N), dtype=A.dtype)
    R = np.zeros((N, N), dtype=A.dtype)
    for k in range(N):
        nrm = A[:, k] @ A[:, k]
        R[k, k] = np.sqrt(nrm)
        Q[:, k] = A[:, k] / R[k, k]
        #pragma parallel for
        for j in range(k + 1, N):
            s = Q[:, k] @ A[:, j]
            R[k, j] = s
            A[:, j] -= Q[:, k] * s
    return Q, R


def test_gramschmidt_column_dot_and_update(gpu):
    rng = np.random.default_rng(2)
    A = rng.random((60, 40)) + np.eye(60, 40)
    (Q, R), (Qr, Rr) = both(gramschmidt, A)
    assert np.allclose(Q, Qr, atol=1e-6) and np.allclose(R, Rr, atol=1e-6)
    assert np.allclose(Q @ R, A, atol=1e-8)


def fdtd_2d(TMAX, ex, ey, hz, _fict_):
    for t in range(TMAX):
        ey[0, :] = _fict_[t]
        #pragma parallel for
        for i in range(1, ey.shape[0]):
            ey[i, :] -= 0.5 * (hz[i, :] - hz[i - 1, :])
        #pragma parallel for
        for i in range(ex.shape[0]):
            ex[i, 1:] -= 0.5 * (hz[i, 1:] - hz[i, :-1])
        #pragma parallel for
        for i in range(hz.shape[0] - 1):
            hz[i, :-1] -= 0.7 * (ex[i, 1:] - ex[i, :-1] + ey[i + 1, :-1] -
                                  ey[i, :-1])
    return ey, ex, hz


def test_fdtd_2d_shifted_slices(gpu):
    rng = np.random.default_rng(3)
    nx, ny, tmax = 70, 90, 8
    got, ref = both(fdtd_2d, tmax, rng.random((nx, ny)), rng.random((nx, ny)), rng.random((nx, ny)),
                    np.arange(tmax, dtype=np.float64))
    assert close(got, ref, atol=1e-6)


def floyd_warshall(path):
    for k in range(path.shape[0]):
        #pragma parallel for
        for i in range(path.shape[0]):
            path[i, :] = np.minimum(path[i, :], path[i, k] + path[k, :])
    return path


def test_floyd_warshall_np_minimum_of_slices(gpu):
    rng = np.random.default_rng(4)
    n = 64
    path = rng.integers(1, 100, (n, n)).astype(np.int32)
    got, ref = both(floyd_warshall, path)
    assert np.array_equal(got, ref)


def jacobi_2d(TSTEPS, A, B):
    for t in range(1, TSTEPS):
        #pragma parallel for
        for i in range(1, A.shape[0] - 1):
            B[i, 1:-1] = 0.2 * (A[i, 1:-1] + A[i, :-2] + A[i, 2:] +
                                 A[i - 1, 1:-1] + A[i + 1, 1:-1])
        #pragma parallel for
        for i in range(1, B.shape[0] - 1):
            A[i, 1:-1] = 0.2 * (B[i, 1:-1] + B[i, :-2] + B[i, 2:] +
                                 B[i - 1, 1:-1] + B[i + 1, 1:-1])
    return A, B


def test_jacobi_2d_interior_slices(gpu):
    rng = np.random.default_rng(5)
    got, ref = both(jacobi_2d, 6, rng.random((80, 80)), rng.random((80, 80)))
    assert close(got, ref, atol=1e-8)


def syr2k(alpha, beta, C, A, B):
    #pragma parallel for
    for i in range(A.shape[0]):
        C[i, :i + 1] *= beta
        for k in range(A.shape[1]):
            C[i, :i + 1] += (A[:i + 1, k] * alpha * B[i, k] +
                             B[:i + 1, k] * alpha * A[i, k])
    return C


def syr2k_loops(alpha, beta, C, A, B):
    #pragma parallel for
    for i in range(A.shape[0]):
        #pragma simd
        for j in range(i + 1):
            C[i, j] *= beta
        for k in range(A.shape[1]):
            #pragma simd
            for j in range(i + 1):
                C[i, j] += (A[j, k] * alpha * B[i, k] +
                            B[j, k] * alpha * A[i, k])
    return C


def test_syr2k_triangular_slices_and_loops(gpu):
    rng = np.random.default_rng(6)
    n, m = 60, 45
    C, A, B = rng.random((n, n)), rng.random((n, m)), rng.random((n, m))
    got, ref = both(syr2k, 1.5, 1.2, C, A, B)
    assert close(got, ref, atol=1e-6)
    got2 = appy.jit(syr2k_loops)(1.5, 1.2, C.copy(), A, B)
    assert close(got2, ref, atol=1e-6)


def jacobi_1d(TSTEPS, A, B):
    for t in range(1, TSTEPS):
        #pragma parallel for simd
        for i in range(1, A.shape[0] - 1):
            B[i] = 0.33333 * (A[i - 1] + A[i] + A[i + 1])
        #pragma parallel for simd
        for i in range(1, A.shape[0] - 1):
            A[i] = 0.33333 * (B[i - 1] + B[i] + B[i + 1])
    return A, B


def test_jacobi_1d(gpu):
    rng = np.random.default_rng(7)
    got, ref = both(jacobi_1d, 10, rng.random(4001), rng.random(4001))
    assert close(got, ref, atol=0)


def gram_schmidt_step_reading_back(Q, A, R, k):
    #pragma parallel for
    for j in range(k + 1, A.shape[1]):
        R[k, j] = np.sum(Q[:, k] * A[:, j])        # stored by one lane of the team ...
        A[:, j] -= Q[:, k] * R[k, j]               # ... and read back by all of them


def test_value_stored_by_the_team_leader_and_read_back_by_the_team(gpu):
    """The read-after-write pattern of docs/metal_simd_memory_hazards.md:38-60 in its
    natural form: correct on teams inside one wavefront, which is what such loop
    nests are kept to (no strip, no workgroup team)."""
    from appy_amd.backends.hip import codegen as cg

    rng = np.random.default_rng(14)
    A = rng.standard_normal((900, 70))
    Q = rng.standard_normal((900, 70))
    R = np.zeros((70, 70))
    k = 3
    ref_R = R.copy()
    ref_R[k, k + 1:] = Q[:, k] @ A[:, k + 1:]
    ref_A = A.copy()
    ref_A[:, k + 1:] -= np.outer(Q[:, k], ref_R[k, k + 1:])
    appy.jit(gram_schmidt_step_reading_back)(Q, A, R, k)
    assert np.allclose(R, ref_R, rtol=1e-12, atol=1e-12) and np.allclose(A, ref_A, rtol=1e-11, atol=1e-11)
    loop = [v[0] for kk, v in cg.code_cache.items() if kk[-1] == "gram_schmidt_step_reading_back"][-1]
    assert loop.analysis.strip is None and not loop.analysis.multi_wave_ok
    assert loop.last_launch.spec.kind == "team" and loop.last_launch.spec.width <= 64


def _slice(rng, length, size):
    """Text of a slice of ``length`` elements inside an axis of ``size``, in one of NumPy's spellings."""
    lo = int(rng.integers(0, size - length + 1))
    hi = lo + length
    forms = [f"{lo}:{hi}"]
    if lo == 0:
        forms.append(f":{hi}")
    if hi == size:
        forms.append(f"{lo}:")
    if lo == 0 and hi == size:
        forms.append(":")
    if hi < size:
        forms.append(f"{lo}:{hi - size}")          # negative upper bound
    return forms[int(rng.integers(len(forms)))]


@pytest.mark.parametrize("seed", range(30))
def test_random_slice_statements_against_numpy(gpu, seed):
    """Random 1-D array statements inside a parallel loop (row slices, column
    slices, whole 1-D arrays, reductions of slice products, in-place operators),
    executed by NumPy and by the kernels."""
    import linecache

    rng = np.random.default_rng(9000 + seed)
    n, m = 23, 61
    L = int(rng.integers(1, m + 1))
    Lc = int(rng.integers(1, n + 1))
    args = {"A": rng.standard_normal((n, m)), "B": rng.standard_normal((n, m)), "C": rng.standard_normal((n, m)),
            "v": rng.standard_normal(m), "r": np.zeros(n), "alpha": 1.25}
    row_ops = [
        f"A[i, {_slice(rng, L, m)}] = B[i, {_slice(rng, L, m)}] * alpha + v[{_slice(rng, L, m)}]",
        f"A[i, {_slice(rng, L, m)}] += B[i, {_slice(rng, L, m)}] * C[i, {_slice(rng, L, m)}]",
        f"A[i, {_slice(rng, L, m)}] = np.maximum(B[i, {_slice(rng, L, m)}], 0.0) - alpha",
        f"r[i] = np.sum(B[i, {_slice(rng, L, m)}] * C[i, {_slice(rng, L, m)}]) + alpha",
        f"r[i] = B[i, {_slice(rng, L, m)}] @ v[{_slice(rng, L, m)}]",
        f"r[i] = np.max(B[i, {_slice(rng, L, m)}]) - np.min(C[i, {_slice(rng, L, m)}])",
        "A[i, :] = v * alpha - B[i, :]",
        f"s = np.sum(C[i, {_slice(rng, L, m)}])\n            A[i, {_slice(rng, L, m)}] -= s * B[i, {_slice(rng, L, m)}]",
    ]
    col_ops = [
        f"A[{_slice(rng, Lc, n)}, j] = B[{_slice(rng, Lc, n)}, j] + alpha",
        f"v[j] = B[{_slice(rng, Lc, n)}, j] @ C[{_slice(rng, Lc, n)}, j]",
        f"A[{_slice(rng, Lc, n)}, j] *= C[{_slice(rng, Lc, n)}, j]",
    ]
    pick = lambda ops, k: "\n            ".join(ops[int(x)] for x in rng.choice(len(ops), size=k, replace=False))  # noqa: E731
    src = ("def kernel(A, B, C, v, r, alpha):\n"
           "    #pragma parallel for\n    for i in range(A.shape[0]):\n            " + pick(row_ops, 2) + "\n"
           "    #pragma parallel for\n    for j in range(A.shape[1]):\n            " + pick(col_ops, 1) + "\n")
    name = f"<random_slices_{seed}>"
    linecache.cache[name] = (len(src), None, src.splitlines(True), name)
    ns = {}
    exec(compile(src, name, "exec"), {"np": np}, ns)
    ref = {k: (x.copy() if isinstance(x, np.ndarray) else x) for k, x in args.items()}
    got = {k: (x.copy() if isinstance(x, np.ndarray) else x) for k, x in args.items()}
    ns["kernel"](**ref)
    appy.jit(ns["kernel"])(**got)
    for key in ("A", "v", "r"):
        assert np.allclose(got[key], ref[key], rtol=1e-12, atol=1e-12), (key, src)


_MORE_FORMS = {
    "implicit row": "B[i] = A[i] * 2",
    "np.dot of rows": "out[i] = np.dot(A[i], x)",
    "matmul of a row": "out[i] = A[i] @ x",
    "sum method": "out[i] = A[i].sum()",
    "mean": "out[i] = np.mean(A[i, :])",
    "centre with the mean method": "B[i, :] = A[i, :] - A[i, :].mean()",
    "std and var": "out[i] = np.std(A[i, :]) + np.var(A[i, 2:])",
    "argmax and argmin": "out[i] = np.argmax(A[i, :]) - A[i].argmin()",
    "max and min methods": "out[i] = A[i, :].max() - A[i, :].min()",
    "sum of a product, as a method": "out[i] = (A[i, :] * x).sum()",
    "any": "out[i] = np.any(A[i, :] > 2.5)",
    "all": "out[i] = np.all(A[i, :] > -2.0)",
    "count_nonzero": "out[i] = np.count_nonzero(A[i, :] > 0)",
    "dot of two rows": "out[i] = np.dot(A[i, :], A[(i + 1) % A.shape[0], :])",
    "axis keyword": "out[i] = A[i, :].mean(axis=0) + np.sum(A[i], axis=-1)",
    "astype": "B[i, :] = A[i, :].astype(np.float32)",
    "zeros_like and ones_like": "B[i, :] = np.zeros_like(A[i, :]) + np.ones_like(x) * 3",
    "len of a slice": "out[i] = len(A[i, 3:]) + len(x)",
    "norm": "out[i] = np.sqrt(np.sum(A[i] ** 2))",
}


@pytest.mark.parametrize("name", sorted(_MORE_FORMS))
def test_more_numpy_spellings_of_row_expressions(gpu, name):
    """Rows without a slice (`A[i]` of a 2-D array), reductions as methods, and the NumPy
    functions that come down to sum / max / min reductions, inside `prange` loops as the
    reference's guide promises for "common NumPy array operations, slicing, and indexing"
    (docs/source/high-level.rst:48-50); each against the same loop run by NumPy."""
    import linecache

    body = _MORE_FORMS[name]
    src = f"def f(A, B, x, out):\n    for i in appy.prange(A.shape[0]):\n        {body}\n"
    fname = f"<row_forms_{name}>"
    linecache.cache[fname] = (len(src), None, src.splitlines(True), fname)
    ns = {}
    exec(compile(src, fname, "exec"), {"np": np, "appy": appy}, ns)
    rng = np.random.default_rng(5)
    A, B, x, out = rng.standard_normal((23, 61)), rng.standard_normal((23, 61)), rng.standard_normal(61), np.zeros(23)
    want = [v.copy() for v in (A, B, x, out)]
    ns["f"](*want)
    got = [A, B, x, out]
    appy.jit(ns["f"])(*got)
    for g, w in zip(got, want):
        assert np.allclose(g, w, rtol=1e-9, atol=1e-9)


def test_overlapping_row_slices_stored_by_two_statements_keep_program_order(gpu):
    """The second statement overwrites part of what the first stored, from other lanes of the
    team; with rows short enough for fully unrolled loops the order must still hold."""
    @appy.jit
    def kernel(A, B, v, alpha):
        #pragma parallel for
        for i in range(A.shape[0]):
            A[i, 18:34] = np.maximum(B[i, 24:40], 0.0) - alpha
            A[i, 12:-33] = B[i, 44:-1] * alpha + v[41:-4]

    @appy.jit
    def shifted(A, B, out):
        #pragma parallel for
        for i in range(A.shape[0]):
            A[i, :-1] = B[i, 1:] * 2.0
            out[i, 1:] = A[i, :-1] + A[i, 0]

    rng = np.random.default_rng(5173)
    for m in (61, 64, 65, 128, 257):
        A, B, v = rng.standard_normal((23, m)), rng.standard_normal((23, m)), rng.standard_normal(m)
        ref = A.copy()
        ref[:, 18:34] = np.maximum(B[:, 24:40], 0.0) - 1.25
        ref[:, 12:m - 33] = B[:, 44:m - 1] * 1.25 + v[41:m - 4]
        got = A.copy()
        kernel(got, B, v, 1.25)
        assert np.array_equal(got, ref), m
        ref, out_ref = A.copy(), np.zeros_like(A)
        ref[:, :-1] = B[:, 1:] * 2.0
        out_ref[:, 1:] = ref[:, :-1] + ref[:, :1]
        got, out = A.copy(), np.zeros_like(A)
        shifted(got, B, out)
        assert np.array_equal(got, ref) and np.array_equal(out, out_ref), m
