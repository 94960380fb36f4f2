"""Parity of the HIP path with the CPU oracle on identical seeded inputs.

Bars: bit-exact for elementwise and integer work; for float32 reductions,
GEMV, SpMV and SpMM ``|out - oracle| <= 1e-5 * sum(|terms|)`` per output, the
oracle being float64 (oracle/vectorised.py).  Every call goes through
``@jit`` -> generated HIP kernel -> libappy_hip.so (C ABI).
"""
import numpy as np
import pytest

from appy_amd.backends.hip import selfcheck
from oracle import loops as lo
from oracle import vectorised as vo
from oracle import workloads as wl

pytestmark = pytest.mark.gpu

TOL = 1e-5  # the tolerance of the parity bar, relative to sum(|terms|)


@pytest.fixture(scope="module")
def k(gpu):
    return selfcheck.kernels()


@pytest.mark.parametrize("n", [1, 3, 255, 256, 4096, 4097, 100_003, 1 << 20, (1 << 22) + 5])
def test_vec_add_bit_exact(k, n):
    a, b = wl.vec_add(n)
    c = k.vec_add(a, b)
    assert c.dtype == np.float32
    assert np.array_equal(c, vo.vec_add(a, b))


def test_vec_add_float64_and_int(k):
    rng = np.random.default_rng(7)
    a = rng.standard_normal(10_001)
    b = rng.standard_normal(10_001)
    assert np.array_equal(k.vec_add(a, b), a + b)
    ai = rng.integers(-1000, 1000, 5003, dtype=np.int32)
    bi = rng.integers(-1000, 1000, 5003, dtype=np.int32)
    assert np.array_equal(k.vec_add(ai, bi), ai + bi)


def test_vec_add_empty(k):
    a = np.empty(0, dtype=np.float32)
    assert k.vec_add(a, a).shape == (0,)


@pytest.mark.parametrize("n", [1, 7, 1000, 4096, 65_537, 1 << 20, (1 << 24) + 3])
def test_vector_sum(k, n):
    A, _ = wl.reduce_inputs(n)
    ref, budget = vo.vector_sum(A)
    got = k.vector_sum(A)
    assert isinstance(got, float)
    assert abs(got - ref) <= TOL * budget


@pytest.mark.parametrize("n", [1, 7, 1000, 4099, 1 << 20, (1 << 24) + 3])
def test_masked_sum(k, n):
    A, M = wl.reduce_inputs(n)
    ref, budget = vo.masked_sum(A, M)
    got = k.masked_sum(A, M)
    assert abs(got - ref) <= TOL * budget


def test_masked_sum_special_masks(k):
    A, _ = wl.reduce_inputs(50_001)
    assert k.masked_sum(A, np.zeros(A.shape, dtype=bool)) == 0.0
    ref, budget = vo.vector_sum(A)
    assert abs(k.masked_sum(A, np.ones(A.shape, dtype=bool)) - ref) <= TOL * budget


def test_small_cases_against_literal_loops(k):
    A, M = wl.reduce_inputs(777)
    assert abs(k.vector_sum(A) - lo.vector_sum(A)) <= TOL * float(np.abs(A).sum())
    assert abs(k.masked_sum(A, M) - lo.masked_sum_ternary(A, M)) <= TOL * float(np.abs(A).sum())
    a, b = wl.vec_add(333)
    assert np.array_equal(k.vec_add(a, b), lo.vec_add(a, b))


@pytest.mark.parametrize("shape", [(1, 1), (3, 5), (64, 64), (100, 1000), (513, 1027), (2048, 4096), (37, 16384)])
def test_gemv(k, shape):
    A, x = wl.gemv(*shape)
    ref, budget = vo.gemv(A, x)
    y = k.gemv(A, x)
    assert y.dtype == np.float32
    ok, worst = vo.within_budget(y, ref, budget, TOL)
    assert ok, worst


def test_gemv_unit_vectors_select_columns(k):
    A, _ = wl.gemv(40, 70)
    for col in (0, 33, 69):
        e = np.zeros(70, dtype=np.float32)
        e[col] = 1.0
        assert np.array_equal(k.gemv(A, e), A[:, col])


@pytest.mark.parametrize("m,per_row", [(1, 1), (10, 3), (1000, 16), (4096, 16), (50_000, 16), (3000, 100)])
def test_spmv_uniform(k, m, per_row):
    data, indptr, indices, x = wl.spmv_uniform(m, max(m, per_row * 2), per_row)
    n = x.shape[0]
    ref, budget = vo.spmv_csr(data, indptr, indices, x, (m, n))
    y = k.spmv(data, indptr, indices, x, m, n)
    ok, worst = vo.within_budget(y, ref, budget, TOL)
    assert ok, worst


@pytest.mark.parametrize("m,clip", [(2000, 64), (8192, 512), (20_000, 4096)])
def test_spmv_powerlaw(k, m, clip):
    data, indptr, indices, x = wl.spmv_powerlaw(m, m, clip=clip)
    ref, budget = vo.spmv_csr(data, indptr, indices, x, (m, m))
    y = k.spmv(data, indptr, indices, x, m, m)
    ok, worst = vo.within_budget(y, ref, budget, TOL)
    assert ok, worst


def test_spmv_empty_rows_and_identity(k):
    # rows 0 and 2 empty
    indptr = np.array([0, 0, 2, 2, 3], dtype=np.int32)
    indices = np.array([1, 3, 0], dtype=np.int32)
    data = np.array([2.0, -1.0, 0.5], dtype=np.float32)
    x = np.array([4.0, 3.0, 2.0, 1.0], dtype=np.float32)
    y = k.spmv(data, indptr, indices, x, 4, 4)
    assert np.array_equal(y, np.array([0.0, 5.0, 0.0, 2.0], dtype=np.float32))
    n = 1000
    eye_ptr = np.arange(n + 1, dtype=np.int32)
    eye_idx = np.arange(n, dtype=np.int32)
    xs = np.random.default_rng(3).standard_normal(n, dtype=np.float32)
    assert np.array_equal(k.spmv(np.ones(n, dtype=np.float32), eye_ptr, eye_idx, xs, n, n), xs)


def test_spmv_int64_indices(k):
    data, indptr, indices, x = wl.spmv_uniform(3000, 3000, 9)
    ref, budget = vo.spmv_csr(data, indptr, indices, x, (3000, 3000))
    y = k.spmv(data, indptr.astype(np.int64), indices.astype(np.int64), x, 3000, 3000)
    assert vo.within_budget(y, ref, budget, TOL)[0]


@pytest.mark.parametrize("m,ncols", [(1, 128), (100, 128), (4096, 128), (1000, 200), (500, 7)])
def test_spmm(k, m, ncols):
    data, indptr, indices, B = wl.spmm(m, max(m, 64), ncols)
    n = B.shape[0]
    ref, budget = vo.spmm_csr(data, indptr, indices, B, (m, n))
    Y = np.full((m, ncols), np.nan, dtype=np.float32)
    k.spmm(data, indptr, indices, B, Y, m)
    ok, worst = vo.within_budget(Y, ref, budget, TOL)
    assert ok, worst


def test_spmm_columns_equal_spmv(k):
    data, indptr, indices, B = wl.spmm(700, 700, 128)
    Y = np.empty((700, 128), dtype=np.float32)
    k.spmm(data, indptr, indices, B, Y, 700)
    for col in (0, 64, 127):
        x = np.ascontiguousarray(B[:, col])
        ref, budget = vo.spmv_csr(data, indptr, indices, x, (700, 700))
        assert vo.within_budget(Y[:, col], ref, budget, TOL)[0]


@pytest.mark.parametrize("shape", [(3, 5), (513, 1027), (300, 9000)])
def test_gemv_with_x_staged_in_lds(gpu, shape):
    """The LDS-tiled schedule (row-invariant operand staged per workgroup) is an
    option of the generator; it must give the same results as the default."""
    import appy_amd as appy

    @appy.jit(hip_spec={"lds_tile": 2048, "width": 32})
    def gemv_lds(A, x, y):
        #pragma parallel for
        for i in range(A.shape[0]):
            yi = 0.0
            #pragma simd
            for j in range(A.shape[1]):
                yi += A[i, j] * x[j]
            y[i] = yi

    A, x = wl.gemv(*shape)
    y = np.full(shape[0], np.nan, dtype=np.float32)
    gemv_lds(A, x, y)
    ref, budget = vo.gemv(A, x)
    ok, worst = vo.within_budget(y, ref, budget, TOL)
    assert ok, worst
    from appy_amd.backends.hip import codegen as cg

    loop = [v[0] for kk, v in cg.code_cache.items() if kk[-1] == "gemv_lds"][-1]
    assert "__tile_x" in loop.last_launch.kernel.src.text


def test_aliased_arguments_and_strided_numpy_views(gpu):
    import appy_amd as appy

    @appy.jit
    def add_into(a, b, c):
        #pragma parallel for simd
        for i in range(a.shape[0]):
            c[i] = a[i] + b[i]

    a = np.arange(10_001, dtype=np.float32)
    add_into(a, a, a)                       # all three names are one buffer: the no-restrict variant
    assert np.array_equal(a, 2 * np.arange(10_001, dtype=np.float32))
    base = np.zeros((5000, 3), dtype=np.float32)
    ones = np.ones(5000, dtype=np.float32)
    add_into(ones, ones, base[:, 1])        # strided output view: packed copy in, copy back out
    assert np.array_equal(base[:, 1], 2 * ones) and base.sum() == 10_000
    add_into(base[:, 1], ones, base[:, 2])  # strided input view
    assert np.array_equal(base[:, 2], 3 * ones)


def test_integer_reductions_and_products(gpu):
    import appy_amd as appy

    @appy.jit
    def count_and_max(a):
        n = 0
        m = -2**62
        #pragma parallel for simd shared(n, m)
        for i in range(a.shape[0]):
            n += 1 if a[i] > 0 else 0
            m = max(m, a[i])
        return n, m

    @appy.jit
    def product(a):
        p = 1.0
        #pragma parallel for simd shared(p)
        for i in range(a.shape[0]):
            p *= a[i]
        return p

    a = np.random.default_rng(9).integers(-1000, 1000, 100_003, dtype=np.int64)
    n, m = count_and_max(a)
    assert (n, m) == (int((a > 0).sum()), int(a.max())) and isinstance(n, int)
    b = np.random.default_rng(10).uniform(0.999, 1.001, 50_000)
    assert product(b) == pytest.approx(float(np.prod(b)), rel=1e-9)


def test_repeated_calls_reuse_pooled_buffers(gpu):
    from appy_amd.backends.hip import runtime as rt
    import ctypes

    k0 = selfcheck.kernels()
    a, b = wl.vec_add(300_000)
    k0.vec_add(a, b)
    used, cached = ctypes.c_uint64(), ctypes.c_uint64()
    rt.check(rt.lib().appy_hip_pool_stats(ctypes.byref(used), ctypes.byref(cached)))
    first, held = cached.value, used.value      # (held: scratch buffers that loops of earlier tests keep)
    for _ in range(5):
        assert np.array_equal(k0.vec_add(a, b), a + b)
    rt.check(rt.lib().appy_hip_pool_stats(ctypes.byref(used), ctypes.byref(cached)))
    assert used.value == held and cached.value == first       # nothing leaked, nothing newly allocated


@pytest.mark.parametrize("n", [1, 1000, 4099, (1 << 22) + 7])
def test_masked_sum_with_control_flow(gpu, n):
    """The `if mask[i]: b += a[i]` form of examples/04-masked_sum.py:7-14 (no simd clause)."""
    import appy_amd as appy

    @appy.jit
    def masked_sum_if(a, mask):
        b = 0.0
        #pragma parallel for shared(b)
        for i in range(a.shape[0]):
            if mask[i]:
                b += a[i]
        return b

    A, M = wl.reduce_inputs(n)
    ref, budget = vo.masked_sum(A, M)
    assert abs(masked_sum_if(A, M) - ref) <= TOL * budget


@pytest.mark.parametrize("shape", [(1, 300_000), (3, 1 << 20), (100, 70_001), (2000, 9000)])
def test_gemv_few_long_rows(k, shape):
    """Few, very long rows: one workgroup per row with the LDS team reduction."""
    A, x = wl.gemv(*shape)
    ref, budget = vo.gemv(A, x)
    y = k.gemv(A, x)
    ok, worst = vo.within_budget(y, ref, budget, TOL)
    assert ok, worst


def test_spmv_few_very_long_rows(k):
    """A handful of rows with tens of thousands of non-zeros: workgroup teams on CSR rows."""
    rng = np.random.default_rng(11)
    m, n = 37, 400_000
    lengths = rng.integers(20_000, 60_000, m)
    lengths[5] = 0
    data, indptr, indices = wl.csr_matrix(lengths, n, rng)
    x = rng.standard_normal(n, dtype=np.float32)
    ref, budget = vo.spmv_csr(data, indptr, indices, x, (m, n))
    y = k.spmv(data, indptr, indices, x, m, n)
    ok, worst = vo.within_budget(y, ref, budget, TOL)
    assert ok, worst


def test_launches_from_several_threads(k):
    """Four interpreter threads launch different loops on their own arrays at once:
    the library's allocator, staging lanes and code caches are shared between them."""
    import threading

    rng = np.random.default_rng(13)
    errors = []

    def work(seed):
        try:
            r = np.random.default_rng(seed)
            for rep in range(6):
                n = int(r.integers(1000, 3_000_000))
                a = r.standard_normal(n, dtype=np.float32)
                b = r.standard_normal(n, dtype=np.float32)
                if not np.array_equal(k.vec_add(a, b), a + b):
                    errors.append((seed, rep, "vec_add"))
                ref, budget = vo.vector_sum(a)
                if abs(k.vector_sum(a) - ref) > TOL * budget:
                    errors.append((seed, rep, "vector_sum"))
                A = r.standard_normal((257, 300), dtype=np.float32)
                x = r.standard_normal(300, dtype=np.float32)
                gref, gb = vo.gemv(A, x)
                ok, worst = vo.within_budget(k.gemv(A, x), gref, gb, TOL)
                if not ok:
                    errors.append((seed, rep, "gemv", worst))
        except Exception as e:          # a failure in a thread must fail the test
            errors.append((seed, repr(e)))

    threads = [threading.Thread(target=work, args=(int(s),)) for s in rng.integers(0, 1 << 30, 4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors


_FLAT_SPECS = [dict(block=b, vec=v, unroll=u, stream_loads=nt, stream_stores=nt)
               for b, v, u, nt in ((64, 1, 1, False), (256, 2, 4, False), (1024, 4, 2, True), (512, 1, 8, False), (128, 4, 1, True))]
_TEAM_SPECS = [dict(block=b, vec=v, width=w, stream_loads=nt)
               for b, v, w, nt in ((256, 1, 1, False), (256, 4, 2, False), (64, 2, 64, True), (512, 4, 16, False),
                                   (1024, 1, 1024, False), (256, 4, 256, True), (128, 2, 8, False))]


@pytest.mark.parametrize("spec", _FLAT_SPECS, ids=lambda s: "b{block}v{vec}u{unroll}".format(**s))
def test_flat_kernels_give_the_same_results_in_every_launch_shape(gpu, spec):
    k = selfcheck.kernels(hip_spec=spec)
    a, b = wl.vec_add(70_001)
    assert np.array_equal(k.vec_add(a, b), vo.vec_add(a, b))
    A, M = wl.reduce_inputs(333_337)
    ref, budget = vo.vector_sum(A)
    assert abs(k.vector_sum(A) - ref) <= TOL * budget
    ref, budget = vo.masked_sum(A, M)
    assert abs(k.masked_sum(A, M) - ref) <= TOL * budget
    c = np.empty_like(a)
    k.copy(a, c)
    assert np.array_equal(a, c)


@pytest.mark.parametrize("spec", _TEAM_SPECS, ids=lambda s: "b{block}v{vec}w{width}".format(**s))
def test_team_kernels_give_the_same_results_in_every_launch_shape(gpu, spec):
    k = selfcheck.kernels(hip_spec=spec)
    Am, x = wl.gemv(301, 1237)
    ref, budget = vo.gemv(Am, x)
    ok, worst = vo.within_budget(k.gemv(Am, x), ref, budget, TOL)
    assert ok, worst
    data, indptr, indices, xs = wl.spmv_powerlaw(3000, 3000, clip=700)
    ref, budget = vo.spmv_csr(data, indptr, indices, xs, (3000, 3000))
    ok, worst = vo.within_budget(k.spmv(data, indptr, indices, xs, 3000, 3000), ref, budget, TOL)
    assert ok, worst
    data, indptr, indices, B = wl.spmm(500, 400, 128)
    ref, budget = vo.spmm_csr(data, indptr, indices, B, (500, 400))
    Y = np.empty((500, 128), dtype=np.float32)
    k.spmm(data, indptr, indices, B, Y, 500)
    ok, worst = vo.within_budget(Y, ref, budget, TOL)
    assert ok, worst


@pytest.mark.parametrize("block,unroll", [(64, 1), (128, 4), (256, 8), (512, 2), (1024, 8)])
def test_strip_kernel_gives_the_same_results_for_every_workgroup_size(gpu, block, unroll):
    k = selfcheck.kernels(hip_spec=dict(kind="strip", block=block, vec=1, unroll=unroll, stream_loads=block == 256))
    Am, _ = wl.gemv(777, 333)
    yv = Am[:, 1].copy()
    ref, budget = vo.gemv(Am.T, yv)
    ok, worst = vo.within_budget(k.gemv_columns(Am, yv), ref, budget, TOL)
    assert ok, worst


def test_arrays_that_a_launch_overwrites_completely_are_not_uploaded(gpu, monkeypatch):
    """``c[i] = ...`` over the whole of ``c``: its old contents stay on the host.
    As soon as the range leaves elements out, or the loop reads the array, it
    is uploaded as before (the untouched elements must survive)."""
    import appy_amd as appy
    from appy_amd.backends.hip import runtime as rt

    uploads = []
    real = rt.memcpy_h2d
    monkeypatch.setattr(rt, "memcpy_h2d", lambda dst, src, n, stream=0: (uploads.append(n), real(dst, src, n, stream))[1])

    @appy.jit
    def fill(a, c, start):
        #pragma parallel for simd
        for i in range(start, a.shape[0]):
            c[i] = a[i] * 2.0

    @appy.jit
    def rows(A, C):
        #pragma parallel for
        for i in range(A.shape[0]):
            C[i, :] = A[i, :] + 1.0

    a = np.arange(5000.0)
    c = np.full(5000, -1.0)
    fill(a, c, 0)
    assert np.array_equal(c, 2.0 * a) and uploads == [a.nbytes]            # only `a` travelled up
    uploads.clear()
    c[:] = -1.0
    fill(a, c, 3)
    assert np.array_equal(c[3:], 2.0 * a[3:]) and (c[:3] == -1.0).all() and uploads == [a.nbytes, c.nbytes]
    uploads.clear()
    A = np.arange(600.0).reshape(20, 30)
    C = np.full((20, 30), -1.0)
    rows(A, C)
    assert np.array_equal(C, A + 1.0) and uploads == [A.nbytes]
    uploads.clear()
    rows(A[:, :20], C[:, :20])                                             # packed copies of views: same rule
    assert np.array_equal(C[:, :20], A[:, :20] + 1.0) and len(uploads) == 1
