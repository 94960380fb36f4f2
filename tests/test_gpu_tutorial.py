"""The reference's GPU integration tests for the loop patterns, run through
``import appy`` exactly as written there (tests/integration/triton/tutorial/:
test_vec_add.py:4-19, test_global_reduction.py:4-44, test_rowwise_reduction.py:4-53,
test_mat_add.py:5-20, test_spmv.py:10-30, test_pi.py:8-26, test_var_write.py:12-23;
npbench/test_gesummv.py:26-55 for array expressions), plus in-place use of GPU
tensors.  ``backend="triton"`` in those files selects "the GPU back end"."""
import math
import warnings

import numpy as np
import pytest
import scipy.sparse as sp

import appy

pytestmark = pytest.mark.gpu
warnings.filterwarnings("ignore", message="backend='triton'")


@appy.jit(backend="triton")
def t_vec_add(a, b):
    c = np.empty_like(a)
    #pragma parallel for simd
    for i in range(a.shape[0]):
        c[i] = a[i] + b[i]
    return c


@appy.jit(backend="triton", dry_run=0)
def t_vec_sum(a):
    sum = 0.0
    #pragma parallel for simd shared(sum)
    for i in range(a.shape[0]):
        sum += a[i]
    return sum


@appy.jit(backend="triton", dry_run=0)
def t_vec_max(a):
    m = -np.inf
    #pragma parallel for simd shared(m)
    for i in range(a.shape[0]):
        m = max(m, a[i])
    return m


@appy.jit(backend="triton", dry_run=0)
def t_vec_min(a):
    m = np.inf
    #pragma parallel for simd shared(m)
    for i in range(a.shape[0]):
        m = min(m, a[i])
    return m


@appy.jit(backend="triton")
def t_rowwise_sum(a, b):
    #pragma parallel for
    for i in range(a.shape[0]):
        #pragma simd
        s = 0.0
        for j in range(a.shape[1]):
            s += a[i, j]
        b[i] = s


@appy.jit(backend="triton")
def t_rowwise_max(a, b):
    #pragma parallel for
    for i in range(a.shape[0]):

        s = -1e308
        #pragma simd
        for j in range(a.shape[1]):
            s = max(s, a[i, j])
        b[i] = s


@appy.jit(backend="triton")
def t_rowwise_min(a, b):
    #pragma parallel for
    for i in range(a.shape[0]):

        s = 1e308
        #pragma simd
        for j in range(a.shape[1]):
            s = min(s, a[i, j])
        b[i] = s


@appy.jit(backend="triton")
def t_mat_add(a, b):
    c = np.empty_like(a)
    #pragma parallel for
    for i in range(a.shape[0]):
        #pragma simd
        for j in range(a.shape[1]):
            c[i, j] = a[i, j] + b[i, j]
    return c


@appy.jit(backend="triton")
def t_spmv(A_data, A_indptr, A_indices, x, M, N):
    y = np.empty(M, dtype=x.dtype)
    #pragma parallel for
    for i in range(M):
        start, end = A_indptr[i], A_indptr[i+1]
        s = 0.0
        #pragma simd
        for j in range(start, end):
            s += A_data[j] * x[A_indices[j]]
        y[i] = s
    return y


@appy.jit
def t_pi(num_steps, step):
    sum = 0.0
    #pragma parallel for simd shared(sum,step)
    for i in range(1, num_steps + 1):
        x = (i - 0.5) * step
        sum += 4.0 / (1.0 + x * x)
    return step * sum


@appy.jit
def t_var_write():
    a = 0
    #pragma parallel for shared(a)
    for i in range(10):
        if i == 3:
            a = 1
    return a


@appy.jit(backend="triton")
def t_gesummv(alpha, beta, A, B, x):
    y = np.empty((A.shape[0], ), dtype=x.dtype)
    #pragma parallel for
    for i in range(A.shape[0]):
        s = 0.0
        #pragma simd
        for j in range(A.shape[1]):
            s += alpha * A[i, j] * x[j] + beta * B[i, j] * x[j]
        y[i] = s
    return y


@appy.jit(backend="triton")
def t_gesummv1(alpha, beta, A, B, x):
    y = np.empty((A.shape[0], ), dtype=x.dtype)
    #pragma parallel for
    for i in range(A.shape[0]):
        y[i] = np.sum(alpha * A[i, :] * x[:] + beta * B[i, :] * x[:])
    return y


def test_vec_add(gpu):
    a = np.ones(100)
    b = np.ones(100)
    assert np.allclose(t_vec_add(a, b), a + b)


def test_global_reductions(gpu):
    a = np.random.default_rng(0).random(1000)
    assert np.allclose(t_vec_sum(a), a.sum())
    assert np.allclose(t_vec_max(a), a.max())
    assert np.allclose(t_vec_min(a), a.min())
    big = np.random.default_rng(1).standard_normal(1_000_003)
    assert t_vec_max(big) == big.max() and t_vec_min(big) == big.min()


def test_rowwise_reductions(gpu):
    a = np.random.default_rng(2).random((100, 100))
    b = np.empty(100)
    t_rowwise_sum(a, b)
    assert np.allclose(b, a.sum(axis=1))
    t_rowwise_max(a, b)
    assert np.allclose(b, a.max(axis=1))
    t_rowwise_min(a, b)
    assert np.allclose(b, a.min(axis=1))


def test_mat_add(gpu):
    a = np.ones((100, 100))
    b = np.ones((100, 100))
    assert np.allclose(t_mat_add(a, b), a + b)
    r = np.random.default_rng(3).standard_normal((37, 211)).astype(np.float32)
    assert np.array_equal(t_mat_add(r, r), r + r)


def test_spmv_csr(gpu):
    N = 1000
    A = sp.random(N, N, density=0.01, format="csr", random_state=4)
    x = np.random.default_rng(5).random(N)
    y = t_spmv(A.data, A.indptr, A.indices, x, N, N)
    assert np.allclose(y, A @ x, atol=1e-6)


def test_pi(gpu):
    num_steps = 1_000_000
    step = 1.0 / num_steps
    assert np.isclose(t_pi(num_steps, step), np.pi, rtol=1e-06, atol=1e-08)


def test_var_write(gpu):
    assert t_var_write() == 1


def test_gesummv_loops_and_array_expressions(gpu):
    N = 100
    alpha, beta = 1.5, 1.2
    A = np.fromfunction(lambda i, j: ((i * j + 1) % N) / N, (N, N), dtype=np.float64)
    B = np.fromfunction(lambda i, j: ((i * j + 2) % N) / N, (N, N), dtype=np.float64)
    x = np.fromfunction(lambda i: (i % N) / N, (N,), dtype=np.float64)
    ref = alpha * A @ x + beta * B @ x
    assert np.allclose(ref, t_gesummv(alpha, beta, A, B, x))
    assert np.allclose(ref, t_gesummv1(alpha, beta, A, B, x))


def test_gpu_tensors_are_used_in_place(gpu):
    import torch

    a = torch.arange(10_000, dtype=torch.float32, device="cuda")
    b = torch.ones(10_000, dtype=torch.float32, device="cuda")

    @appy.jit
    def add_into(a, b, c):
        #pragma parallel for simd
        for i in range(a.shape[0]):
            c[i] = a[i] + b[i]

    c = torch.empty_like(a)
    ptr = c.data_ptr()
    add_into(a, b, c)
    assert c.data_ptr() == ptr and torch.equal(c, a + b)
    # a CPU tensor is copied in and out like a NumPy array
    ac, bc, cc = a.cpu(), b.cpu(), torch.zeros(10_000)
    add_into(ac, bc, cc)
    assert torch.equal(cc, ac + bc)
    # a strided view (last dimension not contiguous) goes through a packed copy
    base = torch.zeros((100, 8), device="cuda")
    col = base[:, 3]
    ones = torch.ones(100, device="cuda")
    add_into(ones, ones, col)
    assert torch.equal(base[:, 3], 2 * ones) and float(base.sum()) == 200.0


def test_launches_follow_the_current_torch_stream(gpu):
    import torch

    @appy.jit
    def scale_add(a, b, f):
        #pragma parallel for simd
        for i in range(a.shape[0]):
            b[i] = a[i] * f + b[i]

    side = torch.cuda.Stream()                      # default priority
    n = 1 << 22
    with torch.cuda.stream(side):
        a = torch.full((n,), 2.0, device="cuda")    # produced on the side stream
        b = torch.ones(n, device="cuda")
        for _ in range(5):
            scale_add(a, b, 0.5)                    # each launch depends on the previous one through b
        total = b.sum()                             # consumed on the same stream, no synchronisation in between
    side.synchronize()
    assert float(total) == n * 6.0


def test_to_gpu_and_to_cpu_helpers(gpu):
    import torch

    a = np.arange(6, dtype=np.float32)
    t, u = appy.to_gpu(a, [1, 2, 3])
    assert t.device.type == "cuda" and u.device.type == "cuda" and appy.to_gpu(3.5) == 3.5
    assert np.array_equal(appy.to_cpu(t), a)
    assert appy.to_cpu(torch.tensor(7.0, device="cuda")) == 7.0


def test_prange_examples_of_the_getting_started_guide(gpu):
    """docs/source/getting_started.rst:38-66: ``prange`` instead of ``range``,
    reductions of scalars detected without a pragma."""
    from appy import jit, prange

    @jit
    def add_one(a):
        for i in prange(a.shape[0]):
            a[i] += 1

    @jit
    def sum_vector(a, N):
        sum = 0
        for i in prange(N):
            sum += a[i]
        return sum

    @jit
    def stats(a):
        lo = float("inf")
        n_pos = 0
        for i in prange(a.shape[0]):
            lo = min(lo, a[i])
            n_pos += 1 if a[i] > 0 else 0
        return lo, n_pos

    a = np.zeros(10)
    add_one(a)
    assert np.array_equal(a, np.ones(10))
    assert sum_vector(np.ones(10), 10) == 10
    x = np.random.default_rng(4).standard_normal(300_001)
    s = sum_vector(x, x.shape[0])
    assert abs(s - math.fsum(x)) <= 1e-9 * np.abs(x).sum()
    lo, n_pos = stats(x)
    assert lo == x.min() and n_pos == int((x > 0).sum()) and type(n_pos) is int


def test_prange_only_programs_vectorise_their_inner_loops(gpu):
    """High-level interface: no pragmas at all; the inner loops are spread over
    lanes by the compiler (docs/source/developer.rst, "Inner Loop
    Vectorization").  Results against NumPy / SciPy on the same inputs."""
    from appy import jit, prange
    from appy_amd.backends.hip import codegen as cg

    @jit
    def hl_gemv(A, x, y, alpha):
        for i in prange(A.shape[0]):
            for j in range(A.shape[1]):
                y[i] += alpha * A[i, j] * x[j]

    @jit
    def hl_spmv(data, indptr, indices, x, y):
        for i in prange(y.shape[0]):
            s = 0.0
            for j in range(indptr[i], indptr[i + 1]):
                s += data[j] * x[indices[j]]
            y[i] = s

    @jit
    def hl_spmm(data, indptr, indices, B, C):
        for i in prange(C.shape[0]):
            for k in range(indptr[i], indptr[i + 1]):
                for c in range(C.shape[1]):
                    C[i, c] += data[k] * B[indices[k], c]

    @jit
    def hl_mat_add(X, Z, Y):
        for i in prange(X.shape[0]):
            for j in range(X.shape[1]):
                t = X[i, j] + Z[i, j]
                Y[i, j] = t

    @jit
    def hl_colsum(A, y):
        for i in prange(A.shape[1]):
            s = 0.0
            for j in range(A.shape[0]):
                s += A[j, i]
            y[i] = s

    rng = np.random.default_rng(12)
    A = rng.standard_normal((300, 517))
    x = rng.standard_normal(517)
    y0 = rng.standard_normal(300)
    y = y0.copy()
    hl_gemv(A, x, y, 1.5)
    assert np.allclose(y, y0 + 1.5 * (A @ x), rtol=1e-12, atol=1e-12)

    M = sp.random(400, 350, density=0.05, format="csr", random_state=3)
    xv = rng.standard_normal(350)
    ys = np.zeros(400)
    hl_spmv(M.data, M.indptr, M.indices, xv, ys)
    assert np.allclose(ys, M @ xv, rtol=1e-12, atol=1e-12)
    B = rng.standard_normal((350, 64))
    C = np.zeros((400, 64))
    hl_spmm(M.data, M.indptr, M.indices, B, C)
    assert np.allclose(C, M @ B, rtol=1e-12, atol=1e-12)

    X, Z = rng.standard_normal((130, 257)), rng.standard_normal((130, 257))
    Y = np.zeros_like(X)
    hl_mat_add(X, Z, Y)
    assert np.array_equal(Y, X + Z)
    cs = np.zeros(517)
    hl_colsum(A, cs)
    assert np.allclose(cs, A.sum(axis=0), rtol=1e-12, atol=1e-12)

    kinds = {key[-1]: loop.analysis.kind for key, (loop, _) in cg.code_cache.items() if str(key[-1]).startswith("hl_")}
    assert kinds == {"hl_gemv": "team", "hl_spmv": "team", "hl_spmm": "team", "hl_mat_add": "team", "hl_colsum": "flat"}


def test_replayed_call_with_an_out_of_range_subscript_offset_is_refused_on_the_host(gpu):
    """The offset of an affine subscript is checked on the host for every value it takes: the
    second call, which would otherwise only repeat the launch, raises before anything runs."""
    import torch

    from appy_amd.backends.hip import codegen as cg

    @appy.jit
    def strided_pick(a, b, off):
        #pragma parallel for simd
        for i in range(b.shape[0]):
            b[i] = a[2 * i + off]

    a = torch.arange(64, dtype=torch.float32, device="cuda")
    b = torch.zeros(8, dtype=torch.float32, device="cuda")
    strided_pick(a, b, 1)
    assert torch.equal(b, a[1:17:2])
    loop = [v[0] for kk, v in cg.code_cache.items() if kk[-1] == "strided_pick"][-1]
    first = loop.last_launch
    strided_pick(a, b, 1)
    assert loop.last_launch is first                          # an exact repeat is replayed
    strided_pick(a, b, 3)                                     # another offset: staged (and checked) again
    assert loop.last_launch is not first and torch.equal(b, a[3:19:2])
    before = b.clone()
    with pytest.raises(IndexError):
        strided_pick(a, b, 60)                                # 2 * 7 + 60 = 74 is past the end of `a`
    with pytest.raises(IndexError):
        strided_pick(a, b, -1)
    torch.cuda.synchronize()
    assert torch.equal(b, before)                             # nothing was launched


def test_repeated_calls_on_gpu_tensors_replay_the_staged_launch(gpu):
    """A call with the same tensors, scalars and stream as before repeats only the
    launch; anything that differs goes through staging again."""
    import torch

    from appy_amd.backends.hip import codegen as cg

    @appy.jit
    def scaled_add(a, b, c, f):
        #pragma parallel for simd
        for i in range(a.shape[0]):
            c[i] = a[i] * f + b[i]

    a = torch.arange(1000, dtype=torch.float64, device="cuda")
    b = torch.ones(1000, dtype=torch.float64, device="cuda")
    c = torch.zeros(1000, dtype=torch.float64, device="cuda")
    scaled_add(a, b, c, 2.0)
    loop = [v[0] for kk, v in cg.code_cache.items() if kk[-1] == "scaled_add"][-1]
    first = loop.last_launch
    a.mul_(3.0)
    scaled_add(a, b, c, 2.0)
    assert loop.last_launch is first                          # replayed ...
    assert torch.equal(c, a * 2.0 + b)                        # ... on the tensors' current contents
    scaled_add(a, b, c, 5.0)                                  # a scalar that only the kernel looks at: patched in
    assert loop.last_launch is first and torch.equal(c, a * 5.0 + b)
    scaled_add(a, b, c, 2)                                    # another type of scalar: another kernel altogether
    assert torch.equal(c, a * 2 + b)

    @appy.jit
    def fill_from(c, start, v):
        #pragma parallel for simd
        for i in range(start, c.shape[0]):
            c[i] = v

    fill_from(c, 10, 1.0)
    fl = [v[0] for kk, v in cg.code_cache.items() if kk[-1] == "fill_from"][-1]
    plan = fl.last_launch
    fill_from(c, 10, 3.0)                                     # `v` travels with the replay ...
    assert fl.last_launch is plan and bool((c[10:] == 3.0).all())
    fill_from(c, 500, 4.0)                                    # ... `start` steers the range: staged again
    assert fl.last_launch is not plan and bool((c[10:500] == 3.0).all()) and bool((c[500:] == 4.0).all())
    c2 = torch.zeros(500, dtype=torch.float64, device="cuda")
    scaled_add(a[:500], b[:500], c2, 2.0)                     # other shapes
    assert torch.equal(c2, a[:500] * 2.0 + b[:500])
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        scaled_add(a, b, c, 2.0)                              # another stream
        assert loop.last_launch.stream == side.cuda_stream
    side.synchronize()
    assert torch.equal(c, a * 2.0 + b)
    with pytest.raises(IndexError):
        scaled_add(a, b[:10], c, 2.0)                         # host checks still run for new shapes


_INNER_STATEMENTS = [
    "t = A[i, j] * 2.0\n            B[i, j] = t + x[j]",
    "B[i, j] = B[i, j - 1] + A[i, j]",                       # carried through B
    "s += A[i, j] * x[j]",
    "s = s * 0.5 + A[i, j]",                                 # carried scalar, not a reduction
    "y[i] += A[i, j]",
    "y[i] = max(y[i], A[i, j])",
    "B[i, p[j]] = A[i, j]",                                  # scatter through a permutation
    "if A[i, j] > 0.0:\n                s += A[i, j]",
    "c[j] += A[i, j]",                                       # every outer iteration feeds c[j]
    "B[i, j] = A[i, j] + s",                                 # reads the running value of s
    "t = A[i, j]\n            B[i, j] = t * t\n            s += t",
    "B[i, j] = x[p[j]] * A[i, j]",                           # gather
    "u = x[j]\n            B[i, j] = u",
]


@pytest.mark.parametrize("seed", range(40))
def test_random_prange_nests_agree_with_the_interpreter(gpu, seed):
    """Random inner loops under ``prange`` (independent ones, carried ones,
    reductions, scatters, gathers): whatever the compiler decides to spread over
    lanes, the result must be the interpreter's."""
    import linecache

    rng = np.random.default_rng(7000 + seed)
    n, m = 19, 83
    k = int(rng.integers(1, 4))
    body = "\n            ".join(_INNER_STATEMENTS[int(x)] for x in rng.choice(len(_INNER_STATEMENTS), size=k, replace=False))
    lo = int(rng.integers(0, 2))
    src = ("def kernel(A, B, x, y, c, p, out):\n    for i in prange(A.shape[0]):\n        s = 0.0\n        t = 0.0\n        u = 0.0\n"
           f"        for j in range({lo if 'j - 1' not in body else 1}, A.shape[1]):\n            {body}\n"
           "        out[i] = s + t + u\n")
    name = f"<random_prange_{seed}>"
    linecache.cache[name] = (len(src), None, src.splitlines(True), name)
    ns = {}
    exec(compile(src, name, "exec"), {"np": np, "prange": appy.prange}, ns)
    base = {"A": rng.standard_normal((n, m)), "B": rng.standard_normal((n, m)), "x": rng.standard_normal(m),
            "y": rng.standard_normal(n), "c": np.zeros(m), "p": rng.permutation(m).astype(np.int32), "out": np.zeros(n)}
    ref = {key: v.copy() for key, v in base.items()}
    got = {key: v.copy() for key, v in base.items()}
    ns["kernel"](**ref)
    appy.jit(ns["kernel"])(**got)
    for key in ("B", "y", "c", "out"):
        assert np.allclose(got[key], ref[key], rtol=1e-10, atol=1e-10), (key, src)


@appy.jit
def nested_pranges(A, B):
    for i in appy.prange(A.shape[0]):
        for j in appy.prange(A.shape[1]):
            B[i, j] = A[i, j] * 2 + i


def test_prange_inside_prange_is_a_range_loop_of_the_kernel(gpu):
    A = np.random.default_rng(3).standard_normal((41, 300))
    B = np.zeros_like(A)
    nested_pranges(A, B)
    assert np.array_equal(B, A * 2 + np.arange(41)[:, None])
    assert "for j in range(A_shape_1)" in nested_pranges.__appy_source__
    assert "#pragma simd" in nested_pranges.__appy_source__        # and the vectoriser sees it
