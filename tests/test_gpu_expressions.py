"""Expression semantics of generated kernels against NumPy, element by element:
integer division and modulo with negative operands (Python/NumPy floor
semantics, not C truncation), powers, comparisons, boolean operators, dtype
promotion with Python scalars, small integer and half-precision arrays,
boolean outputs, gathers with computed indices, maths functions."""
import math

import numpy as np
import pytest

import appy

pytestmark = pytest.mark.gpu
N = 10_007


@pytest.fixture(scope="module")
def rng(gpu):
    return np.random.default_rng(123)


@appy.jit
def int_ops(a, b, q, r, p, s):
    #pragma parallel for simd
    for i in range(a.shape[0]):
        q[i] = a[i] // b[i]
        r[i] = a[i] % b[i]
        p[i] = a[i] ** 2 + abs(b[i])
        s[i] = (a[i] << 2) ^ (b[i] & 7) | (a[i] >> 1)


def test_integer_floor_division_modulo_shifts(rng):
    a = rng.integers(-1000, 1000, N, dtype=np.int32)
    b = rng.integers(1, 50, N, dtype=np.int32) * rng.choice([-1, 1], N).astype(np.int32)
    q, r, p, s = (np.empty_like(a) for _ in range(4))
    int_ops(a, b, q, r, p, s)
    assert np.array_equal(q, a // b) and np.array_equal(r, a % b)
    assert np.array_equal(p, a ** 2 + np.abs(b))
    assert np.array_equal(s, (a << 2) ^ (b & 7) | (a >> 1))


@appy.jit
def float_ops(a, b, out_mod, out_fdiv, out_pow, out_cmp, out_sel):
    #pragma parallel for simd
    for i in range(a.shape[0]):
        out_mod[i] = a[i] % b[i]
        out_fdiv[i] = a[i] // b[i]
        out_pow[i] = a[i] ** 3 - b[i] ** 2
        out_cmp[i] = (0.0 < a[i] < 0.5) or (not b[i] > 0.0 and a[i] <= -0.5)
        out_sel[i] = max(a[i], b[i], 0.25) - min(a[i], b[i])


def test_float_modulo_floor_division_power_comparisons(rng):
    a = rng.uniform(-1, 1, N).astype(np.float32)
    b = rng.uniform(0.1, 1, N).astype(np.float32) * rng.choice([-1, 1], N).astype(np.float32)
    m, f, p, s = (np.empty_like(a) for _ in range(4))
    c = np.empty(N, dtype=bool)
    float_ops(a, b, m, f, p, c, s)
    assert np.allclose(m, np.mod(a, b), rtol=0, atol=1e-6)
    assert np.array_equal(f, np.floor_divide(a, b))
    assert p.dtype == np.float32 and np.allclose(p, a ** 3 - b ** 2, rtol=1e-6, atol=1e-7)
    assert np.array_equal(c, ((0.0 < a) & (a < 0.5)) | (~(b > 0.0) & (a <= -0.5)))
    assert np.array_equal(s, np.maximum(np.maximum(a, b), np.float32(0.25)) - np.minimum(a, b))


@appy.jit
def promote(i32, f32, u8, alpha, out_f32, out_f64, out_u8, out_i64):
    #pragma parallel for simd
    for i in range(i32.shape[0]):
        out_f32[i] = f32[i] * alpha + 1          # Python scalars adopt float32
        out_f64[i] = i32[i] * alpha + i32[i] / 4 # int32 with a Python float / true division: float64
        out_u8[i] = u8[i] + u8[i]                # wraps in uint8
        out_i64[i] = i32[i] * 3 + i             # the loop index is a Python int


def test_dtype_promotion_follows_numpy(rng):
    i32 = rng.integers(-100, 100, N, dtype=np.int32)
    f32 = rng.standard_normal(N).astype(np.float32)
    u8 = rng.integers(0, 256, N, dtype=np.uint8)
    alpha = 0.1
    o32, o64 = np.empty(N, np.float32), np.empty(N, np.float64)
    ou8, oi64 = np.empty(N, np.uint8), np.empty(N, np.int64)
    promote(i32, f32, u8, alpha, o32, o64, ou8, oi64)
    assert np.array_equal(o32, f32 * alpha + 1) and (f32 * alpha + 1).dtype == np.float32
    assert np.array_equal(o64, i32 * alpha + i32 / 4)
    assert np.array_equal(ou8, u8 + u8)
    assert np.array_equal(oi64, i32.astype(np.int64) * 3 + np.arange(N))


@appy.jit
def half_add(a, b, c):
    #pragma parallel for simd
    for i in range(a.shape[0]):
        c[i] = a[i] + b[i] * 2.0


def test_float16_arrays(rng):
    a = rng.standard_normal(N).astype(np.float16)
    b = rng.standard_normal(N).astype(np.float16)
    c = np.empty_like(a)
    half_add(a, b, c)
    assert c.dtype == np.float16 and np.array_equal(c, a + b * np.float16(2.0))


@appy.jit
def gather_shifted(x, idx, y, flag):
    #pragma parallel for simd
    for i in range(idx.shape[0]):
        y[i] = x[idx[i] + 1] - x[idx[i]]
        flag[i] = x[idx[i]] > 0.5


def test_gather_with_computed_index_and_bool_output(rng):
    x = rng.random(5000)
    idx = rng.integers(0, 4999, N, dtype=np.int64)
    y = np.empty(N)
    flag = np.zeros(N, dtype=bool)
    gather_shifted(x, idx, y, flag)
    assert np.array_equal(y, x[idx + 1] - x[idx]) and np.array_equal(flag, x[idx] > 0.5)


@appy.jit
def maths(a, out):
    #pragma parallel for simd
    for i in range(a.shape[0]):
        v = np.sqrt(np.abs(a[i])) + np.exp(-a[i] * a[i]) + math.sin(a[i]) * np.cos(a[i])
        w = np.log1p(np.abs(a[i])) + np.arctan2(a[i], 2.0) + np.floor(a[i]) + np.pi
        out[i] = v + w if a[i] > -10 else float("inf")


@pytest.mark.parametrize("dtype,tol", [(np.float64, 1e-13), (np.float32, 2e-6)])
def test_maths_functions(rng, dtype, tol):
    a = rng.uniform(-3, 3, N).astype(dtype)
    out = np.empty_like(a)
    maths(a, out)
    a64 = a.astype(np.float64)
    ref = (np.sqrt(np.abs(a64)) + np.exp(-a64 * a64) + np.sin(a64) * np.cos(a64)
           + np.log1p(np.abs(a64)) + np.arctan2(a64, 2.0) + np.floor(a64) + np.pi)
    assert out.dtype == dtype and np.allclose(out, ref, rtol=tol, atol=tol * 10)


@appy.jit
def private_scalar(a, t):
    #pragma parallel for simd
    for i in range(a.shape[0]):
        u = t + i
        t = 0.0
        a[i] = u
    return t


def test_scalars_are_passed_by_value(rng):
    a = np.zeros(100)
    assert private_scalar(a, 5.0) == 5.0                 # writes to a by-value scalar are invisible afterwards
    assert a[0] == 5.0 and np.all(a >= 0)


@appy.jit
def from_the_end(a, b, out):
    #pragma parallel for simd
    for i in range(out.shape[0]):
        out[i] = a[-1] + b[-2, i] - a[i]


def test_negative_literal_indices(rng):
    a = rng.random(50)
    b = rng.random((4, 50))
    out = np.empty(50)
    from_the_end(a, b, out)
    assert np.array_equal(out, a[-1] + b[-2, :] - a)


@appy.jit
def sum_2d(a):
    s = 0.0
    #pragma parallel for shared(s)
    for i in range(a.shape[0]):
        #pragma simd
        for j in range(a.shape[1]):
            s += a[i, j]
    return s


@appy.jit
def sum_of_row_maxima(a):
    s = 0.0
    #pragma parallel for shared(s)
    for i in range(a.shape[0]):
        m = -1e30
        #pragma simd
        for j in range(a.shape[1]):
            m = max(m, a[i, j])
        s += m
    return s


def test_shared_reductions_in_team_loops(rng):
    a = rng.standard_normal((301, 777))
    assert sum_2d(a) == pytest.approx(a.sum(), rel=1e-12)
    assert sum_of_row_maxima(a) == pytest.approx(a.max(axis=1).sum(), rel=1e-12)
    a32 = a.astype(np.float32)
    assert sum_2d(a32) == pytest.approx(float(a32.astype(np.float64).sum()), abs=1e-5 * float(np.abs(a32).sum()))


def test_guarded_neighbour_accesses_stay_guarded(gpu):
    """``x[i - 1] if i > 0 else 0.0``: the element before the array is never
    touched, in flat and in team kernels (the reference's heat solver,
    old-tests/codegen/triton/np_array/test_heat.py:60-76)."""
    import appy_amd as appy

    @appy.jit
    def smooth(x, y):
        #pragma parallel for simd
        for i in range(x.shape[0]):
            left = x[i - 1] if i > 0 else 0.0
            right = x[i + 1] if i < x.shape[0] - 1 else 0.0
            y[i] = 0.25 * left + 0.5 * x[i] + 0.25 * right

    @appy.jit
    def heat(n, alpha, dx, dt, u, u_tmp, nsteps):
        r = alpha * dt / (dx * dx)
        r2 = 1.0 - 4.0 * r
        for _ in range(nsteps):
            #pragma parallel for
            for i in range(n):
                #pragma simd
                for j in range(n):
                    center = u[i, j]
                    left = u[i - 1, j] if i > 0 else 0.0
                    right = u[i + 1, j] if i < n - 1 else 0.0
                    down = u[i, j - 1] if j > 0 else 0.0
                    up = u[i, j + 1] if j < n - 1 else 0.0
                    u_tmp[i, j] = r2 * center + r * (left + right + down + up)
            u, u_tmp = u_tmp, u
        return u

    rng = np.random.default_rng(21)
    x = rng.standard_normal(100_003)
    y = np.zeros_like(x)
    smooth(x, y)
    xp = np.concatenate([[0.0], x, [0.0]])
    assert np.allclose(y, 0.25 * xp[:-2] + 0.5 * x + 0.25 * xp[2:], rtol=0, atol=1e-15)

    n, nsteps = 37, 3
    u0 = rng.random((n, n))
    got = heat(n, 0.1, 0.5, 0.01, u0.copy(), np.zeros((n, n)), nsteps)
    r = 0.1 * 0.01 / 0.25
    ref = u0.copy()
    for _ in range(nsteps):
        p = np.pad(ref, 1)
        ref = (1.0 - 4.0 * r) * ref + r * (p[:-2, 1:-1] + p[2:, 1:-1] + p[1:-1, :-2] + p[1:-1, 2:])
    assert np.allclose(got, ref, rtol=1e-12, atol=1e-12)


def test_continue_in_parallel_and_simd_loops(gpu):
    """``continue`` ends one iteration wherever that iteration runs: a lane of a
    flat kernel, a team, a lane of a simd loop inside a team."""
    import appy_amd as appy

    @appy.jit
    def clip_positive(a, out):
        n = 0
        #pragma parallel for simd shared(n)
        for i in range(a.shape[0]):
            if a[i] <= 0.0:
                continue
            out[i] = a[i] * 2.0
            n += 1
        return n

    @appy.jit
    def row_sums_of_marked_rows(A, mark, out):
        #pragma parallel for
        for i in range(A.shape[0]):
            if mark[i] == 0:
                continue
            s = 0.0
            #pragma simd
            for j in range(A.shape[1]):
                if A[i, j] < 0.0:
                    continue
                s += A[i, j]
            out[i] = s

    rng = np.random.default_rng(31)
    a = rng.standard_normal(100_001)
    out = np.full_like(a, -7.0)
    n = clip_positive(a, out)
    assert n == int((a > 0).sum())
    assert np.array_equal(out, np.where(a > 0, a * 2.0, -7.0))

    A = rng.standard_normal((513, 301))
    mark = (rng.random(513) < 0.6).astype(np.int32)
    res = np.full(513, -1.0)
    row_sums_of_marked_rows(A, mark, res)
    ref = np.where(mark == 1, np.where(A >= 0, A, 0.0).sum(axis=1), -1.0)
    assert np.allclose(res, ref, rtol=1e-12, atol=1e-12)


def test_bfloat16_tensors(gpu):
    """bfloat16 exists for tensors only; results must equal PyTorch's own
    (every operation computed in float32 and rounded once)."""
    import torch

    import appy_amd as appy

    @appy.jit
    def fused(a, b, w, out, acc):
        #pragma parallel for simd
        for i in range(a.shape[0]):
            out[i] = a[i] * b[i] + 2.5
            acc[i] = a[i] * w[i]

    @appy.jit
    def row_dot(A, x, y):
        #pragma parallel for
        for i in range(A.shape[0]):
            s = 0.0
            #pragma simd
            for j in range(A.shape[1]):
                s += A[i, j] * x[j]
            y[i] = s

    g = torch.Generator(device="cuda").manual_seed(3)
    n = 100_003
    a = torch.randn(n, device="cuda", generator=g).to(torch.bfloat16)
    b = torch.randn(n, device="cuda", generator=g).to(torch.bfloat16)
    w = torch.randn(n, device="cuda", generator=g)
    out = torch.empty(n, device="cuda", dtype=torch.bfloat16)
    acc = torch.empty(n, device="cuda", dtype=torch.float32)
    fused(a, b, w, out, acc)
    assert torch.equal(out, a * b + 2.5)              # bf16 * bf16 -> bf16, + weak scalar -> bf16
    assert torch.equal(acc, a * w)                    # bf16 * float32 -> float32

    A = torch.randn(300, 1000, device="cuda", generator=g).to(torch.bfloat16)
    x = torch.randn(1000, device="cuda", generator=g).to(torch.bfloat16)
    y = torch.empty(300, device="cuda", dtype=torch.float32)
    row_dot(A, x, y)
    # `s = 0.0; s += bf16` makes s bfloat16 as the un-jitted tensor loop would: compare loosely with float64
    ref = A.double() @ x.double()
    budget = A.double().abs() @ x.double().abs()
    assert ((y.double() - ref).abs() <= 2e-2 * budget + 1e-3).all()


def test_check_bounds_reports_instead_of_faulting(gpu):
    """``check_bounds=True``: an index outside its array inside the kernel (where the
    host cannot see it) becomes an IndexError after the launch; the access itself
    never leaves the array.  A correct program computes the same as without the option."""
    import appy_amd as appy

    def spmv(data, indptr, indices, x, y):
        #pragma parallel for
        for i in range(y.shape[0]):
            s = 0.0
            #pragma simd
            for j in range(indptr[i], indptr[i + 1]):
                s += data[j] * x[indices[j]]
            y[i] = s

    checked = appy.jit(spmv, check_bounds=True)
    plain = appy.jit(spmv)
    rng = np.random.default_rng(8)
    m, n = 500, 300
    lengths = rng.integers(0, 20, m)
    indptr = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    indices = rng.integers(0, n, indptr[-1]).astype(np.int32)
    data = rng.standard_normal(indptr[-1]).astype(np.float32)
    x = rng.standard_normal(n).astype(np.float32)
    y1, y2 = np.zeros(m, np.float32), np.zeros(m, np.float32)
    plain(data, indptr, indices, x, y1)
    checked(data, indptr, indices, x, y2)
    assert np.allclose(y1, y2, rtol=1e-5, atol=1e-5)     # same sums, elements dealt to the lanes differently

    bad = indices.copy()
    bad[indptr[250]] = n + 1000                      # one column index far outside x
    y3 = np.full(m, 7.0, np.float32)
    with pytest.raises(IndexError, match=r"x\[indices\[j\]\]"):
        checked(data, indptr, bad, x, y3)
    assert (y3 == 7.0).all()                         # nothing is copied back from a failed launch
    bad[indptr[250]] = -1                            # negative run-time indices count as outside
    with pytest.raises(IndexError, match=r"x\[indices\[j\]\]"):
        checked(data, indptr, bad, x, y3)

    @appy.jit(check_bounds=True)
    def shifted_store(a, out):
        #pragma parallel for simd
        for i in range(a.shape[0]):
            k = i * 2
            out[k] = a[i]

    a = np.arange(100.0)
    out = np.zeros(150)
    with pytest.raises(IndexError, match=r"out\[k\]"):
        shifted_store(a, out)
    checked(data, indptr, indices, x, y2)            # the runtime is fine afterwards
    assert np.allclose(y1, y2, rtol=1e-5, atol=1e-5)


def test_updates_shared_between_iterations_are_atomic(gpu):
    """Histograms and sums that several iterations of the parallel loop feed
    (no index is the loop variable itself) are updated atomically; the reference's
    guide describes ``a[j] += b[i, j]`` under ``prange(i)`` as a reduction with
    regard to ``i`` (docs/source/developer.rst, "Reduction Detection")."""
    import appy_amd as appy
    from appy_amd import prange

    @appy.jit
    def histogram(bins, weights, hist, wsum, wmax):
        #pragma parallel for simd
        for i in range(bins.shape[0]):
            hist[bins[i]] += 1
            wsum[bins[i]] += weights[i]
            wmax[bins[i]] = max(wmax[bins[i]], weights[i])

    @appy.jit
    def column_sums(a, b):
        for i in prange(b.shape[0]):
            for j in range(b.shape[1]):
                a[j] += b[i, j]

    rng = np.random.default_rng(17)
    n, nb = 1_000_003, 97
    bins = rng.integers(0, nb, n).astype(np.int32)
    weights = rng.random(n)
    hist, wsum, wmax = np.zeros(nb, np.int64), np.zeros(nb), np.full(nb, -1.0)
    histogram(bins, weights, hist, wsum, wmax)
    assert np.array_equal(hist, np.bincount(bins, minlength=nb))
    assert np.allclose(wsum, np.bincount(bins, weights=weights, minlength=nb), rtol=1e-11)
    ref_max = np.full(nb, -1.0)
    np.maximum.at(ref_max, bins, weights)
    assert np.array_equal(wmax, ref_max)

    b = rng.standard_normal((700, 333)).astype(np.float32)
    a = np.zeros(333, np.float32)
    column_sums(a, b)
    assert np.allclose(a, b.sum(axis=0, dtype=np.float64), rtol=1e-4, atol=1e-3)


def _random_expression(rng, depth, leaves):
    if depth == 0 or rng.random() < 0.25:
        return leaves[rng.integers(len(leaves))]
    kind = rng.integers(0, 10)
    a = _random_expression(rng, depth - 1, leaves)
    b = _random_expression(rng, depth - 1, leaves)
    if kind <= 2:
        return f"({a} {['+', '-', '*'][kind]} {b})"
    if kind == 3:
        return f"({a} / (abs({b}) + 1))"
    if kind == 4:
        return f"({a} // (abs({b}) + 1))"
    if kind == 5:
        return f"({a} % (abs({b}) + 2))"
    if kind == 6:
        return f"({a} if {_random_expression(rng, depth - 1, leaves)} > {b} else {b})"
    if kind == 7:
        return f"{['min', 'max'][rng.integers(2)]}({a}, {b})"
    if kind == 8:
        return f"abs({a})"
    return f"(-{a})"


@pytest.mark.parametrize("seed", list(range(60)) + [230, 246, 1320])      # the last three: float `//`, uint8 multiply-add chains, integer division by zero
def test_random_expressions_type_and_value_like_numpy(gpu, seed):
    """Random expression trees over arrays of five dtypes, NumPy scalars and Python
    scalars: the kernel must produce the dtype and the values that NumPy's own
    evaluation of the same expression over the arrays gives (NEP 50 promotion,
    floor division and modulo with Python's sign rules, true division)."""
    import appy_amd as appy

    rng = np.random.default_rng(1000 + seed)
    n = 4099
    env = {
        "f": rng.uniform(-4, 4, n).astype(np.float32),
        "d": rng.uniform(-4, 4, n),
        "k": rng.integers(-20, 20, n).astype(np.int32),
        "l": rng.integers(-20, 20, n).astype(np.int64),
        "u": rng.integers(0, 9, n).astype(np.uint8),
        "s32": np.float32(1.5), "w": 3, "z": 0.75,
    }
    # the builtins keep Python scalars Python scalars (weak), as they do in the un-jitted loop
    plain = (int, float)
    env["abs"] = lambda x: abs(x) if isinstance(x, plain) else np.abs(x)
    env["min"] = lambda x, y: min(x, y) if isinstance(x, plain) and isinstance(y, plain) else np.minimum(x, y)
    env["max"] = lambda x, y: max(x, y) if isinstance(x, plain) and isinstance(y, plain) else np.maximum(x, y)
    env["h"] = rng.integers(-300, 300, n).astype(np.int16)
    leaves = ["f[i]", "d[i]", "k[i]", "l[i]", "u[i]", "h[i]", "s32", "w", "z", "2", "0.5",
              "(k[i] & 7)", "(l[i] >> 1)", "(u[i] << 2)", "(h[i] ^ k[i])", "(u[i] * u[i])", "(h[i] * h[i])",
              "np.sqrt(abs(f[i]))", "np.exp(k[i] * 0.1)", "np.floor(d[i])", "np.tanh(f[i])", "np.sqrt(l[i] * l[i])",
              "np.float32(w)", "np.int32(d[i])"]
    expr = _random_expression(rng, 3, leaves)
    vec_expr = expr.replace("[i]", "").replace("np.int32(d)", "d.astype(np.int32)")
    # `x if c else y` on arrays is np.where(c, x, y)
    import ast as _ast

    class _Where(_ast.NodeTransformer):
        def visit_IfExp(self, node):
            self.generic_visit(node)
            return _ast.Call(func=_ast.Attribute(value=_ast.Name(id="np", ctx=_ast.Load()), attr="where", ctx=_ast.Load()),
                             args=[node.test, node.body, node.orelse], keywords=[])

    tree = _ast.fix_missing_locations(_Where().visit(_ast.parse(vec_expr, mode="eval")))
    with np.errstate(all="ignore"):
        ref = eval(compile(tree, "<ref>", "eval"), {"np": np}, env)
    if isinstance(ref, (int, float)):
        pytest.skip("an expression of Python scalars only")
    ref = np.broadcast_to(np.asarray(ref), (n,)) if np.ndim(ref) == 0 else ref
    if ref.dtype == np.float16:
        pytest.skip("float16 result")
    out = np.zeros(n, dtype=ref.dtype)
    src = (f"def kernel(f, d, k, l, u, h, s32, w, z, out):\n    #pragma parallel for simd\n"
           f"    for i in range(out.shape[0]):\n        out[i] = {expr}\n")
    import linecache

    name = f"<random_expr_{seed}>"
    linecache.cache[name] = (len(src), None, src.splitlines(True), name)
    ns = {}
    exec(compile(src, name, "exec"), {"np": np, "abs": abs, "min": min, "max": max}, ns)
    fn = appy.jit(ns["kernel"])
    fn(env["f"], env["d"], env["k"], env["l"], env["u"], env["h"], env["s32"], env["w"], env["z"], out)
    if ref.dtype.kind == "f":
        # float32 exp / tanh are good to an ulp or two, which later float64 arithmetic carries along
        loose = ref.dtype == np.float32 or "np.exp" in expr or "np.tanh" in expr
        assert np.allclose(out, ref, rtol=3e-6 if loose else 1e-13, atol=1e-5 if loose else 1e-6, equal_nan=True), expr
    else:
        assert np.array_equal(out, ref), expr


def _random_program(rng):
    """A loop body with temporaries, a branch and an inner simd reduction."""
    # (no unsigned operands here: a temporary that is uint8 on one path and float on another wraps
    #  on negation in the interpreter, while a kernel variable has one type, the join of both)
    arr = ["f[i]", "d[i]", "k[i]", "A[i, 0]"]
    temps = []
    lines = []

    def leaf_pool():
        return arr + temps + ["w", "z", "s32", "2", "0.25"]

    for t in range(int(rng.integers(2, 5))):
        lines.append(f"t{t} = {_random_expression(rng, 2, leaf_pool())}")
        temps.append(f"t{t}")
    cond = f"{_random_expression(rng, 1, leaf_pool())} > {_random_expression(rng, 1, leaf_pool())}"
    tgt = temps[int(rng.integers(len(temps)))]
    lines.append(f"if {cond}:")
    lines.append(f"    {tgt} = {_random_expression(rng, 2, leaf_pool())}")
    if rng.random() < 0.5:
        lines.append("else:")
        lines.append(f"    {temps[int(rng.integers(len(temps)))]} = {_random_expression(rng, 1, leaf_pool())}")
    red = ["+", "max", "min"][int(rng.integers(3))]
    init = {"+": "0.0", "max": "-1e30", "min": "1e30"}[red]
    inner = _random_expression(rng, 2, ["A[i, j]", "v[j]", "f[i]", "k[i]", "z"] + temps)
    lines.append(f"s = {init}")
    lines.append("#pragma simd")
    lines.append("for j in range(A.shape[1]):")
    lines.append(f"    s += {inner}" if red == "+" else f"    s = {red}(s, {inner})")
    lines.append(f"out[i] = s + {_random_expression(rng, 1, temps + ['f[i]'])}")
    return lines


@pytest.mark.parametrize("seed", range(50))
def test_random_programs_against_the_interpreter(gpu, seed):
    """Random loop bodies (temporaries that change type, a branch, an inner simd
    reduction) run by the interpreter statement by statement and by the kernel."""
    import linecache

    import appy_amd as appy

    rng = np.random.default_rng(5000 + seed)
    n, m = 67, 45
    args = {
        "f": rng.uniform(-2, 2, n).astype(np.float32), "d": rng.uniform(-2, 2, n),
        "k": rng.integers(-9, 9, n).astype(np.int32), "u": rng.integers(0, 9, n).astype(np.uint8),
        "A": rng.uniform(-1, 1, (n, m)).astype(np.float32), "v": rng.uniform(-1, 1, m),
        "s32": np.float32(1.5), "w": 3, "z": 0.75,
    }
    body = _random_program(rng)
    src = ("def kernel(f, d, k, u, A, v, s32, w, z, out):\n    #pragma parallel for\n    for i in range(out.shape[0]):\n"
           + "".join(f"        {ln}\n" for ln in body))
    name = f"<random_program_{seed}>"
    linecache.cache[name] = (len(src), None, src.splitlines(True), name)
    ns = {}
    exec(compile(src, name, "exec"), {"np": np}, ns)
    ref = np.zeros(n)
    with np.errstate(all="ignore"):
        ns["kernel"](*args.values(), ref)
    out = np.zeros(n)
    appy.jit(ns["kernel"])(*args.values(), out)
    scale = np.maximum(1.0, np.abs(ref))
    assert np.all(np.abs(out - ref) <= 2e-4 * scale * m), "\n".join(body)


def test_more_numpy_functions_and_builtins(gpu):
    import appy_amd as appy

    @appy.jit
    def many(d, k, o1, o2, o3, o4, flags):
        #pragma parallel for simd
        for i in range(d.shape[0]):
            o1[i] = np.clip(d[i], -0.5, 0.75) + np.sign(d[i]) + np.heaviside(d[i], 0.5) + np.reciprocal(d[i] + 3.0)
            o2[i] = np.mod(d[i], 0.7) + np.remainder(k[i], 5) + np.floor_divide(d[i], 0.3) + np.copysign(2.0, d[i])
            o3[i] = np.round(d[i] * 3.0) + round(d[i] * 5.0) + np.deg2rad(d[i]) + np.rad2deg(d[i]) + np.negative(d[i])
            o4[i] = len(d) + d.size + d.ndim + np.multiply(d[i], 2.0) - np.subtract(d[i], 1.0) + np.divide(k[i], 4)
            flags[i] = np.isfinite(d[i]) and (k[i] in (1, 2, 3) or k[i] not in (0, 4, 5, 6, 7))

    rng = np.random.default_rng(44)
    n = 10_007
    d = rng.uniform(-2, 2, n)
    d[::97] = 0.0
    d[5] = np.inf
    k = rng.integers(-3, 9, n).astype(np.int32)
    o1, o2, o3, o4 = (np.zeros(n) for _ in range(4))
    flags = np.zeros(n, bool)
    many(d, k, o1, o2, o3, o4, flags)
    with np.errstate(all="ignore"):
        r1 = np.clip(d, -0.5, 0.75) + np.sign(d) + np.heaviside(d, 0.5) + np.reciprocal(d + 3.0)
        r2 = np.mod(d, 0.7) + np.remainder(k, 5) + np.floor_divide(d, 0.3) + np.copysign(2.0, d)
        r3 = np.round(d * 3.0) + np.rint(d * 5.0) + np.deg2rad(d) + np.rad2deg(d) + np.negative(d)
        r4 = n + n + 1 + np.multiply(d, 2.0) - np.subtract(d, 1.0) + np.divide(k, 4)
    rf = np.isfinite(d) & (np.isin(k, (1, 2, 3)) | ~np.isin(k, (0, 4, 5, 6, 7)))
    fin = np.isfinite(d)
    for got, ref in ((o1, r1), (o2, r2), (o3, r3), (o4, r4)):
        assert np.allclose(got[fin], ref[fin], rtol=1e-12, atol=1e-12)
    assert np.array_equal(flags, rf)


def test_statement_forms_of_ordinary_python(gpu):
    """Swapping tuple assignments (right-hand side first), chained targets,
    annotated assignments, asserts (dropped), ``A[r][c]``, ``elif`` chains."""
    import appy_amd as appy

    @appy.jit
    def forms(d, a, A, out, cls):
        #pragma parallel for simd
        for i in range(d.shape[0]):
            assert d[i] == d[i]
            p = q = d[i] * 2.0
            r: float = a[i]
            p, r = r, p + q                     # r becomes 4 d[i], p becomes a[i]
            p, q = q, p                         # swap: p = 2 d[i], q = a[i]
            out[i] = p * 100.0 + q * 10.0 + r + A[i % 4][i % 5]
            if d[i] > 1.0:
                cls[i] = 2
            elif d[i] > 0.0:
                cls[i] = 1
            else:
                cls[i] = 0

    rng = np.random.default_rng(51)
    n = 5003
    d, a = rng.uniform(-2, 2, n), rng.uniform(-2, 2, n)
    A = rng.uniform(-1, 1, (4, 5))
    out, cls = np.zeros(n), np.zeros(n, np.int64)
    forms(d, a, A, out, cls)
    i = np.arange(n)
    assert np.allclose(out, 2 * d * 100.0 + a * 10.0 + 4 * d + A[i % 4, i % 5], rtol=1e-13, atol=1e-12)
    assert np.array_equal(cls, np.where(d > 1.0, 2, np.where(d > 0.0, 1, 0)))


def test_uint8_square_plus_maximum_regression(gpu):
    """`-(u * u) - max(u * u, u)` over uint8: the compiler once folded the byte multiply-add
    chain into a dot-product instruction that computed `-(2 u*u + u)`."""
    import appy_amd as appy

    @appy.jit
    def kernel(u, out):
        #pragma parallel for simd
        for i in range(out.shape[0]):
            out[i] = (-(u[i] * u[i])) - max((u[i] * u[i]), u[i])

    u = np.random.default_rng(7).integers(0, 256, 100_003).astype(np.uint8)
    want = (-(u * u)) - np.maximum(u * u, u)
    for dt in (np.uint8, np.int32, np.float64):
        out = np.zeros(u.size, dt)
        kernel(u, out)
        assert np.array_equal(out, want.astype(dt))
