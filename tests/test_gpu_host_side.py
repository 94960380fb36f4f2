"""How decorated functions meet the host program on the GPU: the kinds of arguments
(views with strides, transposes, Fortran order, CPU tensors, 0-d values, aliases of one
array), where names come from (globals, closures, defaults, attributes of ``self``),
bounds that ask arrays for their length, decorated functions calling one another.
Every case runs the same function un-jitted on copies of the inputs and compares."""
import math

import numpy as np
import pytest

import appy

pytestmark = pytest.mark.gpu

SCALE = 3.0


def add(a, b, c):
    #pragma parallel for simd
    for i in range(a.shape[0]):
        c[i] = a[i] + b[i]


def rowsum(A, y):
    #pragma parallel for
    for i in range(A.shape[0]):
        s = 0.0
        #pragma simd
        for j in range(A.shape[1]):
            s += A[i, j]
        y[i] = s


jadd, jrowsum = appy.jit(add), appy.jit(rowsum)


def test_aliases_and_views_of_numpy_arrays(gpu):
    rng = np.random.default_rng(0)
    a, b = rng.standard_normal(1001), rng.standard_normal(1001)
    want = a + b
    jadd(a, b, a)                                   # output is one of the inputs
    assert np.array_equal(a, want)
    c = np.zeros(1001)
    jadd(a, a, c)                                   # one array under two names
    assert np.array_equal(c, 2 * a)
    base = rng.standard_normal(2002)
    jadd(base[::2], base[1::2], c)                  # strided inputs
    assert np.array_equal(c, base[::2] + base[1::2])
    out = np.zeros(2002)
    jadd(a, b, out[::2])                            # strided output: the gaps stay untouched
    assert np.array_equal(out[::2], a + b) and not out[1::2].any()
    jadd(a[::-1], b, c)                             # negative stride
    assert np.array_equal(c, a[::-1] + b)
    ro = a.copy()
    ro.setflags(write=False)
    jadd(ro, ro, c)                                 # read-only input
    assert np.array_equal(c, 2 * a)


def test_transposed_and_fortran_ordered_matrices(gpu):
    import torch

    rng = np.random.default_rng(1)
    A = rng.standard_normal((50, 70))
    y = np.zeros(70)
    jrowsum(A.T, y)
    assert np.allclose(y, A.sum(axis=0))
    F = np.asfortranarray(A)
    y = np.zeros(50)
    jrowsum(F, y)
    assert np.allclose(y, A.sum(axis=1))
    At = torch.from_numpy(A).cuda()
    yt = torch.zeros(70, dtype=torch.float64, device="cuda")
    jrowsum(At.T, yt)                               # a transposed GPU tensor is used in place through its strides
    assert np.allclose(yt.cpu().numpy(), A.sum(axis=0))
    base = torch.randn(2002, dtype=torch.float64, device="cuda")
    ct = torch.zeros(1001, dtype=torch.float64, device="cuda")
    jadd(base[::2], base[1::2], ct)
    assert torch.equal(ct, base[::2] + base[1::2])


def test_cpu_tensors_mixed_arguments_and_empty_arrays(gpu):
    import torch

    a, b, c = torch.randn(1001), torch.randn(1001), torch.zeros(1001)
    jadd(a, b, c)                                   # CPU tensors are copied in and out like NumPy arrays
    assert torch.equal(c, a + b)
    x = np.arange(1001.0)
    g = torch.randn(1001, dtype=torch.float64, device="cuda")
    out = np.zeros(1001)
    jadd(x, g, out)
    assert np.array_equal(out, x + g.cpu().numpy())
    e = np.zeros(0)
    jadd(e, e, e)
    jrowsum(np.zeros((0, 5)), np.zeros(0))
    y = np.ones(5)
    jrowsum(np.zeros((5, 0)), y)
    assert not y.any()


def test_names_from_globals_closures_defaults_and_self(gpu):
    k = 2.5

    @appy.jit
    def scaled(a, out, beta=1.0):
        """Uses a global, a closure variable, a default argument and a module."""
        #pragma parallel for simd
        for i in range(a.shape[0]):
            out[i] = SCALE * a[i] + k * beta + math.pi

    a = np.arange(100.0)
    out = np.zeros(100)
    scaled(a, out)
    assert np.allclose(out, 3 * a + 2.5 + math.pi)
    scaled(a, out, beta=2.0)
    assert np.allclose(out, 3 * a + 5.0 + math.pi)
    k = 4.0                                         # closures are late-bound, as in plain Python
    scaled(a, out)
    assert np.allclose(out, 3 * a + 4.0 + math.pi)

    class Model:
        def __init__(self):
            self.w = 4.0

        @appy.jit
        def run(self, a, out):
            w = self.w
            #pragma parallel for simd
            for i in range(a.shape[0]):
                out[i] = w * a[i]

    Model().run(a, out)
    assert np.array_equal(out, 4 * a)


def test_decorated_functions_defined_side_by_side_call_each_other(gpu):
    @appy.jit
    def outer(a, out):
        inner(a, out)                               # defined below: resolved when called
        #pragma parallel for simd
        for i in range(a.shape[0]):
            out[i] = out[i] * 2

    @appy.jit
    def inner(a, out):
        #pragma parallel for simd
        for i in range(a.shape[0]):
            out[i] = a[i] + 1

    a = np.arange(100.0)
    out = np.zeros(100)
    outer(a, out)
    assert np.array_equal(out, (a + 1) * 2)


def test_bounds_may_ask_arrays_for_their_length(gpu):
    @appy.jit
    def shifted(a, out, n):
        #pragma parallel for simd
        for i in range(1, len(a) // 2 + int(n)):
            out[i] = a[i - 1]

    @appy.jit
    def tail(A, y):
        #pragma parallel for
        for i in range(len(A) - 2, A.shape[0]):
            s = 0.0
            #pragma simd
            for j in range(A.size // len(A)):
                s += A[i, j]
            y[i] = s

    a = np.arange(100.0)
    out = np.zeros(100)
    shifted(a, out, 3.0)
    assert np.array_equal(out[1:53], a[:52]) and not out[53:].any() and out[0] == 0
    A = np.arange(35.0).reshape(5, 7)
    y = np.zeros(5)
    tail(A, y)
    assert np.array_equal(y, [0, 0, 0, A[3].sum(), A[4].sum()])


def test_zero_dimensional_arrays_and_tensors_are_scalars(gpu):
    import torch

    @appy.jit
    def scale(a, out, alpha):
        #pragma parallel for simd
        for i in range(a.shape[0]):
            out[i] = alpha * a[i]

    a = np.arange(100.0)
    out = np.zeros(100)
    scale(a, out, np.array(2.0))
    assert np.array_equal(out, 2 * a)
    scale(a, out, a.sum())                          # a NumPy scalar
    assert np.array_equal(out, a.sum() * a)
    at = torch.arange(100.0, device="cuda")
    ot = torch.zeros(100, device="cuda")
    scale(at, ot, torch.tensor(2.0))
    assert torch.equal(ot, 2 * at)
    scale(at, ot, at.max())                         # a 0-d GPU tensor: its value is fetched
    assert torch.equal(ot, 99 * at) and ot.dtype == torch.float32


def test_affine_subscripts_of_the_parallel_variable_are_checked_on_the_host(gpu):
    @appy.jit
    def reverse(a, out, n):
        #pragma parallel for simd
        for i in range(n):
            out[i] = a[n - 1 - i]

    @appy.jit
    def every_other(a, out, n):
        #pragma parallel for simd
        for i in range(n):
            out[i] = a[2 * i]

    @appy.jit
    def from_the_end(a, out, n):
        #pragma parallel for simd
        for i in range(n):
            out[i] = a[-i]

    a = np.arange(100.0)
    out = np.zeros(100)
    reverse(a, out, 100)
    assert np.array_equal(out, a[::-1])
    every_other(a, out, 50)
    assert np.array_equal(out[:50], a[::2])
    with pytest.raises(IndexError, match=r"subscript `2 \* i` runs from 0 to 198"):
        every_other(a, out, 100)
    with pytest.raises(IndexError, match="runs from -99 to 0"):
        from_the_end(a, out, 100)
    with pytest.raises(IndexError, match="runs from 0 to 100"):
        reverse(a, np.zeros(101), 101)


def test_shared_scalars_and_other_tiny_host_arrays_in_repeated_calls(gpu):
    """Host arrays of a few bytes travel through page-locked slots, and a call that differs from an earlier one
    only in their contents repeats that call's launch: every call must see its own values and get its own results."""
    import torch

    from appy_amd.backends.hip import codegen as cg

    @appy.jit
    def offset_sum(A, start):
        s = start
        #pragma parallel for simd shared(s)
        for i in range(A.shape[0]):
            s += A[i]
        return s

    @appy.jit
    def two_names(A, acc, also, n):
        #pragma parallel for simd
        for i in range(n):
            A[i] = A[i] + acc[0] + also[1]

    @appy.jit
    def bump(cell, by, n):
        #pragma parallel for
        for i in range(n):
            cell[i] = cell[i] + by[i]

    A = torch.arange(1000.0, device="cuda", dtype=torch.float64)
    total = float(A.sum())
    for start in (0.0, 2.5, -7.0, 1e6, 0.0):
        assert offset_sum(A, start) == total + start
    B = torch.arange(500.0, device="cuda", dtype=torch.float64)
    assert offset_sum(B, 1.0) == float(B.sum()) + 1.0           # another tensor between two repeats
    assert offset_sum(A, 3.0) == total + 3.0
    loop = [v[0] for kk, v in cg.code_cache.items() if kk[-1] == "offset_sum"][-1]
    assert loop._replays and all(plan.small_fixed for plan in loop._replays.values())
    # the same small array under two names: one copy on the device serves both
    X = torch.zeros(64, device="cuda", dtype=torch.float64)
    for k in range(3):
        pair = np.array([1.0 + k, 10.0])
        two_names(X, pair, pair, 64)
    assert torch.equal(X, torch.full((64,), 36.0, device="cuda", dtype=torch.float64))
    # a stored small array, new contents at every call
    for k in range(4):
        cell = np.array([1.0, 2.0, 3.0]) * (k + 1)
        by = torch.tensor([10.0, 20.0, 30.0], device="cuda", dtype=torch.float64)
        bump(cell, by, 3)
        assert np.array_equal(cell, np.array([11.0, 22.0, 33.0]) + np.array([1.0, 2.0, 3.0]) * k)
