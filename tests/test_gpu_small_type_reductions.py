"""Reductions and atomic updates whose target is narrower than 32 bits (8/16-bit integers,
float16, flags), and flags folded with ``or`` / ``and``: registers and cross-lane steps work
on 32 bits, the memory update is a compare-and-swap on the word that holds the element.
Checked against NumPy on seeded inputs (integers and flags bit-exact)."""
import numpy as np
import pytest

import appy

pytestmark = pytest.mark.gpu


@appy.jit
def extremes(a):
    lo = a[0]
    hi = a[0]
    #pragma parallel for simd shared(lo, hi)
    for i in range(a.shape[0]):
        lo = min(lo, a[i])
        hi = max(hi, a[i])
    return lo, hi


@appy.jit
def histogram(k, h, top):
    #pragma parallel for simd
    for i in range(k.shape[0]):
        h[k[i]] += 1
        top[k[i] % 4] = max(top[k[i] % 4], k[i])


@appy.jit
def flags(a, k, seen):
    found = False
    ok = True
    #pragma parallel for simd shared(found, ok)
    for i in range(a.shape[0]):
        found = found or a[i] > 4.2
        ok = ok and a[i] < 4.2
    #pragma parallel for
    for i in range(k.shape[0]):
        seen[k[i]] = seen[k[i]] or True
    return found, ok


@appy.jit
def row_flags(B, any_, all_, count):
    #pragma parallel for
    for i in range(B.shape[0]):
        f = False
        g = True
        c = np.int16(0)
        #pragma simd
        for j in range(B.shape[1]):
            f = f or B[i, j]
            g = g and not B[i, j]
            c += B[i, j]
        any_[i] = f
        all_[i] = g
        count[i] = c


@pytest.mark.parametrize("dtype", [np.uint8, np.int8, np.int16, np.uint16, np.float16])
def test_max_and_min_into_narrow_shared_scalars(gpu, dtype):
    rng = np.random.default_rng(3)
    if np.dtype(dtype).kind == "f":
        a = (rng.standard_normal(100_003) * 10).astype(dtype)
    else:
        info = np.iinfo(dtype)
        a = rng.integers(info.min, info.max, 100_003, endpoint=True).astype(dtype)
        a[a == info.min] += 1
        a[a == info.max] -= 1
    lo, hi = extremes(a)
    assert lo == a.min() and hi == a.max()


@pytest.mark.parametrize("dtype", [np.uint8, np.int8, np.int16, np.uint16, np.int32])
def test_atomic_updates_of_narrow_elements(gpu, dtype):
    rng = np.random.default_rng(4)
    k = rng.integers(0, 16, 100_003).astype(np.int32)
    h = np.zeros(16, dtype)
    top = np.zeros(5, dtype)[1:]            # a view that starts one element into its buffer
    histogram(k, h, top)
    assert np.array_equal(h, np.bincount(k, minlength=16).astype(dtype))     # wraps like NumPy's in-place add
    assert np.array_equal(top, [12, 13, 14, 15])


def test_flags_folded_with_or_and_and(gpu):
    rng = np.random.default_rng(5)
    a = rng.standard_normal(100_003)
    k = rng.integers(0, 7, 50).astype(np.int32)
    seen = np.zeros(16, bool)
    found, ok = flags(a, k, seen)
    assert found == bool((a > 4.2).any()) and ok == bool((a < 4.2).all())
    assert np.array_equal(seen, np.isin(np.arange(16), k))
    found, ok = flags(a * 0.1, k, seen)
    assert found is False and ok is True
    B = rng.random((37, 301)) < 0.004
    any_, all_, count = np.zeros(37, bool), np.zeros(37, bool), np.zeros(37, np.int16)
    row_flags(B, any_, all_, count)
    assert np.array_equal(any_, B.any(axis=1)) and np.array_equal(all_, ~B.any(axis=1))
    assert np.array_equal(count, B.sum(axis=1))


def test_integer_shared_scalars_refuse_floats(gpu):
    @appy.jit
    def total(a):
        s = 0
        #pragma parallel for simd shared(s)
        for i in range(a.shape[0]):
            s += a[i]
        return s

    assert total(np.arange(1000, dtype=np.int32)) == 499500
    with pytest.raises(TypeError, match="start the shared scalar as a float"):
        total(np.ones(10, np.float32))
