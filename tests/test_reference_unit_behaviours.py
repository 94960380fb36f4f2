"""The behaviours pinned by the reference's own CPU-runnable unit tests
(tests/unit/general/pragma/test_invalid_pragma.py:8-42, test_no_pragma.py:5-31,
tests/unit/general/loop_range/test_irregular_range.py:5-21), written against
``import appy`` as in the reference.  ``dry_run`` keeps them off the GPU: code
generation (and its errors) still happens, the loop is then interpreted."""
import numpy as np
import pytest

import appy


@appy.jit(dry_run=True)
def kernel_bad_clause(a, b):
    c = np.empty_like(a)
    #pragma parallel for simd my_directive
    for i in range(a.shape[0]):
        c[i] = a[i] + b[i]
    return c


@appy.jit(dry_run=True)
def kernel_blank_line(a, b):
    c = np.empty_like(a)
    #pragma parallel for simd 

    for i in range(a.shape[0]):
        c[i] = a[i] + b[i]
    return c


@appy.jit(dry_run=True)
def kernel_step_two(a, b):
    c = np.empty_like(a)
    #pragma parallel for simd
    for i in range(0, a.shape[0], 2):
        c[i] = a[i] + b[i]
    return c


def test_invalid_pragma():
    a = np.ones(10)
    b = np.ones(10)
    assert np.allclose(kernel_blank_line(a, b), a + b)
    with pytest.raises(Exception) as excinfo:
        kernel_bad_clause(a, b)
    assert "my_directive" in str(excinfo.value)


def test_irregular_range():
    a = np.ones(100)
    with pytest.raises(Exception) as excinfo:
        kernel_step_two(a, a)
    assert "range" in str(excinfo.value) and "step" in str(excinfo.value)


def test_unknown_backend():
    @appy.jit(backend="opencl", dry_run=True)
    def f(a):
        #pragma parallel for simd
        for i in range(a.shape[0]):
            a[i] = 1.0

    with pytest.raises(NotImplementedError) as e:
        f(np.zeros(4))
    assert "Unknown backend" in str(e.value)


def test_unknown_function_in_kernel():
    def helper(v):
        return v

    @appy.jit(dry_run=True)
    def f(a):
        #pragma parallel for simd
        for i in range(a.shape[0]):
            a[i] = helper(a[i])

    with pytest.raises(ValueError) as e:
        f(np.zeros(4))
    assert "Unknown function" in str(e.value)


def test_two_dimensional_array_expression_is_rejected():
    @appy.jit(dry_run=True)
    def f(a, b):
        #pragma parallel for
        for i in range(a.shape[0]):
            a[i, :, :] = b[i, :, :]

    with pytest.raises(RuntimeError) as e:
        f(np.zeros((2, 3, 4)), np.zeros((2, 3, 4)))
    assert "dimensionality" in str(e.value)
