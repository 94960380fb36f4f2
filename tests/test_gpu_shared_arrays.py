"""Programs of the reference's Metal test-suite on the GPU: arrays from
``appy.np_shared`` (tests/integration/metal/test_gelu.py, test_gelu_with_y.py,
test_saxpy.py, test_mandel.py, test_vec_add.py; tests/unit/metal/test_div.py,
test_store.py, test_guard_scalar_mem_writes.py), plus the residency contract
of ``appy.resident`` that has no counterpart there.  Expected values come from
NumPy / the un-jitted loop on the same inputs; tolerances are the reference
tests' own."""
import numpy as np
import pytest

import appy
import appy.np_shared as nps
from appy_amd import residency

pytestmark = pytest.mark.gpu


def test_shared_arrays_are_pinned_numpy_arrays_with_a_mirror(gpu):
    from appy_amd.backends.hip import runtime as rt

    a = nps.empty((5, 7), dtype=np.float32)
    assert isinstance(a, np.ndarray) and a.shape == (5, 7) and a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    assert nps.has_device_buffer(a) and nps.has_device_buffer(a.reshape(-1)) and nps.has_device_buffer(a[2:])
    assert not nps.has_device_buffer(np.empty(3))
    assert rt.host_is_pinned(a.ctypes.data, a.nbytes)
    assert nps.get_device_buffer(a[1:]) == nps.get_device_buffer(a) + 7 * 4
    z = nps.zeros(1000, dtype=np.int64)
    assert z.sum() == 0
    c = nps.copy(np.arange(12.0).reshape(3, 4))
    assert np.array_equal(c, np.arange(12.0).reshape(3, 4)) and c.dtype == np.float64
    r = nps.randn(4, 3, dtype=np.float32)
    assert r.shape == (4, 3) and r.dtype == np.float32 and np.isfinite(r).all()
    e = nps.empty_like(r, dtype=np.int32)
    assert e.shape == (4, 3) and e.dtype == np.int32
    assert nps.empty(0).size == 0
    addr = a.ctypes.data
    del a
    import gc

    gc.collect()
    assert residency.lookup(addr, 4) is None and not rt.host_is_pinned(addr, 4)


@appy.jit
def gelu(x, y):
    #pragma parallel for
    for i in range(x.shape[0]):
        xi = x[i]
        x3 = xi * xi * xi
        t = np.tanh(0.79788456 * (xi + 0.044715 * x3))
        y[i] = 0.5 * xi * (1 + t)


@appy.jit
def gelu_returning(x):
    y = nps.empty_like(x)
    #pragma parallel for
    for i in range(x.shape[0]):
        xi = x[i]
        x3 = xi * xi * xi
        t = np.tanh(0.79788456 * (xi + 0.044715 * x3))
        y[i] = 0.5 * xi * (1 + t)
    return y


def _gelu_numpy(x):
    x3 = x * x * x
    return 0.5 * x * (1 + np.tanh(0.79788456 * (x + 0.044715 * x3)))


def test_gelu_on_shared_arrays(gpu):
    x = nps.randn(2_000_003, dtype=np.float32)
    y = nps.empty_like(x)
    gelu(x, y)
    ref = _gelu_numpy(x)
    assert ref.dtype == np.float32 and np.allclose(ref, y, atol=1e-6)
    y2 = gelu_returning(x)
    assert nps.has_device_buffer(y2) and np.allclose(ref, y2, atol=1e-6)


@appy.jit
def saxpy(a, x, y):
    #pragma parallel for
    for i in range(x.shape[0]):
        y[i] = a * x[i] + y[i]


def test_saxpy_in_place_on_shared_arrays(gpu):
    size = 2_000_007
    a = np.float32(2.5)
    x = nps.randn(size, dtype=np.float32)
    y = nps.randn(size, dtype=np.float32)
    ref = a * x + y
    saxpy(a, x, y)
    assert np.array_equal(ref, y)          # one multiply and one add per element, no contraction
    saxpy(a, x, y)                          # the host copy is the truth: the second call starts from the new y
    assert np.array_equal(a * x + ref, y)


@appy.jit
def mandelbrot(xmin, xmax, ymin, ymax, width, height, max_iter, out):
    size = width * height
    #pragma parallel for
    for idx in range(size):
        i = idx // width
        j = idx % width
        y = ymin + (ymax - ymin) * i / (height - 1)
        x = xmin + (xmax - xmin) * j / (width - 1)
        c_re = x
        c_im = y
        z_re = 0.0
        z_im = 0.0
        it = 0
        while z_re * z_re + z_im * z_im <= 4.0 and it < max_iter:
            new_re = z_re * z_re - z_im * z_im + c_re
            new_im = 2.0 * z_re * z_im + c_im
            z_re = new_re
            z_im = new_im
            it += 1
        out[idx] = it


def test_mandelbrot_while_loop(gpu):
    width, height, max_iter = 96, 64, 25
    xmin, xmax = np.float32(-2.0), np.float32(1.0)
    ymin, ymax = np.float32(-1.5), np.float32(1.5)
    out = nps.zeros((height, width), dtype=np.int32)
    mandelbrot(xmin, xmax, ymin, ymax, width, height, max_iter, out.reshape(-1))
    # the same statements run by the interpreter
    ref = np.zeros(height * width, dtype=np.int32)
    with np.errstate(over="ignore"):
        for idx in range(width * height):
            i, j = idx // width, idx % width
            y = ymin + (ymax - ymin) * i / (height - 1)
            x = xmin + (xmax - xmin) * j / (width - 1)
            z_re = z_im = 0.0
            it = 0
            while z_re * z_re + z_im * z_im <= 4.0 and it < max_iter:
                z_re, z_im = z_re * z_re - z_im * z_im + x, 2.0 * z_re * z_im + y
                it += 1
            ref[idx] = it
    assert np.array_equal(out.reshape(-1), ref)
    assert 1 < ref.max() == max_iter and ref.min() < 3


@appy.jit
def first_above(A, thresh, out):
    #pragma parallel for
    for i in range(A.shape[0]):
        pos = -1
        for j in range(A.shape[1]):
            if A[i, j] < 0.0:
                continue
            if A[i, j] > thresh:
                pos = j
                break
        out[i] = pos


def test_break_and_continue_in_sequential_loops(gpu):
    rng = np.random.default_rng(3)
    A = rng.standard_normal((500, 40)).astype(np.float32)
    out = np.zeros(500, dtype=np.int64)
    first_above(A, 1.5, out)
    ref = np.array([next((j for j in range(40) if A[i, j] > 1.5), -1) for i in range(500)])
    assert np.array_equal(out, ref) and (ref == -1).any() and (ref > 0).any()


@appy.jit
def div_kernel(out, alpha, beta):
    #pragma parallel for
    for i in range(out.shape[0]):
        out[i] = alpha / beta


def test_uint8_division_is_true_division(gpu):
    out = nps.empty((10,), dtype=np.float32)
    div_kernel(out, np.uint8(1), np.uint8(2))
    assert np.allclose(out, 0.5)


@appy.jit
def store_scalar(out, alpha):
    #pragma parallel for
    for i in range(out.shape[0]):
        out[i] = alpha


@pytest.mark.parametrize("dtype,value", [
    (np.int32, 10), (np.float32, 3.3), (np.bool_, True), (np.bool_, False), (np.bool_, np.bool_(True)),
    (np.int8, np.int8(10)), (np.uint8, np.uint8(10)), (np.int16, np.int16(10)), (np.uint16, np.uint16(10)),
    (np.int32, np.int32(10)), (np.uint32, np.uint32(10)), (np.float32, np.float32(3.3)),
])
def test_store_scalars_of_every_type(gpu, dtype, value):
    out = nps.empty((10,), dtype=dtype)
    out[...] = 1 if dtype is not np.bool_ else (not value)
    store_scalar(out, value)
    assert np.all(out == np.asarray(value).astype(dtype))


@appy.jit
def write_in_if(A, out, thresh):
    N = A.shape[0]
    #pragma parallel for
    for i in range(N):
        s = np.sum(A[i, :])
        if s > thresh:
            out[i] = s
        else:
            out[i] = 0.0


@appy.jit
def scale_rows(A, out):
    N, M = A.shape
    #pragma parallel for
    for i in range(N):
        out[i, :] = A[i, :] * 2.0


def test_team_kernels_guard_scalar_stores_but_not_row_stores(gpu):
    N, M = 64, 32
    A = nps.copy(np.random.default_rng(1).random((N, M)).astype(np.float32))
    out = nps.zeros((N,), dtype=np.float32)
    thresh = np.float32(M / 2)
    write_in_if(A, out, thresh)
    sums = np.asarray(A).sum(axis=1)
    assert np.allclose(out, np.where(sums > float(thresh), sums, 0.0).astype(np.float32), atol=1e-4)
    assert (out == 0).any() and (out != 0).any()
    out2 = nps.zeros((N, M), dtype=np.float32)
    scale_rows(A, out2)
    assert np.array_equal(out2, np.asarray(A) * 2.0)


# ---- residency ---------------------------------------------------------------------
@appy.jit
def axpy_into(a, x, y, out):
    #pragma parallel for simd
    for i in range(x.shape[0]):
        out[i] = a * x[i] + y[i]


@pytest.mark.parametrize("maker", ["numpy", "shared"])
def test_resident_block_uploads_once_and_downloads_on_exit(gpu, maker):
    n = 300_001
    rng = np.random.default_rng(5)
    mk = (lambda v: v.copy()) if maker == "numpy" else nps.copy
    x, y = mk(rng.standard_normal(n)), mk(rng.standard_normal(n))
    out = mk(np.zeros(n))
    x_old = x.copy()
    with appy.resident(x, y, out) as block:
        axpy_into(2.0, x, y, out)
        assert not out.any()                       # the result is still only in HBM
        block.flush()
        assert np.array_equal(out, 2.0 * x + y)
        x[...] = 1.0                               # a host write the device does not see ...
        axpy_into(1.0, x, y, out)
        appy.sync_host(out)
        assert np.array_equal(out, x_old + y)
        appy.invalidate(x)                         # ... until it is announced
        axpy_into(1.0, x, y, out)
    assert np.array_equal(out, 1.0 + y)            # downloaded on leaving the block
    assert (residency.lookup(x.ctypes.data, 8) is None) == (maker == "numpy")
    # outside the block the host copy is the truth again
    y[...] = 5.0
    axpy_into(1.0, x, y, out)
    assert np.array_equal(out, np.full(n, 6.0))


def test_resident_arguments_mix_with_other_arguments(gpu):
    import torch

    n = 100_000
    x = np.arange(n, dtype=np.float64)
    y = torch.ones(n, dtype=torch.float64, device="cuda")
    out = np.zeros(n)
    with appy.resident(x):
        axpy_into(2.0, x, y, out)           # resident NumPy + GPU tensor + ordinary NumPy output
    assert np.array_equal(out, 2.0 * x + 1.0)
    with pytest.raises(ValueError):
        with appy.resident(x[::2]):
            pass


def test_large_pageable_copies_go_through_the_staging_lanes(gpu):
    """64 MiB up and down through the four pinned lanes: content must survive, ragged sizes included."""
    from appy_amd.backends.hip import runtime as rt

    rt.init(0)
    for nbytes in ((64 << 20) + 12345, 16 << 20, (16 << 20) + 1, 40_000_001):
        src = np.random.default_rng(nbytes % 97).integers(0, 255, nbytes, dtype=np.uint8)
        dst = np.zeros_like(src)
        d = rt.malloc(nbytes)
        try:
            rt.memcpy_h2d(d, src.ctypes.data, nbytes)
            rt.memcpy_d2h(dst.ctypes.data, d, nbytes)
        finally:
            rt.free(d)
        assert np.array_equal(src, dst), nbytes
