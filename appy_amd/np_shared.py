"""NumPy arrays that are cheap to hand to the GPU.

Mirrors the reference's ``appy.np_shared`` module (appy/np_shared.py:6-43:
``empty``, ``empty_like``, ``zeros``, ``copy``, ``randn``,
``has_device_buffer``, ``get_device_buffer``), which allocates NumPy arrays
inside buffers the GPU can see.  On a discrete GPU there is no memory both
sides address at full speed, so an array made here lives in page-locked host
memory (one DMA at link speed per copy instead of the driver's pageable path)
and owns a standing mirror in HBM that launches reuse instead of allocating.
The host copy stays the truth: every launch uploads its arguments and
downloads what it stored, unless the arrays are inside ``appy.resident(...)``.

Without a GPU the functions return ordinary NumPy arrays, so a program can
still be run with ``dry_run=True``.
"""
from __future__ import annotations

import weakref

import numpy as np

from . import residency
from .backends.hip import runtime as rt

_rng = np.random.default_rng()


class _PinnedBlock:
    """Owner of one page-locked allocation; NumPy arrays made from it keep it
    alive through their ``base`` chain, the last one to go releases the memory
    and the HBM mirror."""

    def __init__(self, nbytes: int):
        self.nbytes = nbytes
        self.addr = rt.host_alloc(max(nbytes, 1))
        self.__array_interface__ = {
            "shape": (nbytes,),
            "typestr": "|u1",
            "data": (self.addr, False),
            "version": 3,
        }
        residency.register(self.addr, nbytes, pinned=True)
        weakref.finalize(self, _release, self.addr)


def _release(addr: int) -> None:
    residency.unregister(addr)
    try:
        rt.host_free(addr)
    except Exception:
        pass        # interpreter shutdown


def _have_gpu() -> bool:
    try:
        return rt.device_count() > 0
    except Exception:
        return False


def empty(shape, dtype=np.float64):
    dtype = np.dtype(dtype)
    shape = (shape,) if isinstance(shape, (int, np.integer)) else tuple(int(s) for s in shape)
    if not _have_gpu():
        return np.empty(shape, dtype=dtype)
    rt.init(0)
    n = 1
    for s in shape:
        n *= s
    block = _PinnedBlock(n * dtype.itemsize)
    flat = np.asarray(block)[: n * dtype.itemsize]
    return flat.view(dtype).reshape(shape)


def empty_like(x, dtype=None):
    return empty(x.shape, dtype or x.dtype)


def zeros(shape, dtype=np.float64):
    out = empty(shape, dtype=dtype)
    out[...] = 0
    return out


def copy(x):
    x = np.asarray(x)
    out = empty_like(x)
    out[...] = x
    return out


def randn(*shape, dtype=np.float64):
    out = empty(shape, dtype=dtype)
    if out.size:
        _rng.standard_normal(out.shape, dtype=out.dtype, out=out)
    return out


def has_device_buffer(x) -> bool:
    """True if ``x`` (or the array it is a view of) has a standing HBM mirror."""
    return isinstance(x, np.ndarray) and residency.lookup(x.ctypes.data, x.nbytes) is not None


def get_device_buffer(x) -> int:
    """Device address of the first byte of ``x`` in its HBM mirror."""
    hit = residency.lookup(x.ctypes.data, x.nbytes)
    if hit is None:
        raise KeyError("the array has no device mirror")
    m, off = hit
    return m.device_ptr() + off


resident = residency.resident
sync_host = residency.sync_host
invalidate = residency.invalidate
