"""Device mirrors of host arrays.

For NumPy callers the PCIe copies around a launch outweigh every kernel by one
to two orders of magnitude (the reference copies each NumPy argument to the
device and each stored one back on every call,
appy/backends/triton/passes/host_passes/gen_data_movement.py:25-87; its Metal
back end avoids that with arrays that already live in device-visible memory,
appy/np_shared.py:6-35).  A *mirror* is a buffer in HBM paired with a range of
host memory, found again by address containment, so views (``a.reshape(-1)``,
``a[10:]``) of a mirrored array use the same device bytes.

Two coherence modes:

* **coherent** (default for arrays from :mod:`appy_amd.np_shared`): the host
  copy is the truth.  Every launch uploads the bytes of the argument and
  downloads stored arguments afterwards - from page-locked memory, as one DMA at
  link speed, into a mirror that is never reallocated.
* **resident** (``with appy.resident(a, b): ...`` for any C-contiguous array):
  uploaded once; launches move nothing and return without waiting for the GPU;
  arrays a kernel stored to are downloaded by ``sync_host`` / on leaving the
  ``with`` block.  Host writes in between must be announced with
  ``invalidate`` - that is the explicit part of the contract.
"""
from __future__ import annotations

import bisect
import threading

import numpy as np

from .backends.hip import runtime as rt

_lock = threading.RLock()
_bases: list[int] = []          # sorted base addresses
_by_base: dict[int, "Mirror"] = {}


class Mirror:
    """HBM buffer paired with the host bytes [addr, addr + nbytes)."""

    __slots__ = ("addr", "nbytes", "dptr", "pinned", "resident", "device_dirty", "host_dirty", "keep", "depth",
                 "stream", "busy")

    def __init__(self, addr: int, nbytes: int, pinned: bool, keep=None):
        self.addr = addr
        self.nbytes = nbytes
        self.dptr = 0
        self.pinned = pinned
        self.resident = False
        self.device_dirty = False   # a kernel stored to the mirror since the last download
        self.host_dirty = False     # the host bytes changed since the last upload (resident mode)
        self.keep = keep            # keeps an ordinary array alive while its address is registered
        self.depth = 0              # nested `resident` blocks
        self.stream = 0             # stream of the last launch that used the mirror
        self.busy = False           # a launch on `stream` may still be using the mirror

    def device_ptr(self) -> int:
        if not self.dptr:
            self.dptr = rt.malloc(max(self.nbytes, 1))
        return self.dptr

    def upload(self, stream: int = 0) -> None:
        if self.nbytes:
            rt.memcpy_h2d(self.device_ptr(), self.addr, self.nbytes, stream)
        self.host_dirty = False

    def download(self) -> None:
        if self.nbytes and self.dptr:
            rt.memcpy_d2h(self.addr, self.dptr, self.nbytes, self.stream)   # waits for the stream
            self.busy = False
        self.device_dirty = False


def active() -> bool:
    return bool(_bases)


def register(addr: int, nbytes: int, pinned: bool, keep=None) -> Mirror:
    with _lock:
        hit = lookup(addr, nbytes)
        if hit is not None and hit[0].addr == addr and hit[0].nbytes == nbytes:
            return hit[0]
        i = bisect.bisect_left(_bases, addr)
        below = _by_base[_bases[i - 1]] if i > 0 else None
        if (hit is not None or (i < len(_bases) and _bases[i] < addr + max(nbytes, 1))
                or (below is not None and below.addr + max(below.nbytes, 1) > addr)):
            raise ValueError("the array overlaps another array that is already mirrored on the device")
        m = Mirror(addr, nbytes, pinned, keep)
        _bases.insert(i, addr)
        _by_base[addr] = m
        return m


def unregister(addr: int) -> None:
    """Forget the mirror that starts at ``addr`` and return its HBM to the pool."""
    with _lock:
        m = _by_base.pop(addr, None)
        if m is None:
            return
        i = bisect.bisect_left(_bases, addr)
        if i < len(_bases) and _bases[i] == addr:
            del _bases[i]
        if m.dptr:
            try:
                if m.busy:
                    rt.sync(m.stream)   # the buffer goes back to the pool: nothing may still be reading it
                rt.free(m.dptr)
            except Exception:
                pass    # interpreter shutdown: the library may be gone already
            m.dptr = 0


def lookup(addr: int, nbytes: int):
    """(mirror, byte offset) if [addr, addr + nbytes) lies inside a mirrored range."""
    with _lock:
        if not _bases:
            return None
        i = bisect.bisect_right(_bases, addr) - 1
        if i < 0:
            return None
        m = _by_base[_bases[i]]
        if addr + nbytes <= m.addr + max(m.nbytes, 1):
            return m, addr - m.addr
        return None


def _extent(a):
    if not isinstance(a, np.ndarray):
        raise TypeError(f"expected a NumPy array, got {type(a).__name__}")
    if not a.flags["C_CONTIGUOUS"]:
        raise ValueError("only C-contiguous arrays can be mirrored on the device")
    return a.ctypes.data, a.nbytes


def _mirror_of(a, create: bool):
    addr, nbytes = _extent(a)
    hit = lookup(addr, nbytes)
    if hit is not None:
        return hit[0]
    if not create:
        return None
    return register(addr, nbytes, rt.host_is_pinned(addr, nbytes), keep=a)


class resident:
    """``with appy.resident(A, x, y): ...`` - keep the arrays in HBM for the
    duration of the block: one upload on entry, no copies around the launches
    inside, one download on exit for every array a kernel stored to."""

    def __init__(self, *arrays):
        self.arrays = arrays
        self.mirrors = []

    def __enter__(self):
        for a in self.arrays:
            _extent(a)              # refuse before anything is uploaded
        rt.init(0)
        for a in self.arrays:
            m = _mirror_of(a, create=True)
            with _lock:
                m.depth += 1
                if not m.resident:
                    m.resident = True
                    m.upload()
            self.mirrors.append(m)
        return self

    def flush(self):
        """Download what the kernels have stored so far."""
        for m in self.mirrors:
            if m.device_dirty:
                m.download()

    def __exit__(self, *exc):
        try:
            self.flush()
        finally:
            for m in self.mirrors:
                with _lock:
                    m.depth -= 1
                    if m.depth == 0:
                        m.resident = False
                        if m.keep is not None:      # an ordinary array: the registration ends here
                            unregister(m.addr)
            self.mirrors = []
        return False


def sync_host(*arrays) -> None:
    """Bring the host copies of resident arrays up to date (waits for the GPU)."""
    for a in arrays:
        m = _mirror_of(a, create=False)
        if m is not None and m.device_dirty:
            m.download()


def invalidate(*arrays) -> None:
    """The host wrote to these resident arrays: upload them again before the next launch."""
    for a in arrays:
        m = _mirror_of(a, create=False)
        if m is not None:
            m.host_dirty = True
