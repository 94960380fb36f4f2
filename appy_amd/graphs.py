"""Record the launches of a block of code once, replay them as one submission.

A host loop around parallel loops (time stepping: Jacobi, FDTD, the heat
solver of the reference's tests) launches many short kernels; each launch
costs the interpreter some 20 microseconds while the kernel itself may run
for 3.  Inside ``with appy.graph() as g:`` the launches are captured into a
HIP graph instead of being executed; ``g.launch()`` then replays all of them
with one call.

    with appy.graph() as g:
        for t in range(100):
            step(A, B)              # @appy.jit functions, captured, not run
    for _ in range(50):
        g.launch()                  # 100 steps each
    g.synchronize()

What can be captured: loops whose array arguments already live on the GPU -
GPU tensors, or NumPy arrays inside ``appy.resident(...)``.  Anything that
would need a host/device copy at launch time (ordinary NumPy arguments,
``shared()`` scalars, non-contiguous tensors) raises ``RuntimeError`` instead of
being silently left out of the graph.  Scalar arguments and loop bounds are
frozen at the values they had during capture.  The reference has no
counterpart (its launches go through Triton one at a time).
"""
from __future__ import annotations

import threading

from .backends.hip import runtime as rt

_tls = threading.local()


def current():
    """The graph being captured on this thread, or None."""
    return getattr(_tls, "capturing", None)


class graph:
    def __init__(self, device: int = 0):
        self.device = device
        self.stream = 0
        self.exec = 0
        self.launches = 0          # kernels recorded
        self.stored_mirrors = []   # resident host arrays the recorded kernels store to
        self.used_mirrors = []     # resident host arrays the recorded kernels touch at all
        self.keepalive = []        # tensors whose memory the graph refers to
        self.stored_extents = []   # (name, address, bytes, True) of the memory the recorded kernels store into

    # ---- capture ----------------------------------------------------------------------
    def __enter__(self):
        if current() is not None:
            raise RuntimeError("appy.graph() blocks cannot be nested")
        if self.exec:
            raise RuntimeError("this graph has already been captured")
        rt.init(self.device)
        self.stream = rt.stream_create()
        rt.graph_begin(self.stream)
        _tls.capturing = self
        return self

    def __exit__(self, exc_type, exc, tb):
        _tls.capturing = None
        if exc_type is not None:
            # leave capture mode; whatever was recorded is dropped
            try:
                ex = rt.graph_end(self.stream)
                rt.graph_destroy(ex)
            except Exception:
                pass
            return False
        if self.launches == 0:
            try:
                rt.graph_end(self.stream)
            except Exception:
                pass
            raise RuntimeError("appy.graph(): the block launched no kernel")
        self.exec = rt.graph_end(self.stream)
        return False

    # ---- replay -----------------------------------------------------------------------
    def launch(self, stream=None):
        """Replay on ``stream`` (default: the graph's own stream; pass
        ``torch.cuda.current_stream().cuda_stream`` to order the replay with
        PyTorch work)."""
        if not self.exec:
            raise RuntimeError("the graph has not been captured")
        s = self.stream if stream is None else int(stream)
        if self.stored_extents:
            # orders of CSR elements kept by other loops were built from the contents of their arrays: what this replay
            # stores into is no longer what they were built from
            from .backends.hip import codegen as _cg
            _cg.drop_plans_overlapping(self.stored_extents)
        rt.graph_launch(self.exec, s)
        for m in self.used_mirrors:
            m.stream, m.busy = s, True
        for m in self.stored_mirrors:
            m.device_dirty = True

    def synchronize(self):
        rt.sync(self.stream)

    def close(self):
        if self.exec:
            rt.graph_destroy(self.exec)
            self.exec = 0
        if self.stream:
            rt.stream_destroy(self.stream)
            self.stream = 0
        self.keepalive = []
        self.stored_extents = []
        self.stored_mirrors = []
        self.used_mirrors = []

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
