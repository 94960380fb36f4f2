"""Row plans on the host: the object that owns a plan's device memory and knows what it was built from,
the list of live plans that stores by other launches invalidate, how many workgroups share a cell and
which runs of tiles each workgroup walks."""
from __future__ import annotations

import threading

import numpy as np

from . import runtime as rt
from .kernelgen import Spec

# row plans (the order of the elements of a CSR-like sum, worked out once and kept between launches)
PLAN_ROW_BITS = 15                 # rows per block: what fits a workgroup's LDS as 4-byte sums
PLAN_GROUPS = 8                    # column ranges of the gathered operand, one per XCD
PLANS_PER_LOOP = 2                 # plans a loop keeps (least recently used goes first)

_live_plans = []        # every valid plan of the process: launches that store into their arrays drop them
_plans_lock = threading.Lock()


class RowPlan:
    """The elements of one set of arrays in the order `xcells` kernels walk them, in device memory
    that this object owns.  It describes the arrays as they were when it was built: it is used only
    while every array it read is still the same object with the same version counter (tensors count
    the in-place operations PyTorch performs on them), and it is dropped when a launch of this
    package stores into memory one of those arrays occupies."""

    def __init__(self, device, key, refs, ranges):
        self.device = device
        self.key = key
        self.refs = refs            # weak references to the tensors the plan was built from
        self.ranges = ranges        # (address, bytes) of those tensors
        self.buffers = []           # device allocations of the plan
        self.nbytes = 0
        self.valid = False
        self.bin = {}               # arguments of the kernels that run the plan
        self.ncell = 0
        self.tile = 0
        self.split = 1              # workgroups per cell
        self.grid = 8               # workgroups of the kernel that runs the plan
        self.entries = 0            # positions of the streamed arrays the plan was built from
        self.owner = None           # the loop the plan belongs to
        self.inspector_ms = None

    def alloc(self, nbytes):
        ptr = rt.malloc(max(256, nbytes))
        self.buffers.append(ptr)
        self.nbytes += nbytes
        return ptr

    def alive(self, tensors) -> bool:
        return self.valid and all(r() is t for r, t in zip(self.refs, tensors))

    def release(self):
        self.valid = False
        bufs, self.buffers = self.buffers, []
        for ptr in bufs:
            try:
                rt.free(ptr)
            except Exception:       # the runtime may be shutting down
                pass
        with _plans_lock:
            if self in _live_plans:
                _live_plans.remove(self)


def drop_plans_overlapping(extents):
    """``extents``: (name, address, bytes, stored) of a launch's arrays.  Plans built from memory that
    the launch stores into are no longer true."""
    if not _live_plans:
        return
    stored = [(p, n) for _name, p, n, st in extents if st]
    if not stored:
        return
    with _plans_lock:
        hit = [plan for plan in _live_plans
               if any(p < q + m and q < p + n for p, n in stored for q, m in plan.ranges)]
    for plan in hit:
        plan.valid = False      # its memory goes back once the launches that use it have drained (CompiledLoop.release / next build)
        if plan.owner is not None:
            plan.owner._plan_seen.clear()       # the arrays have changed: they count as new
        with _plans_lock:
            if plan in _live_plans:
                _live_plans.remove(plan)


def plan_kernel_spec(tile: int, entries: int, rows: int, restrict: bool = True) -> Spec:
    """The kernel that runs a row plan of tiles of `tile` elements (over `entries` elements of `rows` rows: one
    shape for all of them)."""
    return Spec("team", block=1024, vec=1, width=1024, unroll=tile // 1024, parts=PLAN_GROUPS, aux="xcells", restrict=restrict)


def plan_split(tiles, cus: int, tile: int, entries: int, forced=None) -> int:
    """Workgroups that share a cell of a row plan (each takes a run of its tiles and has a slot of its own for the
    sums).  `tiles`: tiles per cell.  Few cells (a matrix of few blocks of rows): until there are some four runs per
    compute unit or a run is down to two tiles.  Cells of very different sizes (a banded matrix: one of the eight
    cells of a block of rows holds everything): until the largest run is no more than about what a workgroup gets
    on average.  Every doubling doubles the sums the second kernel reads, so it stops at 32."""
    if forced:
        return int(forced)
    ncell = len(tiles)
    split = max(1, min(-(-4 * cus // ncell), entries // (2 * tile * ncell), 32))
    total, largest = int(tiles.sum()), int(tiles.max()) if ncell else 0
    workgroups = max(8, cus // 8 * 8)
    while split < 32 and largest > 4 * split and -(-largest // split) > 1.25 * total / workgroups:
        split *= 2
    return split


def deal_runs(tiles, split: int, grid: int):
    """The runs of tiles of a row plan dealt to `grid` workgroups (a multiple of eight; workgroup w reads column
    range w mod 8 only): entry w + grid * i of the result is the i-th run of workgroup w, 0xFFFFFFFF for none.
    Run (block * split + part) * 8 + range holds the tiles [part * t / split, (part + 1) * t / split) of its
    cell of t tiles.  Per range the runs are sorted by size and dealt out back and forth, so that workgroups
    end up with about the same number of tiles whatever the sizes of the cells; runs without tiles are dealt
    too (their sums must be written)."""
    tiles = np.asarray(tiles, dtype=np.int64)
    ncell = len(tiles)
    per_range = grid // PLAN_GROUPS
    blocks = ncell // PLAN_GROUPS
    parts = np.arange(split, dtype=np.int64)
    t = tiles.reshape(blocks, PLAN_GROUPS)                                               # [block, range]
    size = ((parts[None, None, :] + 1) * t[:, :, None]) // split - (parts[None, None, :] * t[:, :, None]) // split
    run = (np.arange(blocks, dtype=np.int64)[:, None, None] * split + parts[None, None, :]) * PLAN_GROUPS \
        + np.arange(PLAN_GROUPS, dtype=np.int64)[None, :, None]
    rounds = -(-(blocks * split) // per_range)
    order = np.full(rounds * grid, 0xFFFFFFFF, dtype=np.uint32)
    for g in range(PLAN_GROUPS):
        sz, rn = size[:, g, :].reshape(-1), run[:, g, :].reshape(-1)
        by_size = np.lexsort((rn, -sz))                                                  # largest first, ties by number
        rank = np.arange(len(by_size))
        rnd, pos = rank // per_range, rank % per_range
        member = np.where(rnd % 2 == 0, pos, per_range - 1 - pos)
        order[(g + PLAN_GROUPS * member) + grid * rnd] = rn[by_size].astype(np.uint32)
    return order
