"""HIP back end: loop text + run-time values -> launcher.

Entry point :func:`codegen` has the calling convention of the reference's back
ends (reference tree: appy/backends/triton/codegen.py:9-74 and the call in
appy/dispatcher.py:19-60): ``codegen(loop_source, loop_name, val_map, options)
-> (f, code_src)`` where ``f(*args)`` takes the non-module values of
``val_map`` positionally, returns nothing and delivers results by mutating its
array arguments; ``code_src`` is the generated source (here: HIP C++).

The launcher moves data as the reference's generated host code does
(appy/backends/triton/passes/host_passes/gen_data_movement.py:25-87): NumPy
arrays and CPU tensors are copied to the device before the launch and the ones
the loop stores to are copied back afterwards; tensors that already live on
the GPU are used in place, on PyTorch's current stream, without a
synchronisation.
"""
from __future__ import annotations

import ast
import ctypes as C
import dataclasses
import math
import threading
import types as _types

import numpy as np

from ...frontend import loop_ir
from . import array_expr
from . import dtypes as T
from . import runtime as rt
from ... import graphs, residency
from .exprs import ArrayParam, ScalarParam
from .csr_staging import CsrStaging
from .device import (ARCH, Hardware, Kernel, MI355X, compile_source, device_header, hardware, scratch_limit,  # noqa: F401 - part of this module's interface
                     _current_raw_stream, _ensure_device)
from .kernelgen import KernelBuilder, KernelSource, LoopAnalysis, Spec, Unsupported  # noqa: F401 - part of this module's interface
from .row_plans import (PLAN_GROUPS, PLAN_ROW_BITS, PLANS_PER_LOOP, RowPlan, _live_plans, deal_runs,  # noqa: F401 - part of this module's interface
                        drop_plans_overlapping, plan_kernel_spec, plan_split)

code_cache = {}
_cache_lock = threading.Lock()

# Loop bounds are evaluated on the host with the scalar arguments in scope and
# only these builtins (a bound like ``range(min(n, m))`` is ordinary Python).
_HOST_EVAL_GLOBALS = {"__builtins__": {"min": min, "max": max, "abs": abs, "int": int, "len": len, "float": float,
                                       "round": round, "bool": bool}}


class _ShapeView:
    """What host-side bound expressions may ask of an array argument: ``len(a)``,
    ``a.shape``, ``a.size``, ``a.ndim`` (never its elements)."""

    __slots__ = ("shape", "ndim", "size")

    def __init__(self, a):
        self.shape = tuple(int(d) for d in a.shape)
        self.ndim = len(self.shape)
        self.size = int(np.prod(self.shape, dtype=np.int64))

    def __len__(self):
        if not self.shape:
            raise TypeError("len() of a 0-d array")
        return self.shape[0]


# (the figures of MI355X under their old names: tests and tools that size their inputs by them)
DEFAULT_CUS = MI355X.cus
MALL_BYTES = MI355X.mall_bytes
REDUCTION_WINDOW_BYTES = 6 << 20
CACHED_REDUCTION_WINDOW_BYTES = 4 << 20
TEAM_BYTES_IN_FLIGHT = 8.0e6
# staged launches kept per loop for exact repeats of a call; a host loop that launches once
# per row or per time step (`for i in range(n): <kernel using i in a bound>`) cycles through
# n of them
REPLAY_CACHE_ENTRIES = 2048
# a parallel loop with fewer iterations than this, whose body is one independent sequential loop,
# runs the two loops as one iteration space (one wavefront per iteration would not fill 256 CUs)
COLLAPSE_BELOW_ROWS = 8192
# vector steps of a row that a lane keeps in registers between the simd loops of an iteration
ROW_CACHE_STEPS = 16
# rows whose simd loop has bounds read per row (CSR rows) are sorted by trip count before they run,
# from this many rows on
BIN_MIN_ROWS = 1 << 15
# a gathered operand larger than this is walked one stripe at a time by long rows; eight stripes (one per
# XCD and its 4 MiB L2) of at most STRIPE_BYTES each, or a multiple of eight
STRIPE_MIN_BYTES = MI355X.stripe_min_bytes
STRIPE_BYTES = MI355X.stripe_bytes
GROUP_MIN_TRIP = 4                 # ... for rows of this many elements on average, at least


# ---------------------------------------------------------------------------
# classification of run-time values
# ---------------------------------------------------------------------------
def is_numpy_array(v) -> bool:
    return isinstance(v, np.ndarray)


def is_torch_tensor(v) -> bool:
    # without importing torch: its tensors (and their subclasses) are what has `data_ptr`
    return not isinstance(v, np.ndarray) and hasattr(v, "data_ptr") and type(v).__module__.startswith("torch")


def _torch_np_dtype(t):
    import torch

    table = {
        torch.float32: np.float32, torch.float64: np.float64, torch.float16: np.float16,
        torch.int8: np.int8, torch.uint8: np.uint8, torch.int16: np.int16, torch.int32: np.int32,
        torch.int64: np.int64, torch.bool: np.bool_,
    }
    if t.dtype is torch.bfloat16:
        return "bfloat16"       # no NumPy dtype: named, and typed by the generator's own rules
    if t.dtype not in table:
        raise TypeError(f"tensor dtype {t.dtype} is not supported in generated kernels")
    return np.dtype(table[t.dtype])


def _torch():
    import torch

    return torch


def array_dtype(v):
    return v.dtype if is_numpy_array(v) else _torch_np_dtype(v)


def _signature(val_map):
    """Cache key part: names with the kind, dtype and rank of their values
    (shapes are not part of it: extents reach the kernels as arguments)."""
    sig = []
    for k, v in val_map.items():
        t = type(v)
        if t is _types.ModuleType:
            sig.append((k, t))
        elif hasattr(v, "dtype") and hasattr(v, "ndim"):
            sig.append((k, t, v.dtype, v.ndim))
        else:
            sig.append((k, t))
    return tuple(sig)


def _pow2ceil(x: float) -> int:
    n = 1
    while n < x:
        n <<= 1
    return n



# Page-locked slots with device memory of their own for host arrays of a few bytes (`shared()` scalars):
# (host address, device address) pairs, handed out per launch, per device.
_SMALL_SLOT_BYTES = 64
_small_free = {}
_small_lock = threading.Lock()


def _take_small_slot(device):
    with _small_lock:
        free = _small_free.get(device)
        if free:
            return free.pop()
    return (rt.host_alloc(_SMALL_SLOT_BYTES), rt.malloc(256))


def release_all_plans():
    for _f, _src in list(code_cache.values()):
        _f.release_plans()


class CompiledLoop:
    """Callable launcher of one annotated loop for one argument signature."""

    def __init__(self, loop_source, loop_name, val_map, options):
        self.loop_name = loop_name
        self.options = dict(options)
        self.arg_names = [k for k, v in val_map.items() if not isinstance(v, _types.ModuleType)]
        self.module_names = [k for k, v in val_map.items() if isinstance(v, _types.ModuleType)]

        tree = loop_ir.build(loop_source)
        tree, shape_refs = array_expr.transform(tree, val_map)
        self.tree = tree

        arrays, scalars = {}, {}
        for k, v in val_map.items():
            if isinstance(v, _types.ModuleType):
                continue
            if is_numpy_array(v) or is_torch_tensor(v):
                dt = array_dtype(v)
                if not T.supported(dt):
                    raise TypeError(f"array `{k}` has dtype {dt}, which is not supported in generated kernels")
                arrays[k] = ArrayParam(k, T.from_dtype(dt), v.ndim)
            else:
                ty = T.of_python_value(v)
                if ty is not None:
                    scalars[k] = ScalarParam(k, ty)
        # extents introduced by array statements: scalars filled in from the shapes at launch
        self.derived_shapes = {}
        for arr, dim in shape_refs:
            nm = f"{arr}_shape_{dim}"
            if nm not in scalars:
                scalars[nm] = ScalarParam(nm, T.WEAK_INT)
                self.derived_shapes[nm] = (arr, dim)
        self.analysis = LoopAnalysis(tree, arrays, scalars)
        a = self.analysis
        self._lo_code = compile(ast.Expression(body=ast.fix_missing_locations(_copy(a.lo_node))), "<lo>", "eval")
        self._hi_code = compile(ast.Expression(body=ast.fix_missing_locations(_copy(a.hi_node))), "<hi>", "eval")
        self._affine_check_codes = [(name, dim, text, compile(text, "<subscript>", "eval"))
                                    for name, dim, text in a.affine_checks]
        self._row_cache_codes = None
        if a.row_cache is not None:
            self._row_cache_codes = [
                tuple(compile(ast.Expression(body=ast.fix_missing_locations(_copy(b))), "<row bound>", "eval") for b in pair)
                for pair in a.row_cache[2]]
        self._collapse_codes = None
        if a.collapse is not None:
            self._collapse_codes = tuple(
                compile(ast.Expression(body=ast.fix_missing_locations(_copy(x))), "<inner bound>", "eval")
                for x in a.collapse.iter.args[:2])
        self._simd_loops = self._collect_simd_loops()
        self._row_extent_code = self._find_row_extent()
        self._strip_trip_code = None
        if a.strip is not None:
            # trip count of the first shared-out loop, for the choice between strip and other shapes
            first = next(n for n in ast.walk(a.outer) if isinstance(n, ast.For) and id(n) in a.strip)
            lo, hi, _ = first.iter.args
            self._strip_trip_code = compile(ast.Expression(body=ast.fix_missing_locations(
                ast.BinOp(left=_copy(hi), op=ast.Sub(), right=_copy(lo)))), "<trip>", "eval")
        self.kernels = {}   # Spec -> Kernel
        self._overwrite_codes = {
            name: (None if node is None else compile(ast.Expression(body=ast.fix_missing_locations(_copy(node))), "<n>", "eval"))
            for name, node in a.overwritten.items()}
        self._scratch = {}  # (device, stream) -> (device pointer, bytes): partial results of two-phase launches
        self._group_off = False     # a kernel of the grouped form could not be generated for this loop
        self._hints = {}    # device -> (address, ctypes view) of page-locked words the binned kernels report to
        self._hint_key = {} # device -> which arrays the launch that reports next was about
        self._scratch_retired = []
        self._scratch_gen = 0       # counts the times the scratch memory of this loop was (re)allocated or given back
        self._replays = {}  # call identity -> Launch that can simply be launched again
        self._plans = []    # row plans of this loop, most recently used last
        self._plan_seen = {}        # identity of the arrays of a launch that could use a plan -> launches seen with it
        self._plan_off = False      # a kernel of the planned form could not be generated for this loop
        self._plan_refused = set()  # identities whose arrays the inspector has refused
        self.last_plan = None
        # scalars that no host-side decision looks at (range of the loop, inner trip counts,
        # row extents): a replayed launch may carry new values of these
        steering = set()
        for n in ast.walk(a.outer):
            if isinstance(n, ast.For):
                for arg in n.iter.args:
                    steering.update(x.id for x in ast.walk(arg) if isinstance(x, ast.Name))
        # scalars in subscripts the host checks against the extents (`a[2 * i + off]`): a replay
        # with another value would skip that check, so the value is part of the call's identity
        for _name, _dim, text in a.affine_checks:
            steering.update(x.id for x in ast.walk(ast.parse(text, mode="eval")) if isinstance(x, ast.Name))
        # bounds that ask an array for its length or shape (`range(len(a) // 2)`) are given
        # shape-only stand-ins of the arrays when they are evaluated on the host
        self._bounds_name_arrays = bool(steering & set(a.arrays))
        self._value_only = [i for i, k in enumerate(self.arg_names)
                            if k in a.scalars and k not in steering and k not in a.assigned]
        self._value_only_set = set(self._value_only)
        self._replayable = not self.options.get("check_bounds")
        self._lock = threading.Lock()
        # default variant now: generation / compilation errors surface at first use of the loop
        self.default_spec = self._default_spec()
        self.code_src = self.kernel_for(self.default_spec).src.text
        self.last_launch = None

    # ---- variants ------------------------------------------------------------------
    def _indexed_arrays(self):
        """name -> element size of the arrays that are indexed by a variable (the
        candidates for wide loads); reduction targets like ``s[0]`` do not count."""
        found = self.__dict__.get("_indexed_cache")
        if found is None:       # (the loop does not change: walked once)
            found = {}
            for n in ast.walk(self.analysis.outer):
                if (isinstance(n, ast.Subscript) and isinstance(n.value, ast.Name)
                        and n.value.id in self.analysis.arrays and not isinstance(n.slice, ast.Constant)):
                    found[n.value.id] = self.analysis.arrays[n.value.id].ty.size
            self._indexed_cache = found
        return found

    def _elem_sizes(self):
        return list(self._indexed_arrays().values()) or [4]

    def _simd_elem_sizes(self):
        """Element sizes of the arrays that ``simd`` loops walk with their own
        variable in the contiguous dimension (what a team streams; the per-row
        result ``y[i]`` does not count)."""
        sizes = []
        for lp in ast.walk(self.analysis.outer):
            if not (isinstance(lp, ast.For) and lp is not self.analysis.outer
                    and "simd" in (getattr(lp, "pragma", None) or {}) and isinstance(lp.target, ast.Name)):
                continue
            for n in ast.walk(lp):
                if (isinstance(n, ast.Subscript) and isinstance(n.value, ast.Name) and n.value.id in self.analysis.arrays):
                    last = n.slice.elts[-1] if isinstance(n.slice, ast.Tuple) else n.slice
                    if any(isinstance(x, ast.Name) and x.id == lp.target.id for x in ast.walk(last)):
                        sizes.append(self.analysis.arrays[n.value.id].ty.size)
        return sizes

    def _default_spec(self) -> Spec:
        a = self.analysis
        widest = max(self._elem_sizes())
        v = max(1, min(4, 16 // widest))
        if a.kind == "flat":
            # 16 bytes per lane and access for 1- and 2-byte elements too (uint8 addition over
            # 1 GiB: 4 elements per lane reach 0.56 of peak), as long as the body stays small
            if not a.lane_loops and sum(1 for _ in ast.walk(a.outer)) < 120:
                v = max(1, min(16, 16 // widest))
            # with or without `simd`: iterations of a parallel loop are independent, and
            # lanes handle control flow on their own, so both forms take the vector shape
            return Spec("flat", block=256, vec=v, unroll=2)
        # teams: 16 bytes per lane of the widest element the simd loops stream, at most 8
        # elements (int8 GEMV 16384^2: 0.33 of peak with 2 elements per lane, 0.74 with 8)
        inner = self._simd_elem_sizes()
        if inner:
            v = max(1, min(8, 16 // max(inner)))
        return Spec("team", block=256, vec=v, width=64)

    def kernel_for(self, spec: Spec) -> Kernel:
        k = self.kernels.get(spec)
        if k is None:
            with self._lock:
                k = self.kernels.get(spec)
                if k is None:
                    fn = self.options.get("fn_name")
                    sym = f"{fn}_{self.loop_name}" if fn and str(fn).isidentifier() else self.loop_name
                    # the helper kernels of a loop with binned rows go by names of their own in traces
                    sym += ("_" + spec.aux if spec.aux else {1: "_parts", 2: "_fold"}[spec.phase] if spec.rows == "list" else
                            {1: "_sums", 2: "_rowwise"}[spec.guard] if spec.guard else "")
                    builder = KernelBuilder(self.analysis, sym, self.module_names, spec)
                    k = Kernel(builder.build(device_header()))
                    self.kernels[spec] = k
        return k

    def _collect_simd_loops(self):
        out = []
        for n in ast.walk(self.analysis.outer):
            if n is self.analysis.outer or not isinstance(n, ast.For):
                continue
            if "simd" not in (getattr(n, "pragma", None) or {}):
                continue
            lo, hi, _ = n.iter.args
            extent = ast.Expression(body=ast.fix_missing_locations(ast.BinOp(left=_copy(hi), op=ast.Sub(), right=_copy(lo))))
            streamed = []
            for s in ast.walk(n):
                if (isinstance(s, ast.Subscript) and isinstance(s.value, ast.Name)
                        and s.value.id in self.analysis.arrays and isinstance(s.slice, ast.Name)
                        and s.slice.id == n.target.id):
                    streamed.append(s.value.id)
            out.append((compile(extent, "<extent>", "eval"), streamed))
        return out

    def _find_row_extent(self):
        """Extent expression of a row that a sequential loop updates through a
        ``simd`` loop (``y[i, :] += a * B[k, :]`` inside ``for k``): such rows
        are kept in registers when the extent is known at compile time."""
        for n in ast.walk(self.analysis.outer):
            if (isinstance(n, ast.For) and n is not self.analysis.outer
                    and "simd" not in (getattr(n, "pragma", None) or {}) and len(n.body) == 1):
                inner = n.body[0]
                if (isinstance(inner, ast.For) and "simd" in (getattr(inner, "pragma", None) or {})
                        and len(inner.body) == 1 and isinstance(inner.body[0], ast.Assign)
                        and isinstance(inner.body[0].targets[0], ast.Subscript)):
                    lo, hi, _ = inner.iter.args
                    if isinstance(lo, ast.Constant) and lo.value == 0:
                        return compile(ast.Expression(body=ast.fix_missing_locations(_copy(hi))), "<extent>", "eval")
        return None

    def _estimate_trip(self, env, arrays, n_outer):
        """Expected trip count of the inner ``simd`` loops and whether it is the
        same for every outer iteration (bounds computable on the host)."""
        best, uniform = 0.0, True
        mid = env.get("__appy_mid")
        for code, streamed in self._simd_loops:
            try:
                best = max(best, float(eval(code, _HOST_EVAL_GLOBALS, env)))
                continue
            except Exception:
                uniform = False
            # bounds that follow the parallel variable (triangular loops): the trip count in
            # the middle of the range is the mean one
            if mid is not None:
                try:
                    best = max(best, float(eval(code, _HOST_EVAL_GLOBALS, {**env, self.analysis.var: mid})))
                    continue
                except Exception:
                    pass
            known = False
            for name in streamed:
                v = arrays.get(name)
                if v is not None and v.ndim == 1 and n_outer > 0:
                    best = max(best, v.shape[0] / n_outer)
                    known = True
            if not known:
                # nothing to go by: a middling team (16 lanes x V) loses less on either side than
                # one lane per row does on long rows
                best = max(best, 64.0)
        return best, uniform

    def choose_spec(self, n_outer, env, arrays, restrict=True, listable=True, hw=None) -> Spec:
        """``listable``: the iterations can be named by 32-bit numbers (rows sorted by length are); ``hw``: the
        device the launch is for (MI355X's figures when none is named)."""
        spec = self._choose_spec(n_outer, env, arrays, restrict, listable, hw or MI355X)
        if self.options.get("check_bounds"):
            # one element per access, every access through the checking path
            spec = dataclasses.replace(spec, vec=1, unroll=1, extent=0, lds_tile=0, stream_loads=False,
                                       stream_stores=False, checked=True)
        return spec

    def _choose_spec(self, n_outer, env, arrays, restrict=True, listable=True, hw=MI355X) -> Spec:
        DEFAULT_CUS, MALL_BYTES = hw.cus, hw.mall_bytes      # (the names the rules below were written with)
        forced = self.options.get("hip_spec")
        d = self.default_spec
        if isinstance(forced, dict):
            base = dict(kind=d.kind, block=d.block, vec=d.vec, unroll=d.unroll, width=d.width,
                        restrict=restrict, stream_loads=d.stream_loads)
            base.update(forced)
            return Spec(**base)
        if self.analysis.strip is not None and not self.analysis.outer_reductions:
            # a column reduction: lanes side by side on the contiguous dimension, the
            # wavefronts of a workgroup share out the inner loop (worth it when that
            # loop is long; a trip count the host cannot evaluate is taken to be long)
            try:
                trip = int(eval(self._strip_trip_code, _HOST_EVAL_GLOBALS, env))
            except Exception:
                trip = 1 << 20
            if trip >= 64:
                strips = -(-n_outer // 64)
                block = 1024 if strips < 4 * DEFAULT_CUS else (512 if strips < 16 * DEFAULT_CUS else 256)
                while block > 64 and trip < 4 * (block // 64):
                    block //= 2
                # eight row segments in flight per wavefront; matrices beyond the memory-side
                # cache are read non-temporally (16384^2 float32: 0.84 of peak against 0.72)
                spec = Spec("strip", block=block, vec=1, unroll=8, restrict=restrict,
                            stream_loads=self._bytes_touched(arrays) > MALL_BYTES)
                if (self.analysis.strip_split is not None and strips * 2 <= DEFAULT_CUS
                        and trip >= 64 * (block // 64) and not self.options.get("check_bounds")):
                    # few columns, many rows: one workgroup per strip would leave the chip idle
                    # (2^20 x 64 floats: 4.8 ms), so several workgroups share the rows of a strip
                    # and a second, small kernel finishes the body on their partial results
                    spec = dataclasses.replace(spec, phase=1)
                return spec
        if d.kind == "flat":
            stream = self._bytes_touched(arrays) > MALL_BYTES
            if self.analysis.lane_loops and not self.analysis.outer_reductions:
                # every lane runs loops of its own: what it reads there per step is what adjacent
                # lanes must find adjacent (one iteration per lane if the parallel variable indexes
                # the contiguous dimension), and few iterations are spread over many small
                # workgroups (column sums of 16384^2: 6 ms against 27 ms)
                vec = 1 if self.analysis.lane_loops_strided else d.vec
                block = 64 if n_outer < DEFAULT_CUS * 256 * vec else d.block
                return Spec("flat", block=block, vec=vec, unroll=1, restrict=restrict)
            if d.vec > 1 and n_outer < d.block * d.vec * d.unroll:
                return Spec("flat", block=d.block, vec=d.vec, unroll=1, restrict=restrict)
            if stream and not self.analysis.outer_reductions:
                # pure streaming beyond the memory-side cache: one tile per workgroup, loads and stores
                # non-temporal (copy: 0.82 of peak against 0.67), in large workgroups (c = a + b over 2^27
                # floats: 0.82 of peak with 1024 lanes, 0.78 with 256; copy does best with 512: 0.815 / 0.81)
                # (a store-only loop, c[i] = v over 2^28 floats: 0.85 of peak with 256 lanes, 0.79 / 0.78 with 512 / 1024)
                streams = len(self._indexed_arrays())
                block = 1024 if streams >= 3 else (512 if streams == 2 else 256)
                return Spec("flat", block=block, vec=d.vec, unroll=1, restrict=restrict,
                            stream_loads=True, stream_stores=True)
            if stream and self.analysis.outer_reductions:
                # streaming reduction: 512-lane workgroups, two vector steps per lane for one
                # input stream, four for several (vector_sum 0.90, masked_sum 0.92 of peak)
                unroll = 2 if len(self._indexed_arrays()) <= 1 else 4
                return Spec("flat", block=512, vec=d.vec, unroll=unroll, restrict=restrict, stream_loads=True)
            if self.analysis.outer_reductions and d.vec > 1 and n_outer >= 16 * 1024 * d.vec * 2:
                # input served by the caches: the atomics at the end (one per workgroup, all
                # to one address, ~10 ns each) are what is left to save, so few workgroups of
                # 1024 lanes (2^22 floats: 4.4 us against 12.0 us with 768 workgroups of 256)
                return Spec("flat", block=1024, vec=d.vec, unroll=2, restrict=restrict)
            return Spec("flat", block=d.block, vec=d.vec, unroll=d.unroll, restrict=restrict, stream_loads=stream)
        stream = self._bytes_touched(arrays) > MALL_BYTES
        v = d.vec
        # (arguments that share memory could carry a dependence from one j to the next that the
        #  analysis, which reasons by array name, cannot see)
        nj = self.collapse_count(n_outer, env) if restrict else 0
        if self._row_extent_code is not None and not nj:
            try:
                ext = int(eval(self._row_extent_code, _HOST_EVAL_GLOBALS, env))
            except Exception:
                ext = 0
            ve = v
            while ve > 1 and ext % ve:      # widest vector that divides the extent
                ve //= 2
            if ext > 0:
                w = max(1, min(64, _pow2ceil(ext / ve)))
                if -(-ext // (w * ve)) <= 8:
                    return Spec("team", block=d.block, vec=ve, width=w, restrict=restrict,
                                stream_loads=False, extent=ext)
        if nj:
            n_outer *= nj       # the pairs (i, j) are the rows from here on
        trip, uniform = self._estimate_trip(env, arrays, n_outer)
        if (self.analysis.ragged is not None and not uniform and not nj and n_outer >= BIN_MIN_ROWS and restrict
                and listable and v > 1 and self.options.get("hip_bins", True) and not self.options.get("check_bounds")):
            # rows of very different lengths (CSR): sorted into classes by a pass over their bounds,
            # every class with the team width that suits it, long rows in column stripes
            # (arguments that share memory: the pass over the bounds could read what the rows store)
            return Spec("team", block=256, vec=v, width=64, restrict=restrict, stream_loads=stream, rows="mixed")
        if trip < 2 * v:
            v = 1
        # one vector step per lane for short rows; two rows per wavefront at most
        # (two independent rows in flight per wavefront stream better than one)
        w = max(1, min(32, _pow2ceil(trip / float(v)) if trip > 0 else 1))
        if uniform and trip > 0:
            # dense rows of equal length.  Short ones stream best with two vector steps per
            # lane (2^20 rows of 64 floats: 37 us with W = 8, 53 us with W = 16); when the
            # rows are long but too few to keep 8 MB in flight with half a wavefront each,
            # a whole wavefront takes a row (4096 x 16384: 42 us against 52 us)
            w = max(1, min(32, _pow2ceil(trip / float(2 * v))))
            if trip >= 128 * v and n_outer * 32 * 16 < TEAM_BYTES_IN_FLIGHT:
                w = 64
        block = d.block
        if self.analysis.multi_wave_ok and n_outer * 32 < DEFAULT_CUS * 256 and trip >= 64 * v * 32:
            # few, very long rows: wavefront teams would leave most of the chip idle,
            # so a whole workgroup takes each row (the more lanes the fewer rows there are)
            block = 1024 if n_outer <= DEFAULT_CUS else 256
            w = block
            if (self.analysis.team_split is not None and n_outer * 2 <= DEFAULT_CUS and not nj
                    and trip >= 8 * block * v and not self.options.get("check_bounds")):
                # fewer rows than half the CUs: several workgroups share a row (4 x 2^24 floats
                # added elementwise: 3.4 ms with one workgroup per row), partial results of
                # reductions meet in a second, small kernel
                return Spec("team", block=block, vec=v, width=w, restrict=restrict, stream_loads=stream, phase=1)
        steps = 0
        if (self._row_cache_codes is not None and bool(nj) == (self.analysis.collapse is not None) and v > 1
                and restrict and not self.options.get("check_bounds")):
            # (arguments that share memory: a row that no loop stores to by name may still change)
            # the rows that several simd loops of an iteration read stay in registers when every
            # lane takes a whole, small number of vector steps of them
            try:
                spans = {(int(eval(lo, _HOST_EVAL_GLOBALS, env)), int(eval(hi, _HOST_EVAL_GLOBALS, env)))
                         for lo, hi in self._row_cache_codes}
            except Exception:
                spans = set()
            ext = 0
            if len(spans) == 1:
                (lo_, hi_), = spans
                ext = hi_ - lo_
            shapes = [(w, block)]
            if w == 64 and self.analysis.multi_wave_ok:
                # rows too long for one wavefront's registers: a workgroup takes each row
                shapes += [(256, 256), (1024, 1024)]
            for cw, cb in shapes:
                most = ROW_CACHE_STEPS if cb <= 256 else ROW_CACHE_STEPS // 2     # registers per lane halve at 1024 lanes
                if ext > 0 and ext % (cw * v) == 0 and ext // (cw * v) <= most:
                    steps, w, block = ext // (cw * v), cw, cb
                    break
        return Spec("team", block=block, vec=v, width=w, restrict=restrict, stream_loads=stream, collapse=bool(nj),
                    row_steps=steps)

    def team_parts(self, spec: Spec, n_outer: int, env, arrays, hw=MI355X) -> int:
        """Workgroups per row of a two-phase team launch: two workgroups per CU in all, each
        part at least four vector steps per lane long."""
        trip, _uniform = self._estimate_trip(env, arrays, n_outer)
        parts = min(2 * hw.cus // max(1, n_outer), int(trip // (4 * spec.block * spec.vec)), 1024)
        return max(1, parts)

    def strip_parts(self, spec: Spec, n_outer: int, env, hw=MI355X) -> int:
        """Workgroups per strip of a two-phase strip launch: one workgroup of 1024 lanes per CU
        in all (2^20 x 64 floats: 79 us with 128 workgroups, 98 with 256, 156 with 512 - the
        finishing kernel walks the parts of a column one after the other), each part at least
        four rows per wavefront long."""
        strips = -(-n_outer // 64)
        try:
            trip = int(eval(self._strip_trip_code, _HOST_EVAL_GLOBALS, env))
        except Exception:
            trip = 0
        nw = spec.block // 64
        parts = min(hw.cus // max(1, strips), max(1, trip // (4 * nw)), 1024)
        return max(1, parts)

    def grouped_shape(self, n_outer, env, arrays, hw=MI355X):
        """``(stripes, log2 of the elements per stripe, positions to group)`` for a launch that groups the
        elements of its rows by the stripe of the gathered operand they read, or None when the loop or
        these arrays do not qualify: the operand is larger than an L2 can keep next to the streams and
        no larger than 16 stripes of half an L2, the rows hold a few elements at least."""
        g = self.analysis.grouping
        if g is None or self._group_off or not self.options.get("hip_group", True):
            return None
        nx = int(arrays[g["x"]].shape[0])
        most = hw.stripe_bytes // 4         # elements per stripe: half an L2 at most, 8 or 16 stripes
        if not hw.pinned_stripes or nx * 4 <= hw.stripe_min_bytes or nx > 16 * most:
            return None
        parts = 8 if nx <= 8 * most else 16
        shift = max(1, (-(-nx // parts) - 1).bit_length())
        entries = min(int(arrays[nm].shape[0]) for nm in (g["idx"], g["carried"]) if nm)
        trip, _uniform = self._estimate_trip(env, arrays, n_outer)
        # (positions are 32-bit in the grouping kernel, and its loops step past the end by up to 1024)
        if entries >= (1 << 31) - (1 << 16) or trip < GROUP_MIN_TRIP:
            return None
        return parts, shift, entries

    def scratch(self, device: int, stream: int, nbytes: int):
        """Device memory for partial results of two-phase launches of this loop: one buffer per
        device and stream, kept until `release` (launches on one stream follow one another, so they
        may share it; it only ever grows).  None when the loop would hold more than `scratch_limit`
        allows: the caller then takes a form that needs less."""
        key = (device, stream)
        with self._lock:
            have = self._scratch.get(key)
            if have is not None and have[1] >= nbytes:
                return have[0]
            if nbytes > scratch_limit(device):
                return None
            retired = []
            if have is not None:
                # launches in flight may still name the smaller buffer: it goes back once its stream has drained
                # (at the next growth or at `release`); a buffer that launches recorded into a graph name stays
                # until `release`.  Doubling bounds what is held meanwhile.
                nbytes = min(max(nbytes, 2 * have[1]), max(nbytes, scratch_limit(device)))
                recorded = graphs.current() is not None
                self._scratch_retired.append((have[0], stream, recorded))
                if not recorded:
                    retired = [r for r in self._scratch_retired if not r[2]]
                    self._scratch_retired = [r for r in self._scratch_retired if r[2]]
            have = (rt.malloc(nbytes), nbytes)
            self._scratch[key] = have
            self._scratch_gen += 1
        for ptr, st, _recorded in retired:
            rt.sync(st)
            rt.free(ptr)
        return have[0]

    def scratch_bytes(self, device: int) -> int:
        """Device memory this loop holds on `device` between launches (scratch buffers and row plans)."""
        with self._lock:
            return (sum(n for (dev, _st), (_p, n) in self._scratch.items() if dev == device)
                    + sum(pl.nbytes for pl in self._plans if pl.device == device and pl.buffers))

    def hint(self, device: int):
        """Five page-locked 64-bit words per device that the kernel over binned rows writes (a flag, then
        the number of rows of each class it found; the kernel that groups the elements of short rows sets
        the flag to 2 when it meets rows too long for it) and the host reads when it stages the next launch.
        What is read may be old or half updated: it shapes a launch, it never decides what is computed."""
        with self._lock:
            have = self._hints.get(device)
            if have is None:
                addr = rt.host_alloc(64)
                view = (C.c_int64 * 8).from_address(addr)
                for k in range(8):
                    view[k] = 0
                have = (addr, view)
                self._hints[device] = have
            return have

    def release(self):
        """Give back the device memory this loop holds (scratch buffers of two-phase launches, row plans),
        once the launches that use it have finished."""
        self.release_plans()
        with self._lock:
            self._scratch_gen += 1
            self._replays.clear()       # (staged launches name the memory that goes back)
            held, self._scratch, self._scratch_retired = (
                [(k, p) for k, (p, _n) in self._scratch.items()] + [((None, st), p) for p, st, _rec in self._scratch_retired], {}, [])
        try:
            for dev in {key[0] for key, _ptr in held if key[0] is not None} or ({0} if held else set()):
                _ensure_device(dev)
                rt.device_sync()        # (streams named by the keys may have been destroyed since)
            for _key, ptr in held:
                rt.free(ptr)
            with self._lock:
                hints, self._hints = self._hints, {}
            for addr, _view in hints.values():
                rt.host_free(addr)
        except Exception:           # the runtime may be shutting down
            pass

    def release_plans(self):
        """Give back the memory of this loop's row plans, once the launches that use them have finished."""
        with self._lock:
            plans, self._plans = self._plans, []
            self._plan_seen.clear()
        for plan in plans:
            try:
                _ensure_device(plan.device)
                rt.device_sync()        # (the streams the plan was used on may no longer exist)
            except Exception:
                pass
            plan.release()

    def plan_arrays(self):
        """Names of the arrays a row plan is built from: what the set-up of a row reads, the index array
        and the array whose elements travel with the indices."""
        a = self.analysis
        g = a.grouping
        body = a.outer.body
        at = next(k for k, st in enumerate(body) if st is a.team_split)
        names = []
        for st in body[:at]:
            for n in ast.walk(st):
                if isinstance(n, ast.Name) and n.id in a.arrays and n.id not in names:
                    names.append(n.id)
        for b in a.team_split.iter.args[:2]:
            for n in ast.walk(b):
                if isinstance(n, ast.Name) and n.id in a.arrays and n.id not in names:
                    names.append(n.id)
        for nm in (g["idx"], g["carried"]):
            if nm and nm not in names:
                names.append(nm)
        return names

    def plan_shape(self, n_outer, env, arrays, hw=MI355X):
        """The shape of a row plan for these arrays (runtime.RowPlanShape), or None when they do not
        qualify: the conditions of the grouped form (an operand too large for an L2, rows of a few
        elements), and keys and packed words of 32 bits."""
        base = self.grouped_shape(n_outer, env, arrays, hw)
        if base is None or self._plan_off:
            return None
        g = self.analysis.grouping
        nx = int(arrays[g["x"]].shape[0])
        entries = base[2]
        width = -(-(-(-nx // PLAN_GROUPS)) // 32) * 32
        col_bits = max(5, (width - 1).bit_length())
        if col_bits > 20:
            return None
        lines = PLAN_GROUPS * (width >> 5)
        line_bits = max(1, (lines - 1).bit_length())
        blocks = -(-n_outer // (1 << PLAN_ROW_BITS))
        if (blocks << line_bits) > (1 << 31) or entries >= (1 << 31):
            return None
        return rt.RowPlanShape(entries=entries, row_blocks=blocks, groups=PLAN_GROUPS, group_width=width,
                               col_bits=col_bits, tile=6144 if col_bits <= 19 else 4096, line_bits=line_bits)

    def collapse_count(self, n_outer, env) -> int:
        """Trip count of the sequential loop that may be collapsed into the parallel loop,
        when that is possible and worth it for ``n_outer`` parallel iterations; else 0."""
        if self._collapse_codes is None or n_outer >= COLLAPSE_BELOW_ROWS or self.options.get("check_bounds"):
            return 0
        try:
            lo = int(eval(self._collapse_codes[0], _HOST_EVAL_GLOBALS, env))
            hi = int(eval(self._collapse_codes[1], _HOST_EVAL_GLOBALS, env))
        except Exception:
            return 0
        return hi - lo if hi - lo >= 2 else 0

    def row_hint(self, n_outer, env, arrays):
        """(expected inner trip count, same for every row?) for grid sizing."""
        if self.analysis.kind != "team":
            return 0.0, False
        return self._estimate_trip(env, arrays, n_outer)

    def _bytes_touched(self, arrays) -> int:
        total = 0
        for name, v in arrays.items():
            arr = self.analysis.arrays[name]
            if arr.loaded or arr.stored:
                n = 1
                for d in v.shape:
                    n *= int(d)
                total += n * arr.ty.size
        return total

    def grid_for(self, spec: Spec, n_outer: int, cus: int = MI355X.cus, kernel=None, row_hint=(0.0, False)) -> int:
        if spec.kind == "strip":
            return int(min(max(1, -(-n_outer // 64)), self.options.get("hip_max_blocks") or (1 << 22)))
        if spec.kind == "flat":
            per_block = spec.block * spec.vec * spec.unroll
            need = max(1, -(-n_outer // per_block))
            step_bytes = kernel.src.lane_step_bytes if kernel is not None else 0
            if self.analysis.outer_reductions and step_bytes and not self.options.get("hip_max_blocks"):
                # persistent workgroups sized by the window of the widest input they sweep
                # per grid step: 6 MiB (HBM at 8 TB/s with ~0.8 us of latency wants that
                # much outstanding; fewer workgroups starve it, more only add serialised
                # atomics; measured optimum for every reduction tried)
                widest = spec.vec * max(self._elem_sizes())
                window = REDUCTION_WINDOW_BYTES if spec.stream_loads else CACHED_REDUCTION_WINDOW_BYTES
                want = window / float(spec.block * spec.unroll * widest)
                cap = max(64, min(cus * 8, int(round(want / 64.0)) * 64))
                return int(min(need, cap))
            # reductions end with one atomic per workgroup: few, persistent
            # workgroups (2 per CU); streaming loops take one tile per workgroup
            if self.options.get("hip_max_blocks"):
                cap = self.options["hip_max_blocks"]
            elif self.analysis.outer_reductions:
                cap = cus * 16   # scalar accesses only: more lanes to keep bytes in flight
            elif spec.stream_stores:
                cap = 1 << 22
            else:
                cap = cus * 32
            return int(min(need, cap))
        tpb = spec.block // spec.width
        need = max(1, -(-n_outer // tpb))
        trip, uniform = row_hint
        if uniform and not spec.extent and trip * spec.vec >= 4096 and not self.options.get("hip_max_blocks"):
            # long dense rows stream like a flat loop: persistent workgroups holding
            # ~8 MB in flight, each taking a whole number of row batches (GEMV
            # 16384^2: 1024 workgroups x 2 batches = 0.89 of peak, 2048 x 1 = 0.81)
            step = 16 * 2
            target = max(cus, TEAM_BYTES_IN_FLIGHT / float(spec.block * step))
            passes = max(1, int(round(need / target)))
            return int(max(1, -(-need // passes)))
        return int(min(need, self.options.get("hip_max_blocks") or (1 << 22)))

    # ---- call ------------------------------------------------------------------------
    def __call__(self, *args):
        if len(args) != len(self.arg_names):
            raise TypeError(f"{self.loop_name} expects {len(self.arg_names)} arguments, got {len(args)}")
        key = self._replay_key(args) if self._replayable else None
        if key is not None:
            plan = self._replays.get(key)
            if plan is not None and plan.seq_replay is not None and not self._sequence_still_right(plan, args):
                with self._lock:
                    self._replays.pop(key, None)
                plan = None
            if plan is not None:
                # same tensors (address, shape, strides), same scalars, same stream: the staged
                # launch of last time is still exact, so only the launch itself is repeated
                _ensure_device(plan.device)
                if _live_plans and plan.stored_extents:
                    drop_plans_overlapping(plan.stored_extents)
                if plan.seq_replay is not None:
                    plan.launch_only()      # the kernels of a CSR-like loop, as they were staged
                elif plan.small_fixed:
                    # host arrays of a few bytes (`shared()` scalars): through the slots the plan keeps for them
                    with self._lock:        # the slots and the argument block are shared by all replays of this plan
                        for slot, i, nbytes, _stored in plan.small_fixed:
                            C.memmove(slot[0], args[i].ctypes.data, nbytes)
                            rt.memcpy_h2d_async(slot[1], slot[0], nbytes, plan.stream)
                        for i in self._value_only:
                            fname = plan.scalar_fields.get(self.arg_names[i])
                            if fname is not None:
                                v = args[i]
                                setattr(plan.args, fname, v.item() if isinstance(v, np.generic) else v)
                        rt.launch(plan.function(), plan.grid, plan.block, plan.args, plan.stream)
                        waited = False
                        for slot, i, nbytes, stored in plan.small_fixed:
                            if stored:
                                rt.memcpy_d2h(slot[0], slot[1], nbytes, plan.stream)
                                C.memmove(args[i].ctypes.data, slot[0], nbytes)
                                waited = True
                        if not waited:
                            rt.sync(plan.stream)
                elif self._value_only:
                    with self._lock:        # the argument block is shared by all replays of this plan
                        for i in self._value_only:
                            fname = plan.scalar_fields.get(self.arg_names[i])
                            if fname is not None:
                                v = args[i]
                                setattr(plan.args, fname, v.item() if isinstance(v, np.generic) else v)
                        rt.launch(plan.function(), plan.grid, plan.block, plan.args, plan.stream)
                else:
                    rt.launch(plan.function(), plan.grid, plan.block, plan.args, plan.stream)
                self.last_launch = plan
                return
        vals = dict(zip(self.arg_names, args))
        plan = self.prepare(vals)
        if plan is None:
            return
        plan.keep_small = key is not None
        plan.run()
        if key is not None and plan.replayable():
            plan.small_fixed = [(slot, self.arg_names.index(name), host.nbytes, stored) for slot, host, stored, name in plan.small_kept]
            plan.small_kept = []
            with self._lock:        # launches may come from several interpreter threads
                if len(self._replays) >= REPLAY_CACHE_ENTRIES:
                    # drop the older half (dicts keep insertion order)
                    for old in list(self._replays)[:REPLAY_CACHE_ENTRIES // 2]:
                        self._replays.pop(old, None)
                self._replays[key] = plan
        elif plan.small_kept:
            plan.small, plan.small_kept = plan.small_kept, []
            plan._return_small_slots(wait=False)

    def _sequence_still_right(self, launch, args) -> bool:
        """For a staged sequence of launches that is about to be repeated as it is: the loop's scratch memory
        is the memory the launches name, and
        - over a kept order of the elements (a row plan): the plan still stands (no launch has stored into its
          arrays, it has not been given back) and the arrays are the very tensors it was built from with their
          version counters unmoved;
        - over the raw arrays, in a form chosen from what the last launch reported about the lengths of the
          rows: the report is still about these arrays and still says the same (the results never depend on
          it, the choice of the kernels does)."""
        kind, gen = launch.seq_replay[0], launch.seq_replay[1]
        if gen != self._scratch_gen:
            return False
        if kind == "plan":
            plan, tensors = launch.seq_replay[2], launch.seq_replay[3]
            if not plan.valid:
                return False
            for i, ref, version in tensors:
                t = args[i]
                if ref() is not t or t._version != version:
                    return False
            return True
        ident, seen = launch.seq_replay[2], launch.seq_replay[3]
        if self._hint_key.get(launch.device) != ident:
            return False
        _addr, hint = self.hint(launch.device)
        return all(int(hint[k]) == seen[k] for k in range(5))

    def overwrites(self, name, lo, hi, env, shape) -> bool:
        """True if this launch stores every element of array ``name`` (so that its
        previous contents need not travel to the device)."""
        if name not in self._overwrite_codes or lo != 0 or hi != shape[0]:
            return False
        code = self._overwrite_codes[name]
        if code is None:
            return len(shape) == 1
        try:
            return len(shape) == 2 and int(eval(code, _HOST_EVAL_GLOBALS, env)) == shape[1]
        except Exception:
            return False

    def _replay_key(self, args):
        """Identity of a call whose arrays all live on the GPU already; None for
        any other call (host arrays are copied per call, captures record)."""
        if graphs.current() is not None:
            return None
        key = []
        device = -1
        free = self._value_only_set
        for i, v in enumerate(args):
            t = type(v)
            if t is int or t is float or t is bool:
                key.append(t if i in free else (t, v))
            elif isinstance(v, np.generic):
                key.append(v.dtype.num if i in free else (v.dtype.num, v.item()))
            elif hasattr(v, "data_ptr"):        # a tensor
                if not v.is_cuda:
                    return None
                device = v.device.index or 0
                key.append((v.data_ptr(), v.shape, v.stride()))
            elif t is np.ndarray and 0 < v.nbytes <= _SMALL_SLOT_BYTES and v.flags["C_CONTIGUOUS"] and not residency.active():
                key.append(("small", v.dtype.str, v.shape))      # travels through a slot of the plan at every call
            else:
                return None
        if device < 0:
            return None
        key.append(_current_raw_stream(device))
        return tuple(key)

    def prepare(self, vals):
        """Stage arguments on the device and pick the kernel variant.  Returns
        a :class:`Launch` (None for an empty iteration space)."""
        a = self.analysis
        env = {k: v for k, v in vals.items() if k not in a.arrays}
        env["np"] = np
        env["math"] = math
        if self._bounds_name_arrays:
            for k in a.arrays:
                env[k] = _ShapeView(vals[k])
        lo = int(eval(self._lo_code, _HOST_EVAL_GLOBALS, env))
        hi = int(eval(self._hi_code, _HOST_EVAL_GLOBALS, env))
        if hi <= lo:
            return None
        arrays = {k: vals[k] for k in a.arrays}
        env["__appy_mid"] = (lo + hi) // 2      # where triangular inner loops have their mean length
        for nm, (an, dim) in self.derived_shapes.items():
            env[nm] = int(arrays[an].shape[dim])
        return Launch(self, vals, arrays, env, lo, hi)


class Launch(CsrStaging):
    """One staged launch: device pointers, argument block, grid."""

    serial = 0      # launches staged so far in this process (a diagnostic: which of two loops ran last)

    def __init__(self, loop: CompiledLoop, vals, arrays, env, lo, hi):
        self.loop = loop
        Launch.serial += 1
        self.serial = Launch.serial
        a = loop.analysis
        self.lo, self.hi = lo, hi
        self.env = env
        self.temps = []          # (dptr, host ndarray (contiguous), original, stored)
        self.mirrored = []       # (mirror, dptr, host ndarray, stored): arguments with a standing HBM mirror
        self.oob = 0             # checked kernels: device word that receives the report
        self.keepalive_copies = False   # a non-contiguous tensor was repacked for this launch
        self.staged_twice = {}   # (address, bytes, strides, dtype) of a staged host array -> (index in temps, uploaded?)
        self.aliases = []        # (name, dptr, bytes, stored) of host arrays that share the copy of another name
        self.keepalive = []
        self.sequence = None
        self.bin = None
        self.plan = None         # the row plan this launch runs, if any
        self.small = []          # (slot, host ndarray, stored, name): arrays of a few bytes staged through page-locked slots
        self.keep_small = False  # the slots stay with this launch when it is kept for repeats of the call
        self.small_kept = []
        self.small_fixed = []    # a launch kept for repeats: (slot, argument number, bytes, stored)
        try:
            self._stage(vals, arrays)
        except BaseException:
            # nothing is launched: staging buffers taken so far go back to the pool
            for dptr, *_ in self.temps:
                rt.free(dptr)
            self.temps = []
            self._return_small_slots(wait=True)
            if self.oob:
                rt.free(self.oob)
                self.oob = 0
            raise

    def _stage(self, vals, arrays):
        loop, a, env, lo, hi = self.loop, self.loop.analysis, self.env, self.lo, self.hi
        # -- bounds of accesses indexed by the parallel loop variable (host check, before any device work)
        for name, dim, off in a.bound_checks:
            ext = arrays[name].shape[dim]
            if lo + off < 0 or hi - 1 + off >= ext:
                raise IndexError(
                    f"{loop.loop_name}: `{name}` has extent {ext} in dimension {dim} but the loop "
                    f"range [{lo}, {hi}) indexes it at offset {off:+d}"
                )

        for name, dim, text, code in loop._affine_check_codes:
            ext = arrays[name].shape[dim]
            try:
                ends = [int(eval(code, _HOST_EVAL_GLOBALS, {**env, a.var: x})) for x in (lo, hi - 1)]
            except Exception:
                continue        # not computable on the host: left to the kernel
            if min(ends) < 0 or max(ends) >= ext:
                raise IndexError(
                    f"{loop.loop_name}: `{name}` has extent {ext} in dimension {dim} but over the loop range "
                    f"[{lo}, {hi}) its subscript `{text}` runs from {min(ends)} to {max(ends)} "
                    f"(negative subscripts other than literals count as outside)")

        self.stream = 0
        device = 0
        # -- device and stream: PyTorch's when a GPU tensor takes part
        on_gpu = {}
        for name, v in arrays.items():
            if not isinstance(v, np.ndarray) and v.is_cuda:
                if not on_gpu:
                    device = v.device.index or 0
                    self.stream = _current_raw_stream(device)
                on_gpu[name] = True
        self.capture = graphs.current()
        if self.capture is not None:
            # the launch is recorded into the graph's stream, not executed
            if device != self.capture.device:
                raise RuntimeError(f"{loop.loop_name}: arguments live on device {device}, the graph being "
                                   f"captured on device {self.capture.device}")
            self.stream = self.capture.stream
        _ensure_device(device)
        self.device = device

        # -- device pointers and strides
        self.ptr = {}
        self.strides = {}
        extents = []
        for name, v in arrays.items():
            arr = a.arrays[name]
            if not (arr.loaded or arr.stored):
                continue
            if isinstance(v, np.ndarray):
                host = v if v.flags["C_CONTIGUOUS"] else np.ascontiguousarray(v)
                self._stage_host(name, host, v, arr.stored)
            elif name in on_gpu:
                t = v
                strides = t.stride()
                if strides and strides[-1] != 1 and t.numel() > 1:
                    self._no_capture(name, "its last dimension is not contiguous (it would be repacked per launch)")
                    t = v.contiguous()
                    strides = t.stride()
                    self.keepalive_copies = True
                    if arr.stored:
                        self.keepalive.append(("copy_back", v, t))
                self.keepalive.append(t)
                dptr = t.data_ptr()
                self.ptr[name] = dptr
                self.strides[name] = strides
                extents.append((name, dptr, t.numel() * t.element_size(), arr.stored))
            else:
                # CPU tensor: same path as NumPy through a shared-memory view
                self._no_capture(name, "it is a CPU tensor (it would be copied per launch)")
                tc = v if v.is_contiguous() else v.contiguous()
                host = tc.view(_torch().int16).numpy() if tc.dtype is _torch().bfloat16 else tc.numpy()
                self._stage_host(name, host, v if tc is v else ("tensor", v, tc), arr.stored)
        for dptr, host, _orig, stored, name in self.temps:
            extents.append((name, dptr, host.nbytes, stored))
        for slot, host, stored, name in self.small:
            extents.append((name, slot[1], host.nbytes, stored))
        extents.extend(self.aliases)
        for _m, dptr, host, stored, name in self.mirrored:
            extents.append((name, dptr, host.nbytes, stored))
        restrict = not _overlaps(extents)
        # (what this launch stores into: a launch repeated without being staged again, and the replay of a graph it was
        #  recorded into, must drop the row plans built from that memory just as this staging does)
        self.stored_extents = [e for e in extents if e[3]]
        drop_plans_overlapping(extents)

        # -- kernel variant, argument block, grid
        n_outer = hi - lo
        hw = self.hw = hardware(device)
        spec = loop.choose_spec(n_outer, env, arrays, restrict=restrict, listable=hi < (1 << 31), hw=hw)
        if spec.kind == "flat" and spec.hoist_guarded and a.guarded_checks:
            # loads the program guards with a condition may only be issued early when
            # they cannot leave their array anywhere in the range
            for name, dim, off in a.guarded_checks:
                if lo + off < 0 or hi - 1 + off >= arrays[name].shape[dim]:
                    spec = dataclasses.replace(spec, hoist_guarded=False)
                    break
        self.kernel = loop.kernel_for(spec)
        self.spec = spec
        self.second = None           # (kernel, argument block, grid, block) of the finishing kernel of a two-phase launch
        self.nsplit = 1
        self.scratch_ptr = 0
        if spec.phase == 1 and spec.kind == "strip":
            self.nsplit = loop.strip_parts(spec, n_outer, env, hw)
            reds = len(a.strip[id(a.strip_split)])
            self.scratch_ptr = loop.scratch(device, self.stream, max(1, reds) * self.nsplit * n_outer * 8)
        elif spec.phase == 1:
            self.nsplit = loop.team_parts(spec, n_outer, env, arrays, hw)
            reds = len(loop_ir.reductions_of(a.team_split))
            self.scratch_ptr = loop.scratch(device, self.stream, max(1, reds) * self.nsplit * n_outer * 8)
        if spec.phase == 1 and self.scratch_ptr is None:
            # more scratch memory than the loop may hold: one kernel, one workgroup per strip or row
            spec = dataclasses.replace(spec, phase=0)
            self.kernel, self.spec, self.nsplit, self.scratch_ptr = loop.kernel_for(spec), spec, 1, 0
        self.scalar_fields = {}      # by-value scalar -> field of the argument block
        self.sequence = None         # binned rows: [(kernel, argument block, grid, block)] launched in this order
        self.seq_replay = None       # for a sequence that may be repeated as it is: what must still hold then
        self.plan_pending = False    # a later launch over the same tensors would work out a row plan
        if spec.rows == "mixed":
            if (self._stage_planned(vals, arrays, lo, hi, spec) or self._stage_grouped(vals, arrays, lo, hi, spec)
                    or self._stage_binned(vals, arrays, lo, hi, spec)):
                loop.last_launch = self
                return
            # not even the lists of rows fit what the loop may hold: one team width for all rows
            spec = loop.choose_spec(n_outer, env, arrays, restrict=restrict, listable=False, hw=hw)
            self.kernel, self.spec = loop.kernel_for(spec), spec
        self.args = self._argument_block(self.kernel, vals, arrays, lo, hi)
        if spec.phase == 1 and spec.kind == "strip":
            strips = -(-n_outer // 64)
            if a.strip_split_needs_finish():
                fin = loop.kernel_for(dataclasses.replace(spec, block=64, phase=2))
                self.second = (fin, self._argument_block(fin, vals, arrays, lo, hi), (strips, 1, 1), (64, 1, 1))
            self.grid = (strips * self.nsplit, 1, 1)
        elif spec.phase == 1:
            if a.split_needs_finish():
                fin = loop.kernel_for(dataclasses.replace(spec, block=64, width=64, phase=2))
                self.second = (fin, self._argument_block(fin, vals, arrays, lo, hi), (n_outer, 1, 1), (64, 1, 1))
            self.grid = (n_outer * self.nsplit, 1, 1)
        else:
            if spec.collapse:
                n_outer *= max(1, loop.collapse_count(n_outer, env))
            self.grid = (loop.grid_for(spec, n_outer, cus=hw.cus, kernel=self.kernel,
                                       row_hint=loop.row_hint(n_outer, env, arrays)), 1, 1)
        self.block = (spec.block, 1, 1)
        loop.last_launch = self

    def _argument_block(self, kernel, vals, arrays, lo, hi):
        loop = self.loop
        st = kernel.ArgStruct()
        for fname, p in zip(kernel._field_names, kernel.src.params):
            if p.role == "array":
                val = self.ptr[p.source]
            elif p.role == "stride":
                val = int(self.strides[p.source][p.dim])
            elif p.role == "scalar":
                if p.source in loop.derived_shapes:
                    an, dim = loop.derived_shapes[p.source]
                    val = int(arrays[an].shape[dim])
                else:
                    val = vals[p.source]
                    self.scalar_fields[p.source] = fname
                    if isinstance(val, np.generic):
                        val = val.item()
            elif p.role == "shape":
                val = int(arrays[p.source].shape[p.dim])
            elif p.role == "oob":
                self._no_capture("__oob", "bounds-checked kernels report to the host after every launch")
                self.oob = rt.malloc(4)
                rt.memset_async(self.oob, 0, 4, self.stream)
                val = self.oob
            elif p.role == "scratch":
                val = self.scratch_ptr
            elif p.role == "nsplit":
                val = self.nsplit
            elif p.role in ("threshold", "widthlog"):
                val = self.bin[p.role][p.dim]
            elif p.role in ("rows", "counts", "zero", "nrows", "bnd", "cap", "stripe", "m", "base", "skip", "tlo", "thi", "load", "hint", "rowstart",
                            "flag", "desc", "ent", "shiftc", "entries", "rowmax", "keys", "vals", "nx", "lbits", "cstart", "tbase",
                            "rstream", "ncell", "gwidth", "colbits", "split", "order", "norder"):
                val = self.bin[p.role]
            elif p.role == "lo":
                val = lo
            else:
                val = hi
            setattr(st, fname, val)
        return st

    def _stage_host(self, name, host, original, stored):
        nbytes = host.nbytes
        hit = residency.lookup(host.ctypes.data, nbytes) if (residency.active() and original is host) else None
        if hit is None and 0 < nbytes <= _SMALL_SLOT_BYTES and self.capture is None and original is host:
            # the one-element buffers of `shared()` scalars, and other arrays of a few bytes: through a page-locked
            # slot that owns device memory - a small DMA each way, nothing allocated, nothing moved through the
            # driver's path for pageable memory (which costs some 50 us per copy whatever its size)
            for k, (slot, host0, stored0, name0) in enumerate(self.small):
                if host0.ctypes.data == host.ctypes.data and host0.nbytes == nbytes:
                    # the same array under a second name: one device copy serves both
                    self.small[k] = (slot, host0, stored0 or stored, name0)
                    self.aliases.append((name, slot[1], nbytes, stored))
                    break
            else:
                slot = _take_small_slot(self.device)
                C.memmove(slot[0], host.ctypes.data, nbytes)
                rt.memcpy_h2d_async(slot[1], slot[0], nbytes, self.stream)
                self.small.append((slot, host, stored, name))
            self.ptr[name] = slot[1]
            self.strides[name] = [s // host.itemsize for s in host.strides]
            return
        if hit is not None:
            # the array (or the array this is a view of) has a standing mirror in HBM
            m, off = hit
            if self.capture is not None and (not m.resident or m.host_dirty):
                self._no_capture(name, "it is not resident on the device (use `with appy.resident(...)` around the "
                                       "capture and the replays)" if not m.resident else
                                       "its host copy has changed (appy.invalidate) and would be uploaded per launch")
            if m.resident:
                if m.host_dirty:
                    m.upload(self.stream)
            elif nbytes and not (stored and self.loop.overwrites(name, self.lo, self.hi, self.env, host.shape)):
                # (from page-locked memory the upload is queued, not waited for: `finish` waits for the stream before
                #  the caller can touch the host bytes again)
                (rt.memcpy_h2d_async if m.pinned else rt.memcpy_h2d)(m.device_ptr() + off, host.ctypes.data, nbytes, self.stream)
            dptr = m.device_ptr() + off
            self.mirrored.append((m, dptr, host, stored, name))
            self.ptr[name] = dptr
            self.strides[name] = [s // host.itemsize for s in host.strides]
            return
        self._no_capture(name, "it is a host array that would be copied per launch (use GPU tensors, or NumPy "
                               "arrays inside `with appy.resident(...)`; `shared()` scalars cannot be captured)")
        skip_upload = bool(stored and self.loop.overwrites(name, self.lo, self.hi, self.env, host.shape))
        key = (host.ctypes.data, nbytes, host.strides, host.dtype.str)
        twin = self.staged_twice.get(key) if nbytes else None
        if twin is not None:
            # the same host array under a second name: one device copy serves both, so that what
            # the kernel stores through one name is what it loads through the other
            k, uploaded = twin
            dptr, host0, original0, stored0, name0 = self.temps[k]
            if not uploaded and not skip_upload:
                rt.memcpy_h2d(dptr, host.ctypes.data, nbytes, self.stream)
                self.staged_twice[key] = (k, True)
            self.temps[k] = (dptr, host0, original0, stored0 or stored, name0)
            self.aliases.append((name, dptr, nbytes, stored))
        else:
            dptr = rt.malloc(max(nbytes, 1))
            if nbytes and not skip_upload:
                rt.memcpy_h2d(dptr, host.ctypes.data, nbytes, self.stream)
            self.staged_twice[key] = (len(self.temps), not skip_upload)
            self.temps.append((dptr, host, original, stored, name))
        self.ptr[name] = dptr
        self.strides[name] = [s // host.itemsize for s in host.strides]

    def replayable(self) -> bool:
        """True if nothing but the kernel launch happens when this call is repeated."""
        return not (self.temps or self.mirrored or self.aliases or self.keepalive_copies or self.oob or self.capture is not None
                    or self.second is not None or (self.sequence is not None and self.seq_replay is None))

    def _no_capture(self, name, why):
        if self.capture is not None:
            raise RuntimeError(f"{self.loop.loop_name} cannot be captured into a graph: argument `{name}`: {why}")

    def function(self):
        return self.kernel.function(self.device)

    def launch_only(self):
        if self.sequence is not None:
            # the kernels share the loop's scratch buffer for this stream: queued as one run
            with self.loop._lock:
                for kernel, args, grid, block in self.sequence:
                    if kernel is None:
                        rt.memset_async(args[0], 0, args[1], self.stream)
                    else:
                        rt.launch(kernel.function(self.device), grid, block, args, self.stream)
        elif self.second is None:
            rt.launch(self.function(), self.grid, self.block, self.args, self.stream)
        else:
            # both kernels share the loop's scratch buffer for this stream: they are queued as a
            # pair, so that another thread's pair for the same loop cannot come between them
            fin, args, grid, block = self.second
            with self.loop._lock:
                rt.launch(self.function(), self.grid, self.block, self.args, self.stream)
                rt.launch(fin.function(self.device), grid, block, args, self.stream)
        g = self.capture
        if g is not None:
            g.launches += 1
            g.keepalive.extend(self.keepalive)
            for e in self.stored_extents:
                if e not in g.stored_extents:       # (a loop recorded many times over the same arrays)
                    g.stored_extents.append(e)
            for m, _dptr, _host, stored, _name in self.mirrored:
                if m not in g.used_mirrors:
                    g.used_mirrors.append(m)
                if stored and m not in g.stored_mirrors:
                    g.stored_mirrors.append(m)

    def time_kernel(self, warmup=3, reps=20) -> float:
        """Mean milliseconds per launch (HIP events on the launch stream); for a launch made of
        several kernels, of the whole run of them."""
        if self.sequence is None and self.second is None:
            return rt.launch_timed(self.function(), self.grid, self.block, self.args, self.stream, warmup=warmup, reps=reps)
        for _ in range(warmup):
            self.launch_only()
        e0, e1 = rt.Event(), rt.Event()
        e0.record(self.stream)
        for _ in range(reps):
            self.launch_only()
        e1.record(self.stream)
        e1.synchronize()
        return e0.elapsed_ms(e1) / reps

    def _check_report(self):
        if not self.oob:
            return
        word = C.c_int32(0)
        try:
            rt.memcpy_d2h(C.addressof(word), self.oob, 4, self.stream)
        finally:
            rt.free(self.oob)
            self.oob = 0
        if word.value:
            sites = self.kernel.src.sites
            text = sites[word.value - 1] if 0 < word.value <= len(sites) else "?"
            raise IndexError(f"{self.loop.loop_name}: `{text}` was indexed outside the array "
                             f"(negative indices other than literals count as outside)")

    def finish(self):
        """Copy stored host arrays back and release staging buffers."""
        try:
            self._check_report()
            for dptr, host, original, stored, _name in self.temps:
                if stored and host.nbytes:
                    rt.memcpy_d2h(host.ctypes.data, dptr, host.nbytes, self.stream)
                    if isinstance(original, tuple):          # non-contiguous CPU tensor
                        _, dst, src = original
                        dst.copy_(src)
                    elif original is not host and is_numpy_array(original):
                        original[...] = host
            waited = bool(self.temps)
            for slot, host, stored, _name in self.small:
                if stored:
                    rt.memcpy_d2h(slot[0], slot[1], host.nbytes, self.stream)       # one DMA; waits for the stream
                    C.memmove(host.ctypes.data, slot[0], host.nbytes)
                    waited = True
            if self.small and not waited:
                rt.sync(self.stream)        # the uploads must have left the slots before they are used again
                waited = True
            for m, dptr, host, stored, _name in self.mirrored:
                if m.resident:
                    m.stream, m.busy = self.stream, True
                if not stored:
                    continue
                if m.resident:
                    m.device_dirty = True       # downloaded on request, not per launch
                    m.stream = self.stream
                elif host.nbytes:
                    rt.memcpy_d2h(host.ctypes.data, dptr, host.nbytes, self.stream)
                    waited = True
            if self.mirrored and not waited and any(not m.resident for m, *_ in self.mirrored):
                waited = True    # uploads from pinned memory must have left the host buffer
            if waited:
                rt.sync(self.stream)
            for item in self.keepalive:
                if isinstance(item, tuple) and item[0] == "copy_back":
                    item[1].copy_(item[2])
        finally:
            for dptr, *_ in self.temps:
                rt.free(dptr)
            self.temps = []
            self.mirrored = []
            self.keepalive = []
            self._return_small_slots(wait=False)

    def _return_small_slots(self, wait):
        if self.keep_small and not wait:
            self.small_kept, self.small = self.small, []
            return
        slots, self.small = [entry[0] for entry in self.small], []
        if not slots:
            return
        if wait:
            try:
                rt.sync(self.stream)
            except Exception:
                pass
        with _small_lock:
            _small_free.setdefault(self.device, []).extend(slots)

    def run(self):
        try:
            self.launch_only()
        except Exception:
            for dptr, *_ in self.temps:
                rt.free(dptr)
            self.temps = []
            self._return_small_slots(wait=True)
            if self.oob:
                rt.free(self.oob)
                self.oob = 0
            raise
        self.finish()


def _overlaps(extents) -> bool:
    """True if a stored array shares bytes with any other array argument."""
    for i, (_n1, p1, s1, st1) in enumerate(extents):
        for j, (_n2, p2, s2, st2) in enumerate(extents):
            if i >= j or not (st1 or st2):
                continue
            if p1 < p2 + s2 and p2 < p1 + s1:
                return True
    return False


def _copy(node):
    import copy

    return copy.deepcopy(node)


# ---------------------------------------------------------------------------
# entry point
# ---------------------------------------------------------------------------
def codegen(loop_source, loop_name, val_map, options):
    key = (loop_source, loop_name, _signature(val_map), options.get("hip_spec") and repr(options.get("hip_spec")),
           options.get("hip_max_blocks"), bool(options.get("check_bounds")), bool(options.get("hip_bins", True)),
           bool(options.get("hip_group", True)), options.get("hip_group_rows"), bool(options.get("hip_hints", True)),
           options.get("hip_reuse", True), options.get("hip_plan_split"), options.get("hip_plan_grid"), options.get("fn_name"))
    # `clear_cache=True` regenerates the loop on every call instead of using the cached kernel
    # (reference: appy/backends/metal/codegen.py:23)
    fresh = bool(options.get("clear_cache"))
    hit = None if fresh else code_cache.get(key)
    if hit is not None:
        return hit
    with _cache_lock:
        hit = None if fresh else code_cache.get(key)
        if hit is not None:
            return hit
        stale = code_cache.get(key)
        if stale is not None:
            stale[0].release()          # `clear_cache`: the loop object of the previous call goes away
        f = CompiledLoop(loop_source, loop_name, val_map, options)
        if options.get("dry_run"):
            f.kernels[f.default_spec].code      # nothing will be launched: compile now, so that errors surface
        code_cache[key] = (f, f.code_src)
    if options.get("dump_code"):
        print(f"--- Dumped code for loop {loop_name} ---")
        print(f.code_src)
        print(f"--- End of dumped code for loop {loop_name} ---")
    if options.get("dump_code_to_file"):
        with open(options["dump_code_to_file"], "w") as fh:
            fh.write(f.code_src)
    return f, f.code_src
