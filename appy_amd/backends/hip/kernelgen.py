"""Loop IR -> HIP C++ kernel text for gfx950.

Two execution shapes cover every annotated loop:

``flat``
    ``#pragma parallel for simd`` (and parallel loops without inner ``simd``
    loops): one lane per iteration.  Lanes take V consecutive iterations so
    that ``X[i]`` accesses become one 128-bit load/store; a workgroup walks
    tiles of ``BLOCK*U*V`` iterations with all loads of a tile issued before
    its arithmetic.  Replaces the reference's 256-wide masked Triton program
    per 256 iterations (reference tree: appy/backends/triton/passes/
    block_loop.py:111-149, device_passes/remove_loop_head.py:20-48).

``team``
    ``#pragma parallel for`` whose body holds ``#pragma simd`` loops: one
    team of W adjacent lanes (W = 1..64, a power of two) per outer iteration.
    Statements outside ``simd`` loops run on every lane of the team with
    identical values and their stores are issued by lane 0; ``simd`` loops are
    spread over the lanes (V consecutive iterations per lane where the
    accesses allow) and their reductions end with a DPP/shuffle butterfly over
    the team.  Replaces the reference's one-program-per-outer-iteration
    mapping with masked 256-wide chunks (same passes of the reference).

Reductions of the parallel loop itself (``shared`` scalars, detected as in
appy/frontend/reduction_detection.py:76-104 of the reference) are kept in a
register per lane, reduced over the wavefront with DPP moves, over the
workgroup through LDS, and combined into memory with one atomic per
workgroup - instead of the reference's one atomic per 256 iterations
(device_passes/rewrite_par_reduce_to_atomics.py:18-55).

What a loop allows is worked out in ``loop_analysis.py``; the bodies of the kernels for CSR rows
live in ``csr_kernels.py`` (forms that read the raw arrays) and ``row_plan_kernels.py`` (forms that
run a kept order of the elements), both mixed into :class:`KernelBuilder`.
"""
from __future__ import annotations

import ast
import ctypes as C
from dataclasses import dataclass, field

from ...frontend import loop_ir
from . import dtypes as T
from .csr_kernels import CsrKernels
from .dtypes import Ty
from .exprs import ArrayParam, ExprEmitter, cast, cname, truth
from .loop_analysis import (LoopAnalysis, OuterReduction, Unsupported, _elts, _uses_name, _var_offset,  # noqa: F401
                            guarded_nodes, skips_iterations)  # guarded_nodes is part of this module's interface
from .row_plan_kernels import RowPlanKernels

# accessors of the components of a vector register (the first four also have the usual names)
_COMPONENTS = ["x", "y", "z", "w"] + [f"s{d:x}" for d in range(4, 16)]

_OPS = {"+": "appy::OpAdd", "*": "appy::OpMul", "max": "appy::OpMax", "min": "appy::OpMin"}

_CTYPES = {
    "bool": C.c_bool, "int8": C.c_int8, "uint8": C.c_uint8, "int16": C.c_int16, "uint16": C.c_uint16,
    "int32": C.c_int32, "uint32": C.c_uint32, "int64": C.c_int64, "uint64": C.c_uint64,
    "float32": C.c_float, "float64": C.c_double,
}


@dataclass(frozen=True)
class Spec:
    """Launch-time selectable shape of a kernel."""

    kind: str            # 'flat' | 'team' | 'strip'
    block: int = 256     # threads per workgroup
    vec: int = 1         # consecutive iterations per lane (V)
    unroll: int = 1      # vectors per lane and tile (U), flat only
    width: int = 1       # lanes per team (W), team only
    restrict: bool = True
    stream_loads: bool = False   # non-temporal loads for data that is read once
    extent: int = 0      # compile-time extent of row accumulators (team only; 0 = none)
    stream_stores: bool = False  # non-temporal vector stores
    lds_tile: int = 0    # elements of a row-invariant operand staged in LDS per step (team only; 0 = off)
    checked: bool = False        # every subscript is compared with the extents; violations are reported
    hoist_guarded: bool = True   # flat only: loads the source guards with a condition may be issued
                                 # unconditionally (the host has checked that they stay inside their arrays)
    phase: int = 0               # strips and workgroup teams: 1 = the shared-out loop over one part of its range,
                                 # partial results to a scratch buffer (the grid holds several workgroups per strip
                                 # or row), 2 = the rest of the body on those partial results; 0 = one kernel
    row_steps: int = 0           # team only: every lane takes exactly this many vector steps of the rows that several
                                 # simd loops of one iteration read; those rows stay in registers between the loops
    collapse: bool = False       # team only: the parallel loop and the sequential loop that is its whole body
                                 # run as one iteration space (the analysis has shown the inner iterations independent)
    rows: str = ""               # team only, rows binned by the trip count of their simd loop: 'mixed' = the rows of the
                                 # base class in their natural order plus the listed rows of the other classes, the
                                 # team width chosen per wavefront at run time; 'list' = the rows of one list
    parts: int = 0               # with rows='list' and a phase: the simd loop of a row runs in this many parts whose
                                 # boundaries a planning kernel has written (column stripes of a gathered operand),
                                 # one part per workgroup slot, the stripes dealt to the XCDs by workgroup number
    aux: str = ""                # 'bins' = the kernel that sorts rows into classes, 'plan' = the kernel that finds
                                 # the part boundaries of listed rows; 'group' = the kernel that groups the elements
                                 # of every block of rows by the stripe of the gathered operand they read, 'cells' =
                                 # the kernel that runs those groups (`parts` stripes, dealt to the XCDs by workgroup
                                 # number); '' = a kernel that runs the loop body
    block_rows: int = 0          # with 'group' and 'cells': rows per block (256, 512 or 1024; more where rows are short,
                                 # so that a cell still holds a few hundred elements)
    skip_long: bool = False      # with 'group' and the kernel that adds the sums of its cells: rows whose simd loop is longer
                                 # than a limit given at the launch are passed over (they run in planned parts)
                                 # 'rkeys' = the kernel that turns the elements of `block_rows` rows per wavefront into the
                                 # (key, value) pairs a row plan is built from, 'xcells' = the kernel that runs a row plan
                                 # (`parts` column ranges, `unroll` x 1024 elements per tile)
    guard: int = 0               # 1 = the kernel returns at once when the grouping kernel of this launch has refused
                                 # its input (row ranges that do not follow one another: a flag in device memory),
                                 # 2 = when it has not

    def __post_init__(self):
        def pow2(n):
            return n >= 1 and (n & (n - 1)) == 0

        if self.kind not in ("flat", "team", "strip"):
            raise ValueError(f"kernel shape must be 'flat', 'team' or 'strip', got {self.kind!r}")
        if self.block % 64 or not 64 <= self.block <= 1024:
            raise ValueError(f"workgroup size must be a multiple of 64 up to 1024, got {self.block}")
        if self.vec not in (1, 2, 4, 8, 16):
            raise ValueError(f"vector width must be 1, 2, 4, 8 or 16, got {self.vec}")
        if not 1 <= self.unroll <= 8:
            raise ValueError(f"unroll factor must be 1..8, got {self.unroll}")
        if not pow2(self.width) or (self.width > 64 and self.width != self.block):
            raise ValueError(f"team width must be a power of two up to 64, or the whole workgroup, got {self.width}")
        if self.checked and (self.vec != 1 or self.unroll != 1 or self.extent or self.lds_tile):
            raise ValueError("a bounds-checked kernel takes one element per access (vec = unroll = 1, no row extent, no LDS tile)")
        if self.phase not in (0, 1, 2) or (self.phase and not (
                self.kind == "strip" or (self.kind == "team" and (self.width in (64, self.block) or self.rows == "list"
                                                                 or (self.phase == 2 and self.guard == 1))
                                         and not self.extent and not self.lds_tile and not self.collapse))):
            raise ValueError("only strip kernels, teams of a whole wavefront or workgroup, and teams over listed rows "
                             "run in two phases")
        if self.rows not in ("", "mixed", "list") or self.aux not in ("", "bins", "plan", "group", "cells", "rkeys", "xcells"):
            raise ValueError(f"unknown row source {self.rows!r} / auxiliary kernel {self.aux!r}")
        if (self.rows or self.aux) and (self.kind != "team" or self.extent or self.lds_tile or self.collapse
                                        or self.row_steps or self.checked or (self.width > 64 and self.aux != "xcells")):
            raise ValueError("rows are binned for plain team kernels only (teams inside a wavefront)")
        if self.aux == "rkeys":
            if self.rows or self.phase or self.parts or self.width != 64 or self.block != 256 or self.block_rows != 256:
                raise ValueError("the kernel that writes the pairs of a row plan takes blocks of 256 rows, one per wavefront")
        elif self.aux == "xcells":
            if self.rows or self.phase or self.parts != 8 or self.block != 1024 or self.unroll not in (4, 6) or self.block_rows:
                raise ValueError("a row plan runs in workgroups of 1024 lanes, 8 column ranges, tiles of 4096 or 6144 elements")
        elif self.aux in ("group", "cells"):
            if (self.rows or self.phase or self.parts not in (8, 16) or self.width != 64 or self.block != 256
                    or self.block_rows not in (256, 512, 1024)):
                raise ValueError("elements are grouped by 8 or 16 stripes, one wavefront per block of 256, 512 or 1024 rows, "
                                 "four per workgroup")
        elif self.block_rows:
            raise ValueError("only the kernels over grouped elements work on blocks of rows")
        elif self.parts and (self.rows != "list" or not (self.phase or self.aux == "plan") or self.parts % 8
                             or not 8 <= self.parts <= 64):
            raise ValueError("planned parts belong to the two-phase kernels over listed rows (8, 16, ... 64 parts)")
        if self.skip_long and not (self.aux == "group" or (self.phase == 2 and self.guard == 1 and not self.rows)):
            raise ValueError("only the grouping kernel and the kernel that adds the sums of its cells pass over long rows")
        if self.guard not in (0, 1, 2) or (self.guard and self.kind != "team"):
            raise ValueError("only team kernels wait on the verdict of a grouping kernel (guard 1 or 2)")
        if self.aux == "plan" and (self.rows != "list" or not self.parts or self.width < self.parts):
            raise ValueError("the planning kernel takes listed rows, with one lane per part at least")
        if self.row_steps and (self.kind != "team" or self.phase or self.extent or self.lds_tile or self.vec < 2
                               or not 1 <= self.row_steps <= 16 or self.checked):
            raise ValueError("rows are kept in registers by plain team kernels only, for 1 to 16 vector steps per lane")
        if self.collapse and (self.kind != "team" or self.lds_tile):
            raise ValueError("only team kernels without an LDS tile collapse their two outer loops")
        if self.extent < 0 or self.lds_tile < 0 or self.lds_tile % 4 or self.lds_tile > 16384:
            raise ValueError("row extent / LDS tile out of range (tile: multiple of 4, at most 16384 elements)")

    def tag(self) -> str:
        return (f"{self.kind}_b{self.block}_v{self.vec}_u{self.unroll}_w{self.width}"
                f"{'_r' if self.restrict else ''}{'_nt' if self.stream_loads else ''}"
                f"{'_e' + str(self.extent) if self.extent else ''}{'_nts' if self.stream_stores else ''}"
                f"{'_lds' + str(self.lds_tile) if self.lds_tile else ''}{'' if self.hoist_guarded else '_g'}{'_chk' if self.checked else ''}{'_c2' if self.collapse else ''}{'_p' + str(self.phase) if self.phase else ''}{'_rc' + str(self.row_steps) if self.row_steps else ''}"
                f"{'_' + self.rows if self.rows else ''}{'_s' + str(self.parts) if self.parts else ''}{'_' + self.aux if self.aux else ''}"
                f"{'_R' + str(self.block_rows) if self.block_rows else ''}{'_sl' if self.skip_long else ''}{'_if' + str(self.guard) if self.guard else ''}")


@dataclass
class Param:
    cname: str
    ctype_decl: str      # C++ parameter declaration
    ctype: object        # ctypes type
    role: str            # 'array' | 'stride' | 'scalar' | 'shape' | 'lo' | 'hi'
    source: str = ""     # python-side name (array / scalar name)
    dim: int = 0


@dataclass
class KernelSource:
    name: str
    text: str
    params: list
    spec: Spec
    reductions: list
    stored_arrays: list
    bound_checks: list   # (array, dim, offset) accesses indexed by the parallel loop variable
    lane_step_bytes: int = 0   # bytes one lane moves per vector step of a flat loop
    sites: list = field(default_factory=list)   # checked kernels: source text of every subscript, by site number


class KernelBuilder(CsrKernels, RowPlanKernels):
    def __init__(self, analysis: LoopAnalysis, kernel_name: str, module_names, spec: Spec):
        self.a = analysis
        self.name = kernel_name
        self.spec = spec
        self.ex = ExprEmitter(analysis.arrays, analysis.scalars, module_names)
        self.ex.checked = spec.checked
        self.lines = []
        self.ind = 1
        self.mode = "lane"
        self.partials = {}        # reduction variable -> partial register, inside a spread simd loop
        self.bounds_vary = False  # inside a spread loop whose bounds differ between outer iterations
        self.lds_plan = None      # (spread loop node, [ArrayParam]) staged through LDS, or None
        self.store_subst = {}     # unparsed subscript -> (lvalue code, Ty)
        self.dirty = False
        self.counter = 0
        self.seq_depth = 0        # sequential loops (for / while) around the current statement
        self.skippable = False    # directly inside an iteration body that `continue` may leave
        self.shadowed = [n for n in analysis.assigned if n in analysis.scalars]
        self.red_by_key = {r.key: r for r in analysis.outer_reductions}

    # ---- text helpers ------------------------------------------------------------
    def w(self, line=""):
        self.lines.append("    " * self.ind + line if line else "")

    def fresh(self, stem):
        self.counter += 1
        return f"__{stem}{self.counter}"

    # ---- types of locals ---------------------------------------------------------------
    def set_local(self, name, ty: Ty):
        old = self.ex.locals.get(name)
        new = T.join(old, ty)
        if new != old:
            self.ex.locals[name] = new
            self.dirty = True

    # ---- statements ---------------------------------------------------------------
    def block(self, stmts):
        i = 0
        while i < len(stmts):
            if self.mode == "team" and self.spec.kind == "team":
                used = self.row_accumulate(stmts, i) if self.spec.extent else 0
                if used:
                    i += used
                    continue
                if self.interchange_row_update(stmts[i]):
                    i += 1
                    continue
            self.stmt(stmts[i])
            i += 1

    def iteration_body(self, stmts):
        """One iteration of a parallel or simd loop."""
        if not skips_iterations(stmts):
            return self.block(stmts)
        saved, self.skippable = self.skippable, True
        saved_depth, self.seq_depth = self.seq_depth, 0
        self.w("do {")
        self.ind += 1
        self.block(stmts)
        self.ind -= 1
        self.w("} while (0);")
        self.skippable, self.seq_depth = saved, saved_depth

    def stmt(self, st):
        if isinstance(st, ast.Assign):
            return self.assign(st)
        if isinstance(st, ast.For):
            return self.for_(st)
        if isinstance(st, ast.If):
            return self.if_(st)
        if isinstance(st, ast.While):
            return self.while_(st)
        if isinstance(st, (ast.Break, ast.Continue)):
            if self.seq_depth > 0:
                self.w("break;" if isinstance(st, ast.Break) else "continue;")
            elif isinstance(st, ast.Continue) and self.skippable:
                # the iterations of parallel and simd loops are dealt to lanes, tiles and vector
                # components, each in a `do { } while (0)` block of its own: leaving it ends the iteration
                self.w("break;")
            else:
                raise Unsupported("`break` is only supported inside a sequential loop of the kernel "
                                  "(the iterations of a parallel or simd loop do not run in order)")
            return
        if isinstance(st, ast.Pass):
            return
        if isinstance(st, ast.Expr) and isinstance(st.value, ast.Constant):
            return  # docstring-like
        raise Unsupported(f"Statement not supported in a kernel: {ast.unparse(st)}")

    def if_(self, st: ast.If):
        c, t = self.ex.emit(st.test)
        self.w(f"if ({truth(c, t)}) {{")
        self.ind += 1
        self.block(st.body)
        self.ind -= 1
        if st.orelse:
            self.w("} else {")
            self.ind += 1
            self.block(st.orelse)
            self.ind -= 1
        self.w("}")

    def while_(self, st: ast.While):
        if st.orelse:
            raise Unsupported("`while ... else` is not supported in a kernel")
        # the condition is evaluated again after every pass: as the last statement of an
        # endless loop, so that it may hold loads and calls like any other expression
        self.w("while (true) {")
        self.ind += 1
        c, t = self.ex.emit(st.test)
        self.w(f"if (!({truth(c, t)})) break;")
        self.seq_depth += 1
        self.block(st.body)
        self.seq_depth -= 1
        self.ind -= 1
        self.w("}")

    def assign(self, st: ast.Assign):
        tgt = st.targets[0]
        red_op = getattr(st, "reduce", None)
        if isinstance(tgt, ast.Name):
            name = tgt.id
            if red_op and name in self.partials:
                oc, ot = self.ex.emit(loop_ir.reduction_operand(st))
                p, pty = self.partials[name]
                # the variable takes the type NumPy gives `name (op) operand`
                vty = self.ex.locals.get(name, pty)
                self.set_local(name, T.promote(vty, ot) if red_op in "+*" else T.join(vty, ot))
                self.w(f"{p} = {_OPS[red_op]}::f<{pty.c}>({p}, {cast(oc, ot, pty)});")
                return
            vc, vt = self.ex.emit(st.value)
            self.set_local(name, vt)
            lt = self.ex.locals[name]
            self.w(f"{cname(name)} = {cast(vc, vt, lt)};")
            return
        if not (isinstance(tgt, ast.Subscript) and isinstance(tgt.value, ast.Name)):
            raise Unsupported(f"Assignment target not supported in a kernel: {ast.unparse(tgt)}")
        key = ast.unparse(tgt)
        if red_op and key in self.red_by_key and self.red_by_key[key].op in (
                red_op, {"+": "max", "*": "min"}.get(red_op) if self.red_by_key[key].elem_ty.is_bool else red_op):
            r = self.red_by_key[key]
            oc, ot = self.ex.emit(loop_ir.reduction_operand(st))
            if r.elem_ty.is_int and ot.is_float:
                raise TypeError(
                    f"`{key}` is an integer ({r.elem_ty.name}) but accumulates {ot.name} values, which would be "
                    f"truncated one by one: start the shared scalar as a float (`0.0`)")
            operand = f"(int)({truth(oc, ot)})" if r.elem_ty.is_bool else cast(oc, ot, r.ty)
            upd = f"{r.acc} = {_OPS[r.op]}::f<{r.ty.c}>({r.acc}, {operand});"
            if self.mode == "team":
                self.w(f"if ({self._leader()}) {{ {upd} }}")
            else:
                self.w(upd)
            return
        arr = self.a.arrays.get(tgt.value.id)
        if arr is None:
            raise Unsupported(f"`{tgt.value.id}` is subscripted but is not an array argument")
        shared_update = self._shared_update(st)
        if shared_update is not None:
            return self._atomic_update(st, arr, *shared_update)
        vc, vt = self.ex.emit(st.value)
        if key in self.store_subst:
            lv, _lty = self.store_subst[key]
            self.w(f"{lv} = {self._store_value(vc, vt, arr)};")
            self.ex.load_subst[key] = ((f"({lv} != 0)" if arr.ty.is_bool else lv), arr.ty)
            return
        if self.spec.checked:
            idx = self.ex.index_code(arr, tgt, check=False)
            site = self.ex.site(tgt)
            store = (f"if ({self.ex.inside_code(arr, tgt)}) {cname(arr.name)}[{idx}] = {self._store_value(vc, vt, arr)}; "
                     f"else appy::report(__oob, {site});")
        else:
            idx = self.ex.index_code(arr, tgt)
            store = f"{cname(arr.name)}[{idx}] = {self._store_value(vc, vt, arr)};"
        if self.mode == "team":
            self.w(f"if ({self._leader()}) {{ {store} }}")
        else:
            self.w(store)
        # a later read of the same element in this iteration goes to memory again
        self.ex.load_subst.pop(key, None)

    def _shared_update(self, st: ast.Assign):
        """``X[idx] = X[idx] op e`` on an element that other iterations of the
        parallel loop may update as well (no index is the parallel variable plus a
        constant: ``hist[bin[i]] += 1``, ``colsum[j] += A[i, j]``): returns
        ``(op, e)`` - such an update has to be atomic.  None for updates of
        elements that belong to the iteration, and for plain stores."""
        tgt = st.targets[0]
        if any(_var_offset(e, self.a.var) is not None for e in _elts(tgt)):
            return None
        key = ast.unparse(tgt)
        val = st.value
        if isinstance(val, ast.BinOp) and isinstance(val.op, (ast.Add, ast.Sub, ast.Mult)):
            if ast.unparse(val.left) == key:
                other = val.right
            elif ast.unparse(val.right) == key and not isinstance(val.op, ast.Sub):
                other = val.left
            else:
                return None
            op = {ast.Add: "+", ast.Sub: "-", ast.Mult: "*"}[type(val.op)]
        elif (isinstance(val, ast.Call) and isinstance(val.func, ast.Name) and val.func.id in ("max", "min")
              and len(val.args) == 2 and any(ast.unparse(a) == key for a in val.args)):
            other = val.args[1] if ast.unparse(val.args[0]) == key else val.args[0]
            op = val.func.id
        else:
            return None
        if any(isinstance(n, ast.Subscript) and ast.unparse(n) == key for n in ast.walk(other)):
            return None
        return op, other

    def _atomic_update(self, st, arr: ArrayParam, op: str, other):
        oc, ot = self.ex.emit(other)
        if arr.ty.is_bool:
            op = {"+": "max", "*": "min"}.get(op, op)
            val = f"(unsigned char)({truth(oc, ot)})"
        else:
            val = cast(oc, ot, arr.ty)
        if op == "-":
            op, val = "+", f"(-{val})"
        tgt = st.targets[0]
        if self.spec.checked:
            idx = self.ex.index_code(arr, tgt, check=False)
            guard = f"if ({self.ex.inside_code(arr, tgt)}) "
            tail = f" else appy::report(__oob, {self.ex.site(tgt)});"
        else:
            idx, guard, tail = self.ex.index_code(arr, tgt), "", ""
        arr.loaded = True
        upd = f"{guard}appy::atomic_combine<{_OPS[op]}, {arr.elem_c}>::run(&{cname(arr.name)}[{idx}], {val});{tail}"
        if self.mode == "team":
            self.w(f"if ({self._leader()}) {{ {upd} }}")
        else:
            self.w(upd)
        self.ex.load_subst.pop(ast.unparse(tgt), None)

    def _store_value(self, vc, vt, arr: ArrayParam):
        if arr.ty.is_bool:
            return f"(unsigned char)({truth(vc, vt)})"
        return cast(vc, vt, arr.ty)

    # ---- loops ---------------------------------------------------------------------
    def _range_args(self, st: ast.For):
        it = st.iter
        if not (isinstance(it, ast.Call) and isinstance(it.func, ast.Name) and it.func.id == "range"
                and len(it.args) == 3):
            raise Unsupported(f"Loops in a kernel iterate over range(...): {ast.unparse(it)}")
        lc, lt = self.ex.emit(it.args[0])
        hc, ht = self.ex.emit(it.args[1])
        return cast(lc, lt, T.I64), cast(hc, ht, T.I64)

    def for_(self, st: ast.For):
        pragma = getattr(st, "pragma", None) or {}
        if self.spec.kind == "strip":
            if self.mode == "team" and id(st) in self.a.strip:
                return self.strip_spread_loop(st)
        elif self.mode == "team" and "simd" in pragma:
            return self.spread_loop(st)
        var = st.target.id
        lo, hi = self._range_args(st)
        self.ex.locals[var] = T.WEAK_INT
        hi_v = self.fresh("hi")
        self.w(f"const appy::i64 {hi_v} = {hi};")
        innermost = not any(isinstance(n, (ast.For, ast.While)) for b in st.body for n in ast.walk(b))
        if self.mode == "lane" and innermost and sum(1 for b in st.body for _n in ast.walk(b) if isinstance(_n, ast.stmt)) <= 8:
            # a loop one lane runs by itself: its loads do not depend on one another, so eight
            # iterations' worth are put in flight together (a running sum down the columns of
            # 65536 x 1024 floats: 380 ns per iteration as written, 64 ns unrolled)
            self.w("#pragma unroll 8")
        self.w(f"for (appy::i64 {cname(var)} = {lo}; {cname(var)} < {hi_v}; ++{cname(var)}) {{")
        self.ind += 1
        self.seq_depth += 1
        self.block(st.body)
        self.seq_depth -= 1
        self.ind -= 1
        self.w("}")

    def _vector_accesses(self, body, var: str, hoist_guarded: bool = False):
        """Loads ``X[.., var+c]`` (any depth) and unconditional top-level
        stores ``X[.., var+c] = e`` of a loop body that can move V elements at
        once.  Returns (loads, stores): lists of (key, array, subscript).  Loads
        the program guards with a condition are only taken when the caller
        knows them to be in bounds (``hoist_guarded``)."""
        loads, stores = {}, {}
        blocked = set()
        skips = skips_iterations(body)      # then every store after the `continue` is conditional
        guarded = set() if hoist_guarded else guarded_nodes(body)
        in_place = {}           # guarded loads that stay where the program has them: key -> array
        inner_vars = {n.target.id for s in body for n in ast.walk(s) if isinstance(n, ast.For)}
        for s in body:
            for n in ast.walk(s):
                if not (isinstance(n, ast.Subscript) and isinstance(n.value, ast.Name)
                        and n.value.id in self.a.arrays):
                    continue
                arr = self.a.arrays[n.value.id]
                el = _elts(n)
                if len(el) != arr.ndim or any(isinstance(e, ast.Slice) for e in el):
                    continue
                off = _var_offset(el[-1], var)
                ok = off is not None and not any(_uses_name(e, var) for e in el[:-1])
                # indices that depend on variables of loops nested in the body change per inner iteration
                ok = ok and not any(_uses_name(e, v) for e in el for v in inner_vars)
                # indices may only use values that exist before the body starts
                ok = ok and not any(_uses_name(e, v) for e in el[:-1] for v in self._assigned_in(body))
                key = ast.unparse(n)
                if isinstance(n.ctx, ast.Load):
                    if id(n) in guarded:
                        in_place[key] = arr
                    elif ok:
                        loads[key] = (arr, n)
                else:
                    top = any(isinstance(t, ast.Assign) and t.targets[0] is n for t in body)
                    owner = next((t for t in body if isinstance(t, ast.Assign) and t.targets[0] is n), None)
                    if owner is not None and self._shared_update(owner) is not None:
                        blocked.add(arr.name)       # updated atomically, element by element
                    elif ok and top and not skips:
                        stores[key] = (arr, n)
                    else:
                        blocked.add(arr.name)
        # an array written through a non-vector path must not be cached in registers
        for key in [k for k, (arr, _) in loads.items() if arr.name in blocked]:
            del loads[key]
        for key in [k for k, (arr, _) in stores.items() if arr.name in blocked]:
            del stores[key]
        # a vector store to an array that is also read at another offset would reorder accesses
        for key, (arr, _) in list(stores.items()):
            if (any(a2.name == arr.name and k2 != key for k2, (a2, _) in loads.items())
                    or any(a2.name == arr.name and k2 != key for k2, a2 in in_place.items())):
                del stores[key]
                loads = {k: v for k, v in loads.items() if v[0].name != arr.name}
        return loads, stores

    def _assigned_in(self, body):
        names = set()
        for s in body:
            for n in ast.walk(s):
                if isinstance(n, ast.Assign) and isinstance(n.targets[0], ast.Name):
                    names.add(n.targets[0].id)
        return names

    def _addr(self, arr: ArrayParam, sub: ast.Subscript, var: str, base_code: str) -> str:
        """Address of ``sub`` with ``var`` replaced by ``base_code``."""
        saved = self.ex.locals.get(var)
        self.ex.locals[var] = T.WEAK_INT
        try:
            repl = _Rename(var, "__vbase").visit(_copy(sub))
            self.ex.locals["__vbase"] = T.WEAK_INT
            idx = self.ex.index_code(arr, repl)
        finally:
            self.ex.locals.pop("__vbase", None)
            if saved is None:
                self.ex.locals.pop(var, None)
            else:
                self.ex.locals[var] = saved
        return f"{cname(arr.name)} + ({idx.replace('__vbase', base_code)})"

    def _team_total(self, op: str, ty: Ty, partial: str) -> str:
        """Combine the lanes' partial results of a team; every lane gets the total.
        Teams of up to 64 lanes use the DPP/bpermute butterfly, a team that is the
        whole workgroup (rows too long and too few for wavefront teams) goes
        through LDS."""
        W = self.spec.width
        if self.spec.rows == "mixed":
            return f"appy::team_reduce_dyn<{_OPS[op]}, {ty.c}>({partial}, __W)"
        if W <= 64:
            return f"appy::team_reduce<{_OPS[op]}, {W}, {ty.c}>({partial})"
        return f"appy::workgroup_reduce_all<{_OPS[op]}, {self.spec.block}, {ty.c}>({partial}, {T.identity_literal(op, ty)})"

    def _stores_what_others_read(self, loop: ast.For) -> bool:
        """True if ``loop`` stores to an array that statements outside it load: in a team of
        several wavefronts those statements run on every wavefront, so the wavefronts must
        have passed them before any of them starts storing."""
        stored = {n.targets[0].value.id for n in ast.walk(loop)
                  if isinstance(n, ast.Assign) and isinstance(n.targets[0], ast.Subscript)
                  and isinstance(n.targets[0].value, ast.Name)}
        if not stored:
            return False
        # (loads inside other shared-out loops are kept apart by the barriers those loops end in)
        inside = {id(n) for lp in ast.walk(self.a.outer)
                  if isinstance(lp, ast.For) and lp is not self.a.outer
                  and ("simd" in (getattr(lp, "pragma", None) or {}) or (self.a.strip and id(lp) in self.a.strip))
                  for n in ast.walk(lp)}
        inside |= {id(n) for n in ast.walk(loop)}
        return any(isinstance(n, ast.Subscript) and isinstance(n.ctx, ast.Load) and isinstance(n.value, ast.Name)
                   and n.value.id in stored and id(n) not in inside for n in ast.walk(self.a.outer))

    def _leader(self) -> str:
        """Condition under which a team-level statement has its side effect."""
        if self.spec.kind == "strip":
            return "__wave == 0 && __active"
        return "__lane == 0 && __active" if self.lds_plan else "__lane == 0"

    def _vst(self) -> str:
        return "vstore_stream" if self.spec.stream_stores else "vstore"

    def _streamed(self, sub: ast.Subscript) -> bool:
        """True if the data behind a vectorised load is read once by the whole
        launch (then it is loaded non-temporally so that it does not displace
        reused lines from the caches): always in a flat loop; in a team loop
        when the address depends on the outer iteration, directly or through
        row-dependent loop bounds."""
        if not self.spec.stream_loads:
            return False
        if self.spec.kind == "flat":
            return True
        if isinstance(sub.value, ast.Name) and sub.value.id in self.a.reread:
            return False        # the iteration comes back to this data (softmax: max, sum, write): keep it cached
        return self.bounds_vary or any(_uses_name(e, self.a.var) for e in _elts(sub))

    def vector_body(self, body, var: str, base_code: str, V: int, loads, stores, declare_locals=False, extra=None,
                    cached=None):
        """Emit V consecutive iterations starting at ``base_code``: vector
        loads first, the V scalar bodies, vector stores last."""
        regs = {}
        comp = _COMPONENTS
        for key, (arr, sub) in loads.items():
            r = self.fresh(f"ld_{arr.name}_")
            regs[key] = r
            ld = "vload_stream" if self._streamed(sub) else "vload"
            slot = (cached or {}).get(key)
            if slot is not None:
                name, fill = slot
                if fill:
                    self.w(f"{name}[__k] = appy::{ld}<{arr.elem_c}, {V}>({self._addr(arr, sub, var, base_code)});")
                self.w(f"const appy::vec<{arr.elem_c}, {V}>::type {r} = {name}[__k];")
                continue
            self.w(f"const appy::vec<{arr.elem_c}, {V}>::type {r} = "
                   f"appy::{ld}<{arr.elem_c}, {V}>({self._addr(arr, sub, var, base_code)});")
        sregs = {}
        for key, (arr, sub) in stores.items():
            r = self.fresh(f"st_{arr.name}_")
            sregs[key] = r
            self.w(f"appy::vec<{arr.elem_c}, {V}>::type {r};")
        for k in range(V):
            self.w("{")
            self.ind += 1
            self.w(f"const appy::i64 {cname(var)} = {base_code} + {k};")
            if declare_locals:
                self._declare_locals()
            saved_loads = dict(self.ex.load_subst)
            for key, (arr, _) in loads.items():
                code = f"{regs[key]}.{comp[k]}" if V > 1 else regs[key]
                self.ex.load_subst[key] = ((f"({code} != 0)" if arr.ty.is_bool else code), arr.ty)
            for key, (r, arr) in (extra or {}).items():
                self.ex.load_subst[key] = (f"{r}.{comp[k]}", arr.ty)
            saved_stores = dict(self.store_subst)
            for key, (arr, _) in stores.items():
                self.store_subst[key] = ((f"{sregs[key]}.{comp[k]}" if V > 1 else sregs[key]), arr.ty)
            self.iteration_body(body)
            self.ex.load_subst = saved_loads
            self.store_subst = saved_stores
            self.ind -= 1
            self.w("}")
        for key, (arr, sub) in stores.items():
            self.w(f"appy::{self._vst()}<{arr.elem_c}, {V}>({self._addr(arr, sub, var, base_code)}, {sregs[key]});")

    def spread_loop(self, st: ast.For):
        """A ``simd`` loop inside a team: iterations dealt to the W lanes."""
        if self.lds_plan is not None and st is self.lds_plan[0]:
            return self.tiled_spread_loop(st)
        var = st.target.id
        W, V = self.spec.width, self.spec.vec
        Wc = "__W" if self.spec.rows == "mixed" else str(W)     # the stride of the lanes of a team, in the text
        lo, hi = self._range_args(st)
        self.ex.locals[var] = T.WEAK_INT
        reds = {}
        for key, op in loop_ir.reductions_of(st).items():
            if key in self.ex.locals or key in self.a.assigned:
                reds[key] = op
        self.w("{")
        self.ind += 1
        lo_v, hi_v = self.fresh("lo"), self.fresh("hi")
        self.w(f"const appy::i64 {lo_v} = {lo};")
        self.w(f"const appy::i64 {hi_v} = {hi};")
        saved_partials = dict(self.partials)
        for name, op in reds.items():
            ty = self.ex.locals.get(name)
            if ty is None:
                raise NameError(f"reduction variable `{name}` has no value before the loop")
            p = self.fresh(f"part_{name}_")
            pty = T.partial_type(ty)
            self.partials[name] = (p, pty)
            self.w(f"{pty.c} {p} = {T.partial_identity(op, ty, pty)};")
        if self.spec.phase == 2:
            # the loop has run (phase 1); it is walked into a buffer that is thrown away, for the
            # types of the variables it assigns, and its partial results are picked up
            kept, self.lines = self.lines, []
            saved_mode, self.mode = self.mode, "lane"
            saved_depth, self.seq_depth = self.seq_depth, 0
            self.iteration_body(st.body)
            self.mode, self.seq_depth = saved_mode, saved_depth
            self.lines = kept
            for r, (name, op) in enumerate(reds.items()):
                p, pty = self.partials[name]
                vty = self.ex.locals.get(name, pty)
                self.w("#pragma unroll 16")
                self.w(f"for (appy::i64 __c = 0; __c < __nsplit; ++__c) "
                       f"{p} = {_OPS[op]}::f<{pty.c}>({p}, {self._scratch_slot(r, '__c', pty)});")
                self.w(f"{cname(name)} = {cast(_OPS[op] + '::f<' + pty.c + '>(' + cast(cname(name), vty, pty) + ', ' + p + ')', pty, vty)};")
            self.partials = saved_partials
            self.ind -= 1
            self.w("}")
            return
        if self.spec.phase == 1 and self.spec.parts:
            # the part of this workgroup slot, as the planning kernel has cut the row (relative to its start)
            lo_c, hi_c = self.fresh("lo"), self.fresh("hi")
            self.w("const appy::i64 __first = __start[__t];     // (from the plan: no need to wait for the set-up's loads)")
            self.w(f"const appy::i64 {lo_c} = __first + __bnd[__chunk * __cap + __t];")
            self.w(f"const appy::i64 {hi_c} = __first + __bnd[(__chunk + 1) * __cap + __t];")
            lo_v, hi_v = lo_c, hi_c
        elif self.spec.phase == 1:
            part = self.fresh("part")
            self.w(f"const appy::i64 {part} = ({hi_v} - {lo_v} + __nsplit - 1) / __nsplit;")
            lo_c, hi_c = self.fresh("lo"), self.fresh("hi")
            self.w(f"const appy::i64 {lo_c} = {lo_v} + __chunk * {part};")
            self.w(f"const appy::i64 {hi_c} = ({lo_c} + {part}) < {hi_v} ? ({lo_c} + {part}) : {hi_v};")
            lo_v, hi_v = lo_c, hi_c
        saved_mode = self.mode
        self.mode = "lane"
        saved_depth, self.seq_depth = self.seq_depth, 0
        saved_vary = self.bounds_vary
        outer_locals = set(self.a.assigned) | {self.a.var}
        self.bounds_vary = any(_uses_name(b, n) for b in st.iter.args[:2] for n in outer_locals)
        loads, stores = self._vector_accesses(st.body, var) if V > 1 else ({}, {})
        if W > 64 and self._stores_what_others_read(st):
            self.w("__syncthreads();   // every wavefront has read what it needs of the arrays this loop stores to")
        in_registers = (self.spec.row_steps and self.a.row_cache is not None and id(st) in self.a.row_cache[0]
                        and V > 1 and (loads or stores))
        if in_registers:
            # the host has checked that the loop is exactly row_steps x W x V long: no tail; rows
            # that other loops of the iteration read as well are loaded once and kept
            cached = {}
            for key, (arr, sub) in loads.items():
                rk = self._row_key(sub, var)
                if rk in self.rc_slots:
                    cached[key] = (self.rc_slots[rk], rk not in self.rc_filled)
            base = self.fresh("j")
            self.w("#pragma unroll")
            self.w(f"for (int __k = 0; __k < {self.spec.row_steps}; ++__k) {{")
            self.ind += 1
            self.w(f"const appy::i64 {base} = {lo_v} + ((appy::i64)__lane + (appy::i64)__k * {W}) * {V};")
            self.vector_body(st.body, var, base, V, loads, stores, cached=cached)
            self.ind -= 1
            self.w("}")
            self.rc_filled.update(self._row_key(sub, var) for key, (arr, sub) in loads.items() if key in cached)
        elif V > 1 and (loads or stores):
            nv = self.fresh("nv")
            q = self.fresh("q")
            self.w(f"const appy::i64 {nv} = ({hi_v} - {lo_v}) / {V};")
            self.w("#pragma unroll 2")
            self.w(f"for (appy::i64 {q} = __lane; {q} < {nv}; {q} += {Wc}) {{")
            self.ind += 1
            base = self.fresh("j")
            self.w(f"const appy::i64 {base} = {lo_v} + {q} * {V};")
            self.vector_body(st.body, var, base, V, loads, stores)
            self.ind -= 1
            self.w("}")
            start = f"{lo_v} + {nv} * {V} + __lane"
        else:
            start = f"{lo_v} + __lane"
        if not in_registers:
            self.w(f"for (appy::i64 {cname(var)} = {start}; {cname(var)} < {hi_v}; {cname(var)} += {Wc}) {{")
            self.ind += 1
            self.iteration_body(st.body)
            self.ind -= 1
            self.w("}")
        self.mode = saved_mode
        self.seq_depth = saved_depth
        self.bounds_vary = saved_vary
        if W > 64 and any(isinstance(n, ast.Assign) and isinstance(n.targets[0], ast.Subscript)
                          for b in st.body for n in ast.walk(b)):
            # a team of several wavefronts: what one of them stored is read by the others only after this
            self.w("__syncthreads();")
        elif (1 < W <= 64 or self.spec.rows == "mixed") and any(
                isinstance(n, ast.Subscript) and isinstance(n.value, ast.Name) and n.value.id in self.a.stored
                for b in st.body for n in ast.walk(b)):
            # lanes of one wavefront: the loop touches an array that the nest stores to, and another
            # lane may touch the same elements in a later loop (slices that overlap, shifted reads)
            self.w("appy::wave_fence();")
        for r, (name, op) in enumerate(reds.items()):
            p, ty = self.partials[name]
            vty = self.ex.locals.get(name, ty)
            total = self._team_total(op, ty, p)
            if self.spec.phase == 1:
                t = self.fresh("tot")
                self.w(f"const {ty.c} {t} = {total};")
                self.w(f"if ({self._leader()}) {self._scratch_slot(r, '__chunk', ty)} = {t};")
            else:
                self.w(f"{cname(name)} = {cast(_OPS[op] + '::f<' + ty.c + '>(' + cast(cname(name), vty, ty) + ', ' + total + ')', ty, vty)};")
        self.partials = saved_partials
        self.ind -= 1
        self.w("}")

    # ---- row accumulators ----------------------------------------------------------
    def _match_row_update(self, loop):
        """``for c in range(0, E): T[.., c] = T[.., c] (op) rest`` with ``simd``
        -> (T subscript, op, rest, c, E node) or None."""
        if not (isinstance(loop, ast.For) and "simd" in (getattr(loop, "pragma", None) or {})
                and len(loop.body) == 1 and isinstance(loop.body[0], ast.Assign)):
            return None
        lo, hi, _ = loop.iter.args
        if not (isinstance(lo, ast.Constant) and lo.value == 0):
            return None
        c = loop.target.id
        st = loop.body[0]
        tgt = st.targets[0]
        if not (isinstance(tgt, ast.Subscript) and isinstance(tgt.value, ast.Name) and tgt.value.id in self.a.arrays):
            return None
        el = _elts(tgt)
        if not (isinstance(el[-1], ast.Name) and el[-1].id == c) or any(_uses_name(e, c) for e in el[:-1]):
            return None
        if not any(_var_offset(e, self.a.var) is not None for e in el):
            return None     # a row that other outer iterations update as well cannot live in registers
        key = ast.unparse(tgt)
        arr_name = tgt.value.id
        val = st.value
        op, rest = None, None
        if isinstance(val, ast.BinOp) and isinstance(val.op, (ast.Add, ast.Sub, ast.Mult)):
            if ast.unparse(val.left) == key:
                op, rest = val.op, val.right
            elif ast.unparse(val.right) == key and not isinstance(val.op, ast.Sub):
                op, rest = val.op, val.left
        if op is None:
            # plain store T[.., c] = rest (the initialisation form)
            op, rest = None, val
        if any(isinstance(n, ast.Name) and n.id == arr_name for n in ast.walk(rest)):
            return None
        return tgt, op, rest, c, hi

    def row_accumulate(self, stmts, i) -> int:
        """Keep a row ``T[.., :]`` that a sequential loop updates once per
        iteration in registers: one load (or the initial value) before the
        loop, one store after it, instead of a read-modify-write of the row in
        memory per iteration.  Legal because the row belongs to this team's
        outer iteration alone.  Returns the number of statements consumed."""
        W, V, E = self.spec.width, self.spec.vec, self.spec.extent
        init = None
        k = i
        m0 = self._match_row_update(stmts[k])
        if m0 is not None and m0[1] is None and k + 1 < len(stmts):
            init = m0
            k += 1
        kloop = stmts[k]
        if not (isinstance(kloop, ast.For) and "simd" not in (getattr(kloop, "pragma", None) or {})
                and len(kloop.body) == 1):
            return 0
        m1 = self._match_row_update(kloop.body[0])
        if m1 is None or m1[1] is None:
            return 0
        tgt, op, rest, c, hi = m1
        kvar = kloop.target.id
        if _uses_name(tgt, kvar) or E % V != 0:
            return 0
        if init is not None:
            itgt, _, ival, ic, ihi = init
            same_row = ast.unparse(_Rename(ic, c).visit(_copy(itgt))) == ast.unparse(tgt)
            if not same_row or ast.unparse(ihi) != ast.unparse(hi) or _uses_name(ival, ic):
                return 0
        arr = self.a.arrays[tgt.value.id]
        arr.loaded = arr.loaded or init is None
        nv = -(-E // (W * V))
        if nv > 8:
            return 0
        vt = f"appy::vec<{arr.elem_c}, {V}>::type"
        comp = _COMPONENTS
        self.ex.locals[c] = T.WEAK_INT
        self.w("{")
        self.ind += 1
        self.ex.emit(hi)     # registers the extent as a kernel argument
        self.w(f"// row accumulators: extent {E} is fixed at compile time (asserted by the launcher)")
        accs = [self.fresh("acc") for _ in range(nv)]
        bases = [f"(({t * W}LL + __lane) * {V})" for t in range(nv)]
        full = [(t + 1) * W * V <= E for t in range(nv)]
        for t in range(nv):
            self.w(f"{vt} {accs[t]};")
            guard = "" if full[t] else f"if ({bases[t]} < {E}LL) "
            if init is not None:
                vc, vty = self.ex.emit(init[2])
                val = self._store_value(vc, vty, arr)
                self.w(f"{guard}{{ " + " ".join(f"{accs[t]}.{comp[v]} = {val};" for v in range(V)) + " }")
            else:
                self.w(f"{guard}{accs[t]} = appy::vload<{arr.elem_c}, {V}>({self._addr(arr, tgt, c, bases[t])});")
        lo_c, hi_c = self._range_args(kloop)
        self.ex.locals[kvar] = T.WEAK_INT
        hi_v = self.fresh("hi")
        self.w(f"const appy::i64 {hi_v} = {hi_c};")
        self.w("#pragma unroll 4")
        self.w(f"for (appy::i64 {cname(kvar)} = {lo_c}; {cname(kvar)} < {hi_v}; ++{cname(kvar)}) {{")
        self.ind += 1
        saved_mode = self.mode
        self.mode = "lane"
        loads, _ = self._vector_accesses([ast.Assign(targets=[ast.Name(id="__rest", ctx=ast.Store())], value=rest)], c)
        sym = {ast.Add: "+", ast.Sub: "-", ast.Mult: "*"}[type(op)]
        for t in range(nv):
            self.w("{" if full[t] else f"if ({bases[t]} < {E}LL) {{")
            self.ind += 1
            regs = {}
            for key, (larr, lsub) in loads.items():
                r = self.fresh(f"ld_{larr.name}_")
                regs[key] = r
                ld = "vload_stream" if (self.spec.stream_loads and _uses_name(lsub, self.a.var)) else "vload"
                self.w(f"const appy::vec<{larr.elem_c}, {V}>::type {r} = "
                       f"appy::{ld}<{larr.elem_c}, {V}>({self._addr(larr, lsub, c, bases[t])});")
            for v in range(V):
                saved = dict(self.ex.load_subst)
                for key, (larr, _) in loads.items():
                    code = f"{regs[key]}.{comp[v]}"
                    self.ex.load_subst[key] = ((f"({code} != 0)" if larr.ty.is_bool else code), larr.ty)
                self.w(f"{{ const appy::i64 {cname(c)} = {bases[t]} + {v};")
                rc, rty = self.ex.emit(rest)
                a = f"{accs[t]}.{comp[v]}"
                rt_ = T.promote(arr.ty, rty)
                self.w(f"  {a} = {cast(f'({cast(a, arr.ty, rt_)} {sym} {cast(rc, rty, rt_)})', rt_, arr.ty)}; }}")
                self.ex.load_subst = saved
            self.ind -= 1
            self.w("}")
        self.mode = saved_mode
        self.ind -= 1
        self.w("}")
        for t in range(nv):
            guard = "" if full[t] else f"if ({bases[t]} < {E}LL) "
            self.w(f"{guard}appy::vstore<{arr.elem_c}, {V}>({self._addr(arr, tgt, c, bases[t])}, {accs[t]});")
        if 1 < W <= 64:
            self.w("appy::wave_fence();     // the row is stored: later loops of the team may read other lanes' elements")
        self.ind -= 1
        self.w("}")
        return k - i + 1

    def interchange_row_update(self, kloop) -> bool:
        """``for k in ...:  (simd) for c in range(0, n): T[.., c] = T[.., c] op rest(k, c)``
        is emitted with the loops interchanged: every lane keeps its elements of the
        row in registers while it runs the ``k`` loop, instead of reading and
        writing the row in memory once per ``k`` (and waiting for that round trip
        each time).  Legal because the elements are independent of each other
        (``simd``), ``rest`` does not read ``T``, and the row belongs to this team's
        outer iteration.  Same idea as the row accumulators, for extents that are
        only known at run time."""
        if not (isinstance(kloop, ast.For) and "simd" not in (getattr(kloop, "pragma", None) or {})
                and len(kloop.body) == 1 and not kloop.orelse):
            return False
        m = self._match_row_update(kloop.body[0])
        if m is None or m[1] is None:
            return False
        tgt, op, rest, c, hi = m
        kvar = kloop.target.id
        if _uses_name(tgt, kvar) or _uses_name(hi, kvar) or any(_uses_name(b, c) for b in kloop.iter.args):
            return False
        if loop_ir.reductions_of(kloop.body[0]):
            return False
        arr = self.a.arrays[tgt.value.id]
        arr.loaded = True
        W, V = self.spec.width, self.spec.vec
        sym = {ast.Add: "+", ast.Sub: "-", ast.Mult: "*"}[type(op)]
        comp = _COMPONENTS
        self.w("{")
        self.ind += 1
        self.w("// loops interchanged: the row elements stay in registers across the sequential loop")
        self.ex.locals[c] = T.WEAK_INT
        self.ex.locals[kvar] = T.WEAK_INT
        hc, ht = self.ex.emit(hi)
        n_v = self.fresh("n")
        self.w(f"const appy::i64 {n_v} = {cast(hc, ht, T.I64)};")
        klo, khi = self._range_args(kloop)
        klo_v, khi_v = self.fresh("klo"), self.fresh("khi")
        self.w(f"const appy::i64 {klo_v} = {klo};")
        self.w(f"const appy::i64 {khi_v} = {khi};")
        saved_mode, self.mode = self.mode, "lane"
        saved_depth, self.seq_depth = self.seq_depth, 0
        probe = [ast.Assign(targets=[ast.Name(id="__rest", ctx=ast.Store())], value=rest)]
        loads, _ = self._vector_accesses(probe, c) if V > 1 else ({}, {})
        # loads of `rest` must not see elements of arrays that the k loop itself changes: there are none
        # (its only statement is this update, and `rest` does not read T)
        start = "__lane"
        if V > 1:
            nv, q, base, acc = self.fresh("nv"), self.fresh("q"), self.fresh("c0"), self.fresh("acc")
            self.w(f"const appy::i64 {nv} = {n_v} / {V};")
            self.w(f"for (appy::i64 {q} = __lane; {q} < {nv}; {q} += {W}) {{")
            self.ind += 1
            self.w(f"const appy::i64 {base} = {q} * {V};")
            self.w(f"appy::vec<{arr.elem_c}, {V}>::type {acc} = appy::vload<{arr.elem_c}, {V}>({self._addr(arr, tgt, c, base)});")
            self.w("#pragma unroll 2")
            self.w(f"for (appy::i64 {cname(kvar)} = {klo_v}; {cname(kvar)} < {khi_v}; ++{cname(kvar)}) {{")
            self.ind += 1
            regs = {}
            for key, (larr, lsub) in loads.items():
                r = self.fresh(f"ld_{larr.name}_")
                regs[key] = r
                self.w(f"const appy::vec<{larr.elem_c}, {V}>::type {r} = "
                       f"appy::vload<{larr.elem_c}, {V}>({self._addr(larr, lsub, c, base)});")
            for v in range(V):
                saved = dict(self.ex.load_subst)
                for key, (larr, _) in loads.items():
                    code = f"{regs[key]}.{comp[v]}"
                    self.ex.load_subst[key] = ((f"({code} != 0)" if larr.ty.is_bool else code), larr.ty)
                self.w(f"{{ const appy::i64 {cname(c)} = {base} + {v};")
                rc, rty = self.ex.emit(rest)
                a = f"{acc}.{comp[v]}"
                rt_ = T.promote(arr.ty, rty)
                self.w(f"  {a} = {cast(f'({cast(a, arr.ty, rt_)} {sym} {cast(rc, rty, rt_)})', rt_, arr.ty)}; }}")
                self.ex.load_subst = saved
            self.ind -= 1
            self.w("}")
            self.w(f"appy::vstore<{arr.elem_c}, {V}>({self._addr(arr, tgt, c, base)}, {acc});")
            self.ind -= 1
            self.w("}")
            start = f"{nv} * {V} + __lane"
        acc = self.fresh("acc")
        self.w(f"for (appy::i64 {cname(c)} = {start}; {cname(c)} < {n_v}; {cname(c)} += {W}) {{")
        self.ind += 1
        idx = self.ex.index_code(arr, tgt)
        self.w(f"{arr.ty.c} {acc} = {cname(arr.name)}[{idx}];")
        self.w(f"for (appy::i64 {cname(kvar)} = {klo_v}; {cname(kvar)} < {khi_v}; ++{cname(kvar)}) {{")
        self.ind += 1
        rc, rty = self.ex.emit(rest)
        rt_ = T.promote(arr.ty, rty)
        self.w(f"{acc} = {cast(f'({cast(acc, arr.ty, rt_)} {sym} {cast(rc, rty, rt_)})', rt_, arr.ty)};")
        self.ind -= 1
        self.w("}")
        self.w(f"{cname(arr.name)}[{idx}] = {acc};")
        self.ind -= 1
        self.w("}")
        self.mode, self.seq_depth = saved_mode, saved_depth
        if 1 < W <= 64:
            self.w("appy::wave_fence();     // the row is stored: later loops of the team may read other lanes' elements")
        self.ind -= 1
        self.w("}")
        return True

    # ---- kernel skeletons ---------------------------------------------------------
    def _declare_locals(self):
        for name in self.a.assigned:
            ty = self.ex.locals.get(name)
            if ty is None:
                continue
            init = f" = {cname(name)}__arg" if name in self.shadowed else " = 0"
            self.w(f"{ty.c} {cname(name)}{init};")

    def _iteration(self, idx_code: str, body=None):
        self.w("{")
        self.ind += 1
        if body is not None:
            self.w(f"const appy::i64 {cname(self.a.var)} = {idx_code};")
            self._declare_locals()
            self.iteration_body(body)
        elif self.spec.collapse:
            # idx_code counts the pairs (i, j) from zero, j fastest
            inner = self.a.collapse
            self.w(f"const appy::i64 {cname(self.a.var)} = __lo + ({idx_code}) / __nj;")
            self.w(f"const appy::i64 {cname(inner.target.id)} = __jlo + ({idx_code}) % __nj;")
            self.ex.locals[inner.target.id] = T.WEAK_INT
            self._declare_locals()
            self._declare_row_cache(inner.body)
            self.iteration_body(inner.body)
        else:
            self.w(f"const appy::i64 {cname(self.a.var)} = {idx_code};")
            self._declare_locals()
            self._declare_row_cache(self.a.outer.body)
            self.iteration_body(self.a.outer.body)
        self.ind -= 1
        self.w("}")

    def _row_key(self, sub: ast.Subscript, var: str) -> str:
        """A subscript with the loop variable blanked out: the same element of the row,
        whatever the loop that touches it calls its variable."""
        node = ast.parse(ast.unparse(sub), mode="eval").body
        for n in ast.walk(node):
            if isinstance(n, ast.Name) and n.id == var:
                n.id = "__step"
        return ast.unparse(node)

    def _declare_row_cache(self, body):
        self.rc_slots, self.rc_filled = {}, set()
        if not self.spec.row_steps or self.a.row_cache is None:
            return
        if bool(self.spec.collapse) != (self.a.collapse is not None):
            return      # the loops sit under a sequential loop here: nothing outlives one pass of it
        loops, arrays, _bounds = self.a.row_cache
        V = self.spec.vec
        for st in body:
            if isinstance(st, ast.For) and id(st) in loops:
                loads, _stores = self._vector_accesses(st.body, st.target.id)
                for _key, (arr, sub) in loads.items():
                    rk = self._row_key(sub, st.target.id)
                    if arr.name in arrays and rk not in self.rc_slots:
                        slot = f"__rc{len(self.rc_slots)}"
                        self.rc_slots[rk] = slot
                        self.w(f"appy::vec<{arr.elem_c}, {V}>::type {slot}[{self.spec.row_steps}];   // {ast.unparse(sub)}")

    def _body_flat(self):
        s = self.spec
        V, U, B = s.vec, s.unroll, s.block
        var = self.a.var
        self.ex.locals[var] = T.WEAK_INT
        loads, stores = self._vector_accesses(self.a.outer.body, var, s.hoist_guarded) if V > 1 else ({}, {})
        vectorised = V > 1 and (loads or stores)
        self.lane_step_bytes = sum(V * arr.ty.size for arr, _ in list(loads.values()) + list(stores.values()))
        self.w("const appy::i64 __tid = threadIdx.x;")
        self.w("const appy::i64 __nblk = gridDim.x;")
        if vectorised:
            tile = B * U * V
            self.w(f"const appy::i64 __ntiles = (__hi - __lo) / {tile};")
            self.w("for (appy::i64 __t = blockIdx.x; __t < __ntiles; __t += __nblk) {")
            self.ind += 1
            self.w(f"const appy::i64 __tile0 = __lo + __t * {tile} + __tid * {V};")
            if U == 1:
                self.vector_body(self.a.outer.body, var, "__tile0", V, loads, stores, declare_locals=True)
            else:
                # all loads of the tile first, then the arithmetic, then the stores
                self._flat_unrolled_tile(V, U, B, loads, stores)
            self.ind -= 1
            self.w("}")
            self.w(f"const appy::i64 __rest0 = __lo + __ntiles * {tile};")
            self.w(f"const appy::i64 __nrv = (__hi - __rest0) / {V};")
            self.w(f"for (appy::i64 __q = blockIdx.x * {B}LL + __tid; __q < __nrv; __q += __nblk * {B}LL) {{")
            self.ind += 1
            self.w(f"const appy::i64 __vb = __rest0 + __q * {V};")
            self.vector_body(self.a.outer.body, var, "__vb", V, loads, stores, declare_locals=True)
            self.ind -= 1
            self.w("}")
            tail0 = f"__rest0 + __nrv * {V}"
        else:
            tail0 = "__lo"
        self.w(f"for (appy::i64 __i = {tail0} + blockIdx.x * {B}LL + __tid; __i < __hi; __i += __nblk * {B}LL) {{")
        self.ind += 1
        self._iteration("__i")
        self.ind -= 1
        self.w("}")

    def _flat_unrolled_tile(self, V, U, B, loads, stores):
        comp = _COMPONENTS
        var = self.a.var
        regs = {}
        for u in range(U):
            base = f"(__tile0 + {u * B * V})"
            for key, (arr, sub) in loads.items():
                r = self.fresh(f"ld_{arr.name}_")
                regs[(u, key)] = r
                ld = "vload_stream" if self._streamed(sub) else "vload"
                self.w(f"const appy::vec<{arr.elem_c}, {V}>::type {r} = "
                       f"appy::{ld}<{arr.elem_c}, {V}>({self._addr(arr, sub, var, base)});")
        sregs = {}
        for u in range(U):
            for key, (arr, sub) in stores.items():
                r = self.fresh(f"st_{arr.name}_")
                sregs[(u, key)] = r
                self.w(f"appy::vec<{arr.elem_c}, {V}>::type {r};")
        for u in range(U):
            base = f"(__tile0 + {u * B * V})"
            for k in range(V):
                self.w("{")
                self.ind += 1
                self.w(f"const appy::i64 {cname(var)} = {base} + {k};")
                self._declare_locals()
                saved_loads = dict(self.ex.load_subst)
                saved_stores = dict(self.store_subst)
                for key, (arr, _) in loads.items():
                    code = f"{regs[(u, key)]}.{comp[k]}"
                    self.ex.load_subst[key] = ((f"({code} != 0)" if arr.ty.is_bool else code), arr.ty)
                for key, (arr, _) in stores.items():
                    self.store_subst[key] = (f"{sregs[(u, key)]}.{comp[k]}", arr.ty)
                self.iteration_body(self.a.outer.body)
                self.ex.load_subst = saved_loads
                self.store_subst = saved_stores
                self.ind -= 1
                self.w("}")
        for u in range(U):
            base = f"(__tile0 + {u * B * V})"
            for key, (arr, sub) in stores.items():
                self.w(f"appy::{self._vst()}<{arr.elem_c}, {V}>({self._addr(arr, sub, var, base)}, {sregs[(u, key)]});")

    def _body_strip(self):
        """Column loops: the 64 lanes of a wavefront take 64 consecutive outer
        iterations (so that ``A[j, i]`` is one contiguous row segment per step) and
        the wavefronts of the workgroup are the team of each of them: statements
        outside the shared-out loops run on every wavefront with equal values and
        store from wavefront 0, the shared-out loops deal their iterations to the
        wavefronts, partial results meet in LDS.  Lanes past the end of the range
        run on the last iteration with their effects switched off, so that every
        thread reaches every barrier."""
        if self.a.strip is None or self.a.outer_reductions:
            raise Unsupported("the loop nest does not suit the strip shape")
        NW = self.spec.block // 64
        var = self.a.var
        self.ex.locals[var] = T.WEAK_INT
        self.w("const int __lane = threadIdx.x & 63;")
        self.w("const int __wave = threadIdx.x >> 6;")
        self.w(f"__shared__ double __strip_slots[{NW}][64];   // one slot per wavefront and lane, any 4- or 8-byte type")
        body = self.a.outer.body
        if self.spec.phase:
            if self.a.strip_split is None:
                raise Unsupported("the loop nest does not suit the two-phase strip shape")
        if self.spec.phase == 1:
            # __nsplit workgroups per strip, each with its part of the shared-out loop's range;
            # the grid holds exactly strips x __nsplit workgroups
            self.w("const appy::i64 __chunk = blockIdx.x % __nsplit;")
            self.w("for (appy::i64 __s = blockIdx.x / __nsplit; __lo + __s * 64 < __hi; __s += gridDim.x / __nsplit) {")
            body = body[:body.index(self.a.strip_split) + 1]
        else:
            self.w("for (appy::i64 __s = blockIdx.x; __lo + __s * 64 < __hi; __s += gridDim.x) {")
        self.ind += 1
        self.w("const bool __active = __lo + __s * 64 + __lane < __hi;")
        self.w(f"const appy::i64 {cname(var)} = __active ? __lo + __s * 64 + __lane : __hi - 1;")
        self._declare_locals()
        self.mode = "team"
        self.block(body)
        self.mode = "lane"
        self.ind -= 1
        self.w("}")

    def _scratch_slot(self, r: int, chunk: str, pty: Ty) -> str:
        """Partial result number ``r`` of part ``chunk`` of this lane's column (8-byte slots)."""
        var = cname(self.a.var)
        if self.spec.rows == "list":
            # listed rows: the slot follows the position in the list, `__cap` rows at most
            return f"*reinterpret_cast<{pty.c}*>(__scratch + (({r} * __nsplit + {chunk}) * __cap + __t))"
        if self.spec.guard == 1 and pty.size == 4:
            # sums of grouped elements: 4-byte slots
            return f"reinterpret_cast<{pty.c}*>(__scratch)[({r} * __nsplit + {chunk}) * (__hi - __lo) + ({var} - __lo)]"
        return f"*reinterpret_cast<{pty.c}*>(__scratch + (({r} * __nsplit + {chunk}) * (__hi - __lo) + ({var} - __lo)))"

    def strip_spread_loop(self, st: ast.For):
        """A loop of a strip kernel whose iterations are dealt to the wavefronts."""
        ops = self.a.strip[id(st)]
        NW = self.spec.block // 64
        var = st.target.id
        lo, hi = self._range_args(st)
        self.ex.locals[var] = T.WEAK_INT
        self.w("{")
        self.ind += 1
        lo_v, hi_v = self.fresh("lo"), self.fresh("hi")
        self.w(f"const appy::i64 {lo_v} = {lo};")
        self.w(f"const appy::i64 {hi_v} = {hi};")
        saved_partials = dict(self.partials)
        typed = {}
        for name, op in ops.items():
            ty = self.ex.locals.get(name)
            if ty is None:
                raise NameError(f"reduction variable `{name}` has no value before the loop")
            pty = T.partial_type(ty)
            p = self.fresh(f"part_{name}_")
            typed[name] = (p, pty)
            self.partials[name] = (p, pty)
            self.w(f"{pty.c} {p} = {T.partial_identity(op, ty, pty)};")
        if self.spec.phase == 2:
            # The loop has run already (phase 1): pick up the partial results of its parts.  The
            # loop is still walked, into a buffer that is thrown away, because its statements
            # decide the types of the variables they assign - both phases must agree on those.
            kept, self.lines = self.lines, []
            saved_mode, self.mode = self.mode, "lane"
            saved_depth, self.seq_depth = self.seq_depth, 0
            self.iteration_body(st.body)
            self.mode, self.seq_depth = saved_mode, saved_depth
            self.lines = kept
            for r, (name, (p, pty)) in enumerate(typed.items()):
                op = _OPS[ops[name]]
                vty = self.ex.locals[name]
                self.w("if (__active) {")
                self.w("    #pragma unroll 16")
                self.w(f"    for (appy::i64 __c = 0; __c < __nsplit; ++__c) "
                       f"{p} = {op}::f<{pty.c}>({p}, {self._scratch_slot(r, '__c', pty)});")
                self.w("}")
                self.w(f"{cname(name)} = {cast(op + '::f<' + pty.c + '>(' + cast(cname(name), vty, pty) + ', ' + p + ')', pty, vty)};")
            self.partials = saved_partials
            self.ind -= 1
            self.w("}")
            return
        if self.spec.phase == 1 and self.spec.parts:
            # the part of this workgroup slot, as the planning kernel has cut the row (relative to its start)
            lo_c, hi_c = self.fresh("lo"), self.fresh("hi")
            self.w(f"const appy::i64 {lo_c} = __bnd[__chunk * __cap + __t];")
            self.w(f"const appy::i64 {hi_c} = __bnd[(__chunk + 1) * __cap + __t];")
            lo_v, hi_v = lo_c, hi_c
        elif self.spec.phase == 1:
            part = self.fresh("part")
            self.w(f"const appy::i64 {part} = ({hi_v} - {lo_v} + __nsplit - 1) / __nsplit;")
            lo_c, hi_c = self.fresh("lo"), self.fresh("hi")
            self.w(f"const appy::i64 {lo_c} = {lo_v} + __chunk * {part};")
            self.w(f"const appy::i64 {hi_c} = ({lo_c} + {part}) < {hi_v} ? ({lo_c} + {part}) : {hi_v};")
            lo_v, hi_v = lo_c, hi_c
        saved_mode, self.mode = self.mode, "lane"
        saved_depth, self.seq_depth = self.seq_depth, 0
        saved_stream = set(self.ex.stream_arrays)
        if self.spec.stream_loads:
            # matrices walked once by the launch (indexed by both loop variables) bypass the caches
            for b in st.body:
                for n in ast.walk(b):
                    if (isinstance(n, ast.Subscript) and isinstance(n.value, ast.Name) and n.value.id in self.a.arrays
                            and _uses_name(n, var) and _uses_name(n, self.a.var)):
                        self.ex.stream_arrays.add(n.value.id)
        if self._stores_what_others_read(st):
            self.w("__syncthreads();   // every wavefront has read what it needs of the arrays this loop stores to")
        # lanes past the end of the range skip the loop as a whole (its bounds stay wavefront-uniform,
        # which keeps the unrolled loads of a step in flight together); the barriers are outside
        self.w("if (__active) {")
        self.ind += 1
        self.w(f"#pragma unroll {max(4, self.spec.unroll)}")
        self.w(f"for (appy::i64 {cname(var)} = {lo_v} + __wave; {cname(var)} < {hi_v}; {cname(var)} += {NW}) {{")
        self.ind += 1
        self.iteration_body(st.body)
        self.ind -= 1
        self.w("}")
        self.ind -= 1
        self.w("}")
        self.ex.stream_arrays = saved_stream
        self.mode, self.seq_depth = saved_mode, saved_depth
        self.partials = saved_partials
        stores = any(isinstance(n, ast.Assign) and isinstance(n.targets[0], ast.Subscript)
                     for b in st.body for n in ast.walk(b))
        if stores and not typed:
            self.w("__syncthreads();   // what one wavefront stored, the others may read from here on")
        for name, (p, pty) in typed.items():
            op = _OPS[ops[name]]
            vty = self.ex.locals[name]
            slot = f"reinterpret_cast<{pty.c}*>(&__strip_slots[0][0])"
            self.w(f"{slot}[__wave * 64 + __lane] = {p};")
            self.w("__syncthreads();")
            t = self.fresh("tot")
            self.w(f"{pty.c} {t} = {slot}[__lane];")
            self.w(f"for (int __w = 1; __w < {NW}; ++__w) {t} = {op}::f<{pty.c}>({t}, {slot}[__w * 64 + __lane]);")
            if self.spec.phase == 1:
                r = list(typed).index(name)
                self.w(f"if (__wave == 0 && __active) {self._scratch_slot(r, '__chunk', pty)} = {t};")
            else:
                self.w(f"{cname(name)} = {cast(op + '::f<' + pty.c + '>(' + cast(cname(name), vty, pty) + ', ' + t + ')', pty, vty)};")
            self.w("__syncthreads();   // the slots are free again")
        self.ind -= 1
        self.w("}")

    def _find_lds_plan(self):
        """A ``simd`` loop directly in the body of the parallel loop whose bounds
        are the same for every outer iteration and that reads 1-D arrays indexed
        by its own variable only (``x[j]`` of GEMV): those operands are the same
        for every row, so a workgroup stages them in LDS once per tile and all
        its teams read them from there."""
        if not self.spec.lds_tile or self.a.outer_reductions:
            return None
        if skips_iterations(self.a.outer.body):
            return None     # every thread has to reach the barriers of the tile loop
        # teams past the end of the range run on a clamped row with their team-level
        # side effects switched off; stores issued from inside simd loops cannot be
        # switched off that way, so such kernels keep the plain form
        for n in ast.walk(self.a.outer):
            if isinstance(n, ast.For) and n is not self.a.outer and "simd" in (getattr(n, "pragma", None) or {}):
                if any(isinstance(a, ast.Assign) and isinstance(a.targets[0], ast.Subscript) for a in ast.walk(n)):
                    return None
        outer_locals = set(self.a.assigned) | {self.a.var}
        for st in self.a.outer.body:
            if not (isinstance(st, ast.For) and "simd" in (getattr(st, "pragma", None) or {})):
                continue
            if any(_uses_name(b, n) for b in st.iter.args[:2] for n in outer_locals):
                continue
            j = st.target.id
            found = {}
            guarded = guarded_nodes(st.body)
            for n in ast.walk(st):
                if (isinstance(n, ast.Subscript) and isinstance(n.value, ast.Name) and n.value.id in self.a.arrays
                        and isinstance(n.ctx, ast.Load) and isinstance(n.slice, ast.Name) and n.slice.id == j
                        and id(n) not in guarded):
                    arr = self.a.arrays[n.value.id]
                    if arr.ndim == 1 and arr.name not in self.a.stored and not arr.ty.is_bool:
                        found[arr.name] = arr
            if found:
                return st, list(found.values())
        return None

    def _body_team(self):
        s = self.spec
        W, B = s.width, s.block
        tpb = B // W
        var = self.a.var
        self.ex.locals[var] = T.WEAK_INT
        self.lds_plan = self._find_lds_plan()
        if s.guard:
            # the grouping kernel of this launch raises the flag when it refuses its input
            self.w(f"if ((__flag[0] != 0) == {'true' if s.guard == 1 else 'false'}) return;")
        if s.aux or s.rows:
            if self.a.ragged is None or self.lds_plan is not None:
                raise Unsupported("the loop nest does not suit kernels over binned rows")
            if s.aux in ("group", "cells", "rkeys", "xcells"):
                if self.a.grouping is None:
                    raise Unsupported("the simd loop is not a sum of terms that gather from one operand")
                return {"group": self._body_group, "cells": self._body_cells, "rkeys": self._body_rkeys,
                        "xcells": self._body_xcells}[s.aux]()
            if s.aux == "bins":
                return self._body_bins()
            if s.rows == "mixed":
                return self._body_mixed()
            return self._body_listed()
        self.w(f"const int __lane = threadIdx.x & {W - 1};")
        self.w(f"const appy::i64 __team = threadIdx.x / {W};")
        if self.spec.phase:
            if self.a.team_split is None or self.lds_plan is not None:
                raise Unsupported("the loop nest does not suit the two-phase team shape")
            self.mode = "team"
            if self.spec.phase == 1:
                # __nsplit workgroups per row, each with its part of the simd loop's range
                self.w("const appy::i64 __chunk = blockIdx.x % __nsplit;")
                self.w(f"for (appy::i64 __i = __lo + (blockIdx.x / __nsplit) * {tpb}LL + __team; __i < __hi; "
                       f"__i += (gridDim.x / __nsplit) * {tpb}LL) {{")
                self.ind += 1
                body = self.a.outer.body
                self._iteration("__i", body[:body.index(self.a.team_split) + 1])
            else:
                self.w(f"for (appy::i64 __i = __lo + blockIdx.x * {tpb}LL + __team; __i < __hi; __i += gridDim.x * {tpb}LL) {{")
                self.ind += 1
                if s.skip_long:
                    # rows beyond the limit have run in planned parts, their statements after the loop with them
                    self._split_iteration("__i", guard="__trip <= __rowmax")
                else:
                    self._iteration("__i")
            self.mode = "lane"
            self.ind -= 1
            self.w("}")
            return
        if self.spec.collapse:
            if self.a.collapse is None or self.lds_plan is not None:
                raise Unsupported("the loop nest does not suit the collapsed shape")
            jlo, jhi = self._range_args(self.a.collapse)
            self.w(f"const appy::i64 __jlo = {jlo};")
            self.w(f"const appy::i64 __nj = ({jhi}) > __jlo ? ({jhi}) - __jlo : 0;")
            self.w(f"for (appy::i64 __c = blockIdx.x * {tpb}LL + __team; __c < (__hi - __lo) * __nj; __c += gridDim.x * {tpb}LL) {{")
            self.ind += 1
            self.mode = "team"
            self._iteration("__c")
            self.mode = "lane"
            self.ind -= 1
            self.w("}")
            return
        if self.lds_plan is None:
            self.w(f"for (appy::i64 __i = __lo + blockIdx.x * {tpb}LL + __team; __i < __hi; __i += gridDim.x * {tpb}LL) {{")
            self.ind += 1
            self.mode = "team"
            self._iteration("__i")
            self.mode = "lane"
            self.ind -= 1
            self.w("}")
            return
        # Every thread of the workgroup takes part in filling the LDS tiles, so
        # teams past the end of the range stay in the loop on a clamped row and
        # only their side effects are switched off.
        for arr in self.lds_plan[1]:
            self.w(f"__shared__ __attribute__((aligned(16))) {arr.elem_c} __tile_{cname(arr.name)}[{s.lds_tile}];")
        self.w(f"for (appy::i64 __ib = __lo + blockIdx.x * {tpb}LL; __ib < __hi; __ib += gridDim.x * {tpb}LL) {{")
        self.ind += 1
        self.w("const bool __active = (__ib + __team) < __hi;")
        self.w("const appy::i64 __i = __active ? (__ib + __team) : (__hi - 1);")
        self.mode = "team"
        self._iteration("__i")
        self.mode = "lane"
        self.ind -= 1
        self.w("}")

    def tiled_spread_loop(self, st: ast.For):
        """The LDS-staged form of :meth:`spread_loop` for the loop of the plan."""
        var = st.target.id
        W, V, TILE, B = self.spec.width, self.spec.vec, self.spec.lds_tile, self.spec.block
        staged = self.lds_plan[1]
        lo, hi = self._range_args(st)
        self.ex.locals[var] = T.WEAK_INT
        reds = {k: op for k, op in loop_ir.reductions_of(st).items() if k in self.ex.locals or k in self.a.assigned}
        self.w("{")
        self.ind += 1
        lo_v, hi_v = self.fresh("lo"), self.fresh("hi")
        self.w(f"const appy::i64 {lo_v} = {lo};")
        self.w(f"const appy::i64 {hi_v} = {hi};")
        saved_partials = dict(self.partials)
        for name, op in reds.items():
            ty = self.ex.locals.get(name)
            if ty is None:
                raise NameError(f"reduction variable `{name}` has no value before the loop")
            p = self.fresh(f"part_{name}_")
            pty = T.partial_type(ty)
            self.partials[name] = (p, pty)
            self.w(f"{pty.c} {p} = {T.partial_identity(op, ty, pty)};")
        jt = self.fresh("jt")
        self.w(f"for (appy::i64 {jt} = {lo_v}; {jt} < {hi_v}; {jt} += {TILE}) {{")
        self.ind += 1
        n_t = self.fresh("nt")
        self.w(f"const appy::i64 {n_t} = ({hi_v} - {jt}) < {TILE} ? ({hi_v} - {jt}) : {TILE};")
        self.w("__syncthreads();   // the previous tile has been consumed")
        for arr in staged:
            t = f"__tile_{cname(arr.name)}"
            q = self.fresh("f")
            self.w(f"for (appy::i64 {q} = (appy::i64)threadIdx.x * {V}; {q} < {n_t}; {q} += {B * V}) {{")
            self.ind += 1
            self.w(f"if ({q} + {V} <= {n_t}) {{")
            self.w(f"    appy::lds_vstore<{arr.elem_c}, {V}>(&{t}[{q}], appy::vload<{arr.elem_c}, {V}>({cname(arr.name)} + {jt} + {q}));")
            self.w("} else {")
            self.w(f"    for (appy::i64 __e = {q}; __e < {n_t}; ++__e) {t}[__e] = {cname(arr.name)}[{jt} + __e];")
            self.w("}")
            self.ind -= 1
            self.w("}")
        self.w("__syncthreads();   // the tile is complete")
        saved_mode, self.mode = self.mode, "lane"
        saved_depth, self.seq_depth = self.seq_depth, 0
        loads, stores = self._vector_accesses(st.body, var) if V > 1 else ({}, {})
        staged_keys = {f"{a.name}[{var}]" for a in staged}
        if V > 1 and (loads or stores):
            nv = self.fresh("nv")
            q = self.fresh("q")
            self.w(f"const appy::i64 {nv} = {n_t} / {V};")
            self.w("#pragma unroll 2")
            self.w(f"for (appy::i64 {q} = __lane; {q} < {nv}; {q} += {W}) {{")
            self.ind += 1
            base = self.fresh("j")
            self.w(f"const appy::i64 {base} = {jt} + {q} * {V};")
            global_loads = {k: v for k, v in loads.items() if k not in staged_keys}
            saved_loads = dict(self.ex.load_subst)
            regs = {}
            for key in staged_keys & set(loads):
                arr = loads[key][0]
                r = self.fresh(f"lds_{arr.name}_")
                regs[key] = (r, arr)
                self.w(f"const appy::vec<{arr.elem_c}, {V}>::type {r} = "
                       f"appy::lds_vload<{arr.elem_c}, {V}>(&__tile_{cname(arr.name)}[{q} * {V}]);")
            self.vector_body(st.body, var, base, V, global_loads, stores, extra=regs)
            self.ex.load_subst = saved_loads
            self.ind -= 1
            self.w("}")
            start = f"{jt} + {nv} * {V} + __lane"
        else:
            start = f"{jt} + __lane"
        self.w(f"for (appy::i64 {cname(var)} = {start}; {cname(var)} < {jt} + {n_t}; {cname(var)} += {W}) {{")
        self.ind += 1
        saved_loads = dict(self.ex.load_subst)
        for arr in staged:
            self.ex.load_subst[f"{arr.name}[{var}]"] = (f"__tile_{cname(arr.name)}[{cname(var)} - {jt}]", arr.ty)
        self.iteration_body(st.body)
        self.ex.load_subst = saved_loads
        self.ind -= 1
        self.w("}")
        self.seq_depth = saved_depth
        self.mode = saved_mode
        self.ind -= 1
        self.w("}")
        for name, op in reds.items():
            p, ty = self.partials[name]
            vty = self.ex.locals.get(name, ty)
            total = self._team_total(op, ty, p)
            self.w(f"{cname(name)} = {cast(_OPS[op] + '::f<' + ty.c + '>(' + cast(cname(name), vty, ty) + ', ' + total + ')', ty, vty)};")
        self.partials = saved_partials
        self.ind -= 1
        self.w("}")

    def _epilogue(self):
        B = self.spec.block
        for r in self.a.outer_reductions:
            ident = self._outer_identity(r)
            elem_c = self.a.arrays[r.array].elem_c
            total = "__tot" if r.elem_ty == r.ty else (
                "(unsigned char)(__tot != 0)" if r.elem_ty.is_bool else cast("__tot", r.ty, r.elem_ty))
            self.w("{")
            self.ind += 1
            self.w(f"const {r.ty.c} __tot = appy::block_reduce<{_OPS[r.op]}, {B}, {r.ty.c}>({r.acc}, {ident});")
            self.w(f"if (threadIdx.x == 0) appy::atomic_combine<{_OPS[r.op]}, {elem_c}>::run(&{cname(r.array)}[{r.index}], {total});")
            self.ind -= 1
            self.w("}")

    @staticmethod
    def _outer_identity(r: OuterReduction) -> str:
        """Neutral element of the element type, written in the accumulator type (the
        smallest int8 for a maximum over int8 values held in 32-bit registers)."""
        if r.elem_ty == r.ty:
            return T.identity_literal(r.op, r.ty)
        if r.elem_ty.is_bool:
            return "0" if r.op == "max" else "1"
        return f"(({r.ty.c}){T.identity_literal(r.op, r.elem_ty)})"

    # ---- parameters -----------------------------------------------------------------
    def _params(self):
        params = []
        used_arrays = [a for a in self.a.arrays.values() if a.loaded or a.stored]
        rs = " __restrict__" if self.spec.restrict else ""
        for arr in used_arrays:
            const = "" if arr.stored else "const "
            params.append(Param(cname(arr.name), f"{const}{arr.elem_c}*{rs} {cname(arr.name)}", C.c_void_p, "array", arr.name))
        for arr in used_arrays:
            for d in range(arr.ndim - 1):
                nm = f"{cname(arr.name)}_stride_{d}"
                params.append(Param(nm, f"const appy::i64 {nm}", C.c_int64, "stride", arr.name, d))
        for sc in self.a.scalars.values():
            if sc.name not in self.used_scalars:
                continue
            nm = cname(sc.name) + ("__arg" if sc.name in self.shadowed else "")
            params.append(Param(nm, f"const {sc.ty.c} {nm}", _CTYPES[sc.ty.name], "scalar", sc.name))
        for arr, dim in sorted(self.ex.shape_scalars):
            nm = cname(f"{arr}_shape_{dim}")
            if any(p.cname == nm for p in params):
                continue
            params.append(Param(nm, f"const appy::i64 {nm}", C.c_int64, "shape", arr, dim))
        if self.spec.checked:
            params.append(Param("__oob", "int* __oob", C.c_void_p, "oob"))
        if self.spec.phase:
            params.append(Param("__scratch", "double* __scratch", C.c_void_p, "scratch"))
            params.append(Param("__nsplit", "const appy::i64 __nsplit", C.c_int64, "nsplit"))
        sp = self.spec
        if sp.aux == "bins":
            params.append(Param("__rows", "int* __rows", C.c_void_p, "rows"))
            params.append(Param("__counts", "int* __counts", C.c_void_p, "counts"))
            params.append(Param("__zero", "int* __zero", C.c_void_p, "zero"))
        elif sp.rows == "mixed":
            params.append(Param("__rows", "const int* __rows", C.c_void_p, "rows"))
            params.append(Param("__counts", "const int* __counts", C.c_void_p, "counts"))
        elif sp.rows == "list":
            params.append(Param("__rows", "const int* __rows", C.c_void_p, "rows"))
            params.append(Param("__nrows", "const int* __nrows", C.c_void_p, "nrows"))
            params.append(Param("__bnd", ("int* __bnd" if sp.aux == "plan" else "const int* __bnd"), C.c_void_p, "bnd"))
            params.append(Param("__cap", "const appy::i64 __cap", C.c_int64, "cap"))
            if sp.aux == "plan" or sp.phase == 1:
                params.append(Param("__start", ("appy::i64* __start" if sp.aux == "plan" else "const appy::i64* __start"),
                                    C.c_void_p, "rowstart"))
            if sp.aux == "plan":
                params.append(Param("__stripe", "const appy::i64 __stripe", C.c_int64, "stripe"))
                params.append(Param("__load", "unsigned long long* __load", C.c_void_p, "load"))
            elif sp.phase == 1:
                params.append(Param("__load", "const unsigned long long* __load", C.c_void_p, "load"))
        if sp.aux in ("group", "cells"):
            params.append(Param("__ent", ("long long* __ent" if sp.aux == "group" else "const long long* __ent"), C.c_void_p, "ent"))
            params.append(Param("__desc", ("int* __desc" if sp.aux == "group" else "const int* __desc"), C.c_void_p, "desc"))
            params.append(Param("__shiftc", "const int __shiftc", C.c_int32, "shiftc"))
        if sp.aux == "rkeys":
            params.append(Param("__keys", "unsigned* __keys", C.c_void_p, "keys"))
            params.append(Param("__vals", "unsigned long long* __vals", C.c_void_p, "vals"))
            params.append(Param("__len", "const appy::i64 __len", C.c_int64, "entries"))
            params.append(Param("__nx", "const appy::i64 __nx", C.c_int64, "nx"))
            params.append(Param("__lbits", "const int __lbits", C.c_int32, "lbits"))
            params.append(Param("__flag", "long long* __flag", C.c_void_p, "flag"))
        if sp.aux == "xcells":
            # (nothing the kernel stores to overlaps the plan: with `__restrict__` the starts of the cells, read once per run
            #  of tiles, come through the scalar cache and no vector load in flight has to be waited for)
            params.append(Param("__ent", "const unsigned long long* __restrict__ __ent", C.c_void_p, "ent"))
            params.append(Param("__cstart", "const unsigned* __restrict__ __cstart", C.c_void_p, "cstart"))
            params.append(Param("__tbase", "const unsigned* __restrict__ __tbase", C.c_void_p, "tbase"))
            params.append(Param("__rstream", "const unsigned* __restrict__ __rstream", C.c_void_p, "rstream"))
            params.append(Param("__ncell", "const appy::i64 __ncell", C.c_int64, "ncell"))
            params.append(Param("__split", "const appy::i64 __split", C.c_int64, "split"))
            params.append(Param("__order", "const unsigned* __restrict__ __order", C.c_void_p, "order"))
            params.append(Param("__norder", "const appy::i64 __norder", C.c_int64, "norder"))
            params.append(Param("__gwidth", "const appy::i64 __gwidth", C.c_int64, "gwidth"))
            params.append(Param("__colbits", "const int __colbits", C.c_int32, "colbits"))
            params.append(Param("__nx", "const appy::i64 __nx", C.c_int64, "nx"))
            params.append(Param("__scratch", "double* __scratch", C.c_void_p, "scratch"))
        if sp.aux == "group" and sp.skip_long:
            params.append(Param("__counts", "const int* __counts", C.c_void_p, "counts"))
            params.append(Param("__base", "const int __base", C.c_int32, "base"))
        if sp.aux == "group":
            params.append(Param("__len", "const appy::i64 __len", C.c_int64, "entries"))
            params.append(Param("__rowmax", "const appy::i64 __rowmax", C.c_int64, "rowmax"))
            params.append(Param("__hint", "long long* __hint", C.c_void_p, "hint"))
        if sp.skip_long and sp.aux != "group":
            params.append(Param("__rowmax", "const appy::i64 __rowmax", C.c_int64, "rowmax"))
        if sp.aux == "cells":
            params.append(Param("__scratch", "double* __scratch", C.c_void_p, "scratch"))
        if sp.aux == "group" or sp.guard:
            params.append(Param("__flag", ("long long* __flag" if sp.aux == "group" else "const long long* __flag"), C.c_void_p, "flag"))
        if sp.aux == "bins" or sp.rows == "mixed":
            params.append(Param("__m", "const appy::i64 __m", C.c_int64, "m"))
            params.append(Param("__base", "const int __base", C.c_int32, "base"))
        if sp.aux == "bins":
            for k in range(3):
                params.append(Param(f"__t{k}", f"const appy::i64 __t{k}", C.c_int64, "threshold", dim=k))
        if sp.rows == "mixed":
            for k in range(4):
                params.append(Param(f"__wl{k}", f"const int __wl{k}", C.c_int32, "widthlog", dim=k))
            params.append(Param("__skip3", "const appy::i64 __skip3", C.c_int64, "skip"))
            params.append(Param("__hint", "long long* __hint", C.c_void_p, "hint"))
            params.append(Param("__tlo", "const appy::i64 __tlo", C.c_int64, "tlo"))
            params.append(Param("__thi", "const appy::i64 __thi", C.c_int64, "thi"))
        params.append(Param("__lo", "const appy::i64 __lo", C.c_int64, "lo"))
        params.append(Param("__hi", "const appy::i64 __hi", C.c_int64, "hi"))
        return params

    # ---- driver ------------------------------------------------------------------------
    def _emit_body(self):
        self.lines = []
        self.ind = 1
        self.counter = 0
        self.ex.load_subst = {}
        self.ex.sites = []
        self.store_subst = {}
        self.partials = {}
        self.lds_plan = None
        self.rc_slots, self.rc_filled = {}, set()
        for r in self.a.outer_reductions:
            self.w(f"{r.ty.c} {r.acc} = {self._outer_identity(r)};")
        if self.spec.kind == "flat":
            self._body_flat()
        elif self.spec.kind == "strip":
            self._body_strip()
        else:
            self._body_team()
        self._epilogue()

    def build(self, header: str) -> KernelSource:
        # names of shapes produced by array-statement lowering act as scalars
        for _pass in range(8):
            self.dirty = False
            self._emit_body()
            if not self.dirty:
                break
        else:
            raise Unsupported("types of local variables do not settle")
        body = "\n".join(self.lines)
        self.used_scalars = set()
        for sc in self.a.scalars.values():
            if _word_in(cname(sc.name), body) or sc.name in self.shadowed:
                self.used_scalars.add(sc.name)
        params = self._params()
        sig = ",\n    ".join(p.ctype_decl for p in params)
        text = (
            f"{header}\n"
            f"// kernel for {self.name}: {self.spec.tag()}\n"
            f'extern "C" __global__ void __launch_bounds__({self.spec.block})\n'
            f"_{self.name}(\n    {sig})\n{{\n{body}\n}}\n"
        )
        return KernelSource(
            name="_" + self.name,
            text=text,
            params=params,
            spec=self.spec,
            reductions=list(self.a.outer_reductions),
            stored_arrays=sorted(n for n in self.a.stored if n in self.a.arrays),
            bound_checks=list(self.a.bound_checks),
            sites=list(self.ex.sites),
            lane_step_bytes=getattr(self, "lane_step_bytes", 0),
        )


def _word_in(word: str, text: str) -> bool:
    import re

    return re.search(r"(?<![A-Za-z0-9_])" + re.escape(word) + r"(?![A-Za-z0-9_])", text) is not None


def _copy(node):
    import copy

    return copy.deepcopy(node)


class _Rename(ast.NodeTransformer):
    def __init__(self, old, new):
        self.old, self.new = old, new

    def visit_Name(self, node):
        if node.id == self.old:
            return ast.copy_location(ast.Name(id=self.new, ctx=node.ctx), node)
        return node
