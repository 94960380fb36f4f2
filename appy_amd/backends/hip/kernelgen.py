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
"""
from __future__ import annotations

import ast
import ctypes as C
from dataclasses import dataclass, field

from ...frontend import loop_ir
from . import dtypes as T
from .dtypes import Ty
from .exprs import ArrayParam, ExprEmitter, cast, cname, truth

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
class OuterReduction:
    key: str             # e.g. 's[0]'
    op: str
    array: str
    index: int
    ty: Ty               # type of the register accumulators (at least 32 bits wide)
    acc: str             # register name
    elem_ty: Ty = None   # type of the array element the totals are combined into


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


class Unsupported(NotImplementedError):
    pass


def _elts(sub: ast.Subscript):
    return sub.slice.elts if isinstance(sub.slice, ast.Tuple) else [sub.slice]


def _uses_name(node, name: str) -> bool:
    return any(isinstance(n, ast.Name) and n.id == name for n in ast.walk(node))


def _var_offset(node, var: str):
    """``var`` -> 0, ``var + 3`` -> 3, ``var - 1`` -> -1, else None."""
    if isinstance(node, ast.Name) and node.id == var:
        return 0
    if isinstance(node, ast.BinOp) and isinstance(node.op, (ast.Add, ast.Sub)):
        l, r = node.left, node.right
        if isinstance(l, ast.Name) and l.id == var and isinstance(r, ast.Constant) and type(r.value) is int:
            return r.value if isinstance(node.op, ast.Add) else -r.value
        if (isinstance(node.op, ast.Add) and isinstance(r, ast.Name) and r.id == var
                and isinstance(l, ast.Constant) and type(l.value) is int):
            return l.value
    return None


def _affine_in(node, var: str, scalars) -> bool:
    """True if ``node`` is an affine expression of the loop variable ``var`` with integer
    constants and by-value scalars as coefficients (``2 * i + 1``, ``n - 1 - i``, ``-i``) and
    does mention ``var``: its extreme values over a range are taken at the ends of the range."""
    def walk(n):
        """(is affine, mentions var)"""
        if isinstance(n, ast.Constant):
            return type(n.value) is int, False
        if isinstance(n, ast.Name):
            return (n.id == var or n.id in scalars), n.id == var
        if isinstance(n, ast.UnaryOp) and isinstance(n.op, (ast.USub, ast.UAdd)):
            return walk(n.operand)
        if isinstance(n, ast.BinOp) and isinstance(n.op, (ast.Add, ast.Sub, ast.Mult)):
            (la, lv), (ra, rv) = walk(n.left), walk(n.right)
            if not (la and ra) or (isinstance(n.op, ast.Mult) and lv and rv):
                return False, False
            return True, lv or rv
        return False, False

    ok, uses = walk(node)
    return ok and uses


def guarded_nodes(stmts) -> set:
    """ids of the subscripts that the program evaluates only under a condition:
    in the arms of ``a if c else b``, after the first operand of ``and`` / ``or``
    and of a comparison chain, in the bodies of ``if`` / ``while`` statements and
    of nested loops (which may run zero times).  Such an access may lie outside
    its array when the condition is false (``u[i - 1] if i > 0 else 0.0``), so it
    must not be executed early."""
    out = set()

    def mark(node):
        for n in ast.walk(node):
            if isinstance(n, ast.Subscript):
                out.add(id(n))

    def visit(node):
        if isinstance(node, ast.IfExp):
            mark(node.body)
            mark(node.orelse)
        elif isinstance(node, ast.BoolOp):
            for v in node.values[1:]:
                mark(v)
        elif isinstance(node, ast.Compare) and len(node.comparators) > 1:
            for v in node.comparators[1:]:
                mark(v)
        elif isinstance(node, (ast.If, ast.While)):
            for st in node.body + node.orelse:
                mark(st)
            if isinstance(node, ast.While):
                mark(node.test)
        elif isinstance(node, ast.For):
            for st in node.body:
                mark(st)
        for child in ast.iter_child_nodes(node):
            visit(child)

    def leaves_early(node) -> bool:
        """The statement may end the iteration it belongs to (``continue`` / ``break``
        not enclosed in a loop of its own)."""
        if isinstance(node, (ast.Continue, ast.Break)):
            return True
        if isinstance(node, (ast.For, ast.While)):
            return False
        return any(leaves_early(c) for c in ast.iter_child_nodes(node))

    def visit_block(block):
        skipped = False
        for st in block:
            if skipped:
                mark(st)
            visit(st)
            skipped = skipped or leaves_early(st)

    def visit_blocks(node):
        for f in ("body", "orelse"):
            sub = getattr(node, f, None)
            if isinstance(sub, list) and sub and isinstance(sub[0], ast.stmt):
                visit_block(sub)
                for st in sub:
                    visit_blocks(st)

    visit_block(stmts)
    for st in stmts:
        visit_blocks(st)
    return out


def skips_iterations(stmts) -> bool:
    """True if the body holds a ``continue`` that ends an iteration of the loop
    the body belongs to (not of a loop nested in it)."""
    for st in stmts:
        if isinstance(st, ast.Continue):
            return True
        if isinstance(st, (ast.For, ast.While)):
            continue
        for f in ("body", "orelse"):
            sub = getattr(st, f, None)
            if isinstance(sub, list) and sub and isinstance(sub[0], ast.stmt) and skips_iterations(sub):
                return True
    return False


def _has_simd_loop(stmts) -> bool:
    for st in stmts:
        for n in ast.walk(st):
            if isinstance(n, ast.For) and "simd" in (getattr(n, "pragma", None) or {}):
                return True
    return False


class LoopAnalysis:
    """Facts about a loop nest that do not depend on the launch shape."""

    def _fully_overwritten(self):
        """Arrays of which the loop stores every element it covers without reading any:
        ``X[i] = e`` (1-D) or ``for j in range(0, n): X[i, j] = e`` (2-D rows) as
        unconditional statements of the body.  ``{name: None}`` for the 1-D form,
        ``{name: extent node of the inner loop}`` for the row form.  When the outer
        range then spans the whole first dimension (and the inner loop the second),
        a host copy of such an array need not be uploaded before the launch."""
        if skips_iterations(self.outer.body):
            return {}
        out = {}
        loaded = {n.value.id for n in ast.walk(self.outer)
                  if isinstance(n, ast.Subscript) and isinstance(n.ctx, ast.Load) and isinstance(n.value, ast.Name)}
        for st in self.outer.body:
            if isinstance(st, ast.Assign) and isinstance(st.targets[0], ast.Subscript):
                t = st.targets[0]
                el = _elts(t)
                if (isinstance(t.value, ast.Name) and t.value.id in self.arrays and t.value.id not in loaded
                        and len(el) == 1 and isinstance(el[0], ast.Name) and el[0].id == self.var):
                    out[t.value.id] = None
            elif (isinstance(st, ast.For) and isinstance(st.target, ast.Name) and not st.orelse
                  and isinstance(st.iter.args[0], ast.Constant) and st.iter.args[0].value == 0
                  and not skips_iterations(st.body)):
                jv = st.target.id
                for inner in st.body:
                    if not (isinstance(inner, ast.Assign) and isinstance(inner.targets[0], ast.Subscript)):
                        continue
                    t = inner.targets[0]
                    el = _elts(t)
                    if (isinstance(t.value, ast.Name) and t.value.id in self.arrays and t.value.id not in loaded
                            and len(el) == 2 and isinstance(el[0], ast.Name) and el[0].id == self.var
                            and isinstance(el[1], ast.Name) and el[1].id == jv):
                        out[t.value.id] = st.iter.args[1]
        return out

    def _leader_store_reloaded(self) -> bool:
        """True if some wavefront of a multi-wavefront team could read an array element
        on the wrong side of a store that only the leading wavefront issues.

        Statements outside the shared-out loops run on every wavefront, their stores on
        one.  A store to ``X`` is harmless when every other load of ``X`` in the loop nest
        (a) comes earlier in program order, (b) shares no sequential loop with the store
        (no later iteration reads after it) and (c) stands inside a shared-out loop, whose
        closing barrier every wavefront passes after its loads and before the store
        (in-place updates such as ``B[i, j] = alpha * (B[i, j] + sum_k A[k, i] * B[k, j])``).
        Anything else counts as a reload."""
        shared_out = set()          # ids of the nodes inside shared-out loops
        spread = [n for n in ast.walk(self.outer)
                  if isinstance(n, ast.For) and n is not self.outer and "simd" in (getattr(n, "pragma", None) or {})]
        if not spread:
            parts = _find_strip_parts(self.outer.body, self.var)
            if parts is not None:
                spread = [lp for lp, _ops in parts]
        for lp in spread:
            shared_out.update(id(x) for x in ast.walk(lp))

        order, loops_of = {}, {}    # id(node) -> position of its statement; -> enclosing inner loops
        counter = [0]

        def number(stmts, chain):
            for st in stmts:
                counter[0] += 1
                here = counter[0]
                if isinstance(st, (ast.For, ast.While, ast.If)):
                    header = [st.iter] if isinstance(st, ast.For) else [st.test]
                    for h in header:
                        for x in ast.walk(h):
                            order[id(x)], loops_of[id(x)] = here, chain
                    inner = chain + (id(st),) if isinstance(st, (ast.For, ast.While)) else chain
                    number(st.body, inner)
                    number(st.orelse, inner)
                else:
                    for x in ast.walk(st):
                        order[id(x)], loops_of[id(x)] = here, chain

        number(self.outer.body, ())
        for st in ast.walk(self.outer):
            if not (isinstance(st, ast.Assign) and id(st) not in shared_out):
                continue
            t = st.targets[0]
            if not (isinstance(t, ast.Subscript) and isinstance(t.value, ast.Name) and t.value.id in self.arrays):
                continue
            mine = {id(x) for x in ast.walk(st)}
            for n in ast.walk(self.outer):
                if (isinstance(n, ast.Subscript) and isinstance(n.ctx, ast.Load) and isinstance(n.value, ast.Name)
                        and n.value.id == t.value.id and id(n) not in mine):
                    earlier = order.get(id(n), 1 << 60) < order.get(id(st), -1)
                    apart = not (set(loops_of.get(id(n), ())) & set(loops_of.get(id(st), ())))
                    if not (earlier and apart and id(n) in shared_out):
                        return True
        return False

    def _find_strip_split(self):
        """The one shared-out loop of a strip, if the loop nest can run in two phases:
        partial results of that loop over parts of its range (several workgroups per strip,
        for matrices with few columns and many rows), then the rest of the body.  That needs
        a single shared-out loop with reductions, directly in the body of the parallel loop,
        and nothing but scalar assignments in front of it (they are run by both phases)."""
        if not self.strip or len(self.strip) != 1:
            return None
        body = self.outer.body
        at = next((k for k, st in enumerate(body) if isinstance(st, ast.For) and id(st) in self.strip), None)
        if at is None:
            return None
        for st in body[:at]:
            if not (isinstance(st, ast.Assign) and isinstance(st.targets[0], ast.Name)):
                return None
        if not self._set_up_is_repeatable(body[:at], body[at]):
            return None
        return body[at]

    def _set_up_is_repeatable(self, pre, loop) -> bool:
        """The statements in front of a split loop are run by every workgroup that takes a part
        of the loop, and again by the finishing kernel: they must not read what the loop stores."""
        stored = {n.targets[0].value.id for n in ast.walk(loop)
                  if isinstance(n, ast.Assign) and isinstance(n.targets[0], ast.Subscript)
                  and isinstance(n.targets[0].value, ast.Name)}
        return not any(isinstance(n, ast.Name) and n.id in stored for st in pre for n in ast.walk(st))

    def _find_team_split(self):
        """The one ``simd`` loop of a team nest, if the nest can run in two phases (few,
        very long rows: several workgroups share a row): a single ``simd`` loop, directly in
        the body of the parallel loop, with nothing but scalar assignments in front of it."""
        if self.kind != "team" or not self.multi_wave_ok:
            return None
        loops = [n for n in ast.walk(self.outer)
                 if isinstance(n, ast.For) and n is not self.outer and "simd" in (getattr(n, "pragma", None) or {})]
        if len(loops) != 1 or not any(loops[0] is st for st in self.outer.body):
            return None
        body = self.outer.body
        at = next(k for k, st in enumerate(body) if st is loops[0])
        for st in body[:at]:
            if not (isinstance(st, ast.Assign) and isinstance(st.targets[0], ast.Name)):
                return None
        for key in loop_ir.reductions_of(loops[0]):
            if not key.isidentifier():
                return None
        if not self._set_up_is_repeatable(body[:at], loops[0]):
            return None
        return loops[0]

    def _find_ragged(self):
        """``(loop, gather)`` when the rows of a team nest can be sorted by the trip count of
        their ``simd`` loop before they run (CSR rows): the nest has the two-phase form (scalar
        set-up, one ``simd`` loop directly in the body, the rest), the bounds of that loop come
        out of the set-up, and nothing else ties the iterations together.  ``gather`` is
        ``(X, IDX)`` when the loop reads ``X[IDX[j]]`` with ``j`` its own variable, ``X`` and
        ``IDX`` one-dimensional and not stored to: long rows can then be walked one stripe of
        ``X`` at a time."""
        loop = self.team_split
        if loop is None or self.outer_reductions or skips_iterations(self.outer.body):
            return None
        lo, hi, _ = loop.iter.args
        if not any(isinstance(n, ast.Name) and (n.id in self.assigned or n.id == self.var)
                   for b in (lo, hi) for n in ast.walk(b)):
            return None
        # the sorting kernel and the kernels that run the rows each evaluate the set-up and the bounds of a row;
        # a body that stores to an array they read (`ln[i] = 0` after a loop over `range(ln[i])`) would have a
        # row that has run already classified anew, and run again
        body = self.outer.body
        at = next(k for k, st in enumerate(body) if st is loop)
        read_first = {n.id for st in body[:at] for n in ast.walk(st) if isinstance(n, ast.Name)}
        read_first |= {n.id for b in (lo, hi) for n in ast.walk(b) if isinstance(n, ast.Name)}
        if read_first & set(self.stored):
            return None
        jv = loop.target.id
        pairs = set()
        for n in ast.walk(loop):
            if not (isinstance(n, ast.Subscript) and isinstance(n.ctx, ast.Load) and isinstance(n.value, ast.Name)):
                continue
            x = self.arrays.get(n.value.id)
            inner = n.slice
            if (x is None or x.ndim != 1 or x.name in self.stored or not isinstance(inner, ast.Subscript)
                    or not isinstance(inner.value, ast.Name)):
                continue
            idx = self.arrays.get(inner.value.id)
            if (idx is not None and idx.ndim == 1 and idx.ty.is_int and not idx.ty.is_bool and idx.name not in self.stored
                    and isinstance(inner.slice, ast.Name) and inner.slice.id == jv):
                pairs.add((x.name, idx.name))
        gather = next(iter(pairs)) if len(pairs) == 1 else None
        return loop, gather

    def _find_grouping(self):
        """``{"x", "idx", "carried", "stmt", "name"}`` when the ``simd`` loop of a ragged nest is nothing
        but ``s += f(A[j], X[IDX[j]])``: one sum into a scalar whose terms read the gathered operand
        ``X`` through ``IDX``, at most one other array ``A`` (``carried``) at the loop's own position, and
        values that do not change from row to row.  The terms of such a loop can be computed in any
        grouping - by column stripe of ``X`` instead of by row - and added to their rows afterwards.
        ``X``, ``IDX`` and ``A`` have 4-byte elements (``IDX`` signed)."""
        if self.ragged is None or self.ragged[1] is None:
            return None
        loop = self.team_split
        x_name, idx_name = self.ragged[1]
        reds = loop_ir.reductions_of(loop)
        if len(reds) != 1 or len(loop.body) != 1:
            return None
        (name, op), = reds.items()
        st = loop.body[0]
        if not (op == "+" and isinstance(st, ast.Assign) and getattr(st, "reduce", None) == "+"
                and isinstance(st.targets[0], ast.Name) and st.targets[0].id == name):
            return None
        x, idx = self.arrays[x_name], self.arrays[idx_name]
        # (64-bit indices are narrowed where they are loaded: by the kernels that group the elements and by the kernel that
        #  writes the pairs of a row plan; the kernels that run the groups and the plan do not read them)
        if x.ty.size != 4 or x.ty.is_bool or idx.ty.name not in ("int32", "int64"):
            return None
        jv = loop.target.id
        term = loop_ir.reduction_operand(st)
        gather = f"{x_name}[{idx_name}[{jv}]]"
        carried = set()
        covered = set()          # subscript nodes that are (part of) an accepted load

        def accept(n):
            for m in ast.walk(n):
                covered.add(id(m))

        for n in ast.walk(term):
            if id(n) in covered:
                continue
            if isinstance(n, ast.Subscript):
                text = ast.unparse(n)
                if text == gather:
                    accept(n)
                    continue
                arr = self.arrays.get(n.value.id) if isinstance(n.value, ast.Name) else None
                if (arr is None or arr.ndim != 1 or arr.name in self.stored or arr.ty.size != 4 or arr.ty.is_bool
                        or not (isinstance(n.slice, ast.Name) and n.slice.id == jv) or arr.name == idx_name):
                    return None
                carried.add(arr.name)
                accept(n)
            elif isinstance(n, ast.Name) and isinstance(n.ctx, ast.Load):
                if n.id == jv or n.id == self.var or n.id in self.assigned or n.id in self.arrays:
                    return None
            elif isinstance(n, (ast.Lambda, ast.NamedExpr, ast.ListComp, ast.Starred)):
                return None
        if len(carried) > 1 or gather not in ast.unparse(term):
            return None
        return {"x": x_name, "idx": idx_name, "carried": next(iter(carried), None), "stmt": st, "name": name}

    def split_needs_finish(self) -> bool:
        """True if the two-phase form of a team nest needs its second kernel (the loop
        reduces into scalars, or statements follow it)."""
        loop = self.team_split
        return bool(loop_ir.reductions_of(loop)) or self.outer.body[-1] is not loop

    def strip_split_needs_finish(self) -> bool:
        loop = self.strip_split
        return bool(self.strip[id(loop)]) or self.outer.body[-1] is not loop

    def _find_reread(self) -> set:
        """Arrays that one iteration of the parallel loop reads more than once: loaded in two
        or more ``simd`` loops, or in a ``simd`` loop inside a sequential loop whose variable
        the subscript does not use.  Such data should stay in the caches between the passes."""
        seen = {}
        out = set()

        def visit(stmts, seq_vars):
            for st in stmts:
                if isinstance(st, ast.For):
                    if "simd" in (getattr(st, "pragma", None) or {}):
                        for n in ast.walk(st):
                            if (isinstance(n, ast.Subscript) and isinstance(n.ctx, ast.Load) and isinstance(n.value, ast.Name)
                                    and n.value.id in self.arrays):
                                name = n.value.id
                                if seen.setdefault(name, id(st)) != id(st):
                                    out.add(name)
                                if any(not _uses_name(n, v) for v in seq_vars):
                                    out.add(name)
                    else:
                        inner = seq_vars + [st.target.id]
                        visit(st.body, inner)
                        visit(st.orelse, inner)
                elif isinstance(st, (ast.If, ast.While)):
                    visit(st.body, seq_vars)
                    visit(st.orelse, seq_vars)

        visit(self.outer.body, [])
        return out

    def _find_row_cache(self):
        """``(loops, arrays, bounds)`` when an iteration of the parallel loop walks the same rows
        in several ``simd`` loops (soft-max: maximum, sum, quotient; layer norm: mean, variance,
        result): simd loops directly in the body whose bounds do not depend on the iteration
        (``bounds`` lists the distinct ones), and arrays that two or more of them load and none of the nest stores.  With
        few enough vector steps per lane those rows can stay in registers between the loops."""
        if self.kind != "team":
            return None
        # (in a nest whose `for j` can be collapsed into the parallel loop, the loops of that body:
        #  they share a row only when the pairs (i, j) are the iterations)
        body = self.outer.body if self.collapse is None else self.collapse.body
        loops = [st for st in body
                 if isinstance(st, ast.For) and "simd" in (getattr(st, "pragma", None) or {}) and isinstance(st.target, ast.Name)]
        if len(loops) < 2:
            return None
        blocked = set(self.assigned) | set(self.loop_vars) | {self.var} | set(self.arrays)
        loops = [lp for lp in loops
                 if not any(isinstance(n, ast.Name) and n.id in blocked for b in lp.iter.args[:2] for n in ast.walk(b))]
        if len(loops) < 2:
            return None
        # bounds that read differently (the row length of one array, then of another) may still
        # be equal: the launch evaluates them all and keeps rows in registers only if they are
        bounds = {}
        for lp in loops:
            lo, hi = lp.iter.args[:2]
            bounds.setdefault((ast.unparse(lo), ast.unparse(hi)), (lo, hi))
        seen, arrays = {}, set()
        for lp in loops:
            for n in ast.walk(lp):
                if (isinstance(n, ast.Subscript) and isinstance(n.ctx, ast.Load) and isinstance(n.value, ast.Name)
                        and n.value.id in self.arrays and n.value.id not in self.stored):
                    if seen.setdefault(n.value.id, id(lp)) != id(lp):
                        arrays.add(n.value.id)
        if not arrays:
            return None
        return {id(lp) for lp in loops}, arrays, list(bounds.values())

    def _find_collapse(self):
        """The sequential loop ``for j in range(lo, hi)`` that is the whole body of the
        parallel loop, if its iterations are provably independent - then the pairs (i, j)
        may run as one parallel iteration space (3-D stencils written as `parallel i / for j
        / simd k`, row operations on 3-D arrays): with few `i` the chip would otherwise hold
        one team per `i` and nothing else.  None if the nest is not of that form.

        Independence as checked here: the bounds of the loop do not depend on `i` or on
        anything the nest assigns; every scalar the loop assigns is a temporary of one
        iteration (assigned before it is read); every array it stores to is indexed by
        `j + c` in one dimension, the same for all its stores, and loaded - if at all -
        with `j + c` in that dimension too, so that iteration `j` only ever touches its
        own slab; nothing leaves the loop early."""
        body = self.outer.body
        if len(body) != 1 or not isinstance(body[0], ast.For) or "simd" in self.pragma:
            return None
        loop = body[0]
        if getattr(loop, "pragma", None) or loop.orelse or not isinstance(loop.target, ast.Name):
            return None
        it = loop.iter
        if not (isinstance(it, ast.Call) and isinstance(it.func, ast.Name) and it.func.id == "range" and len(it.args) == 3):
            return None
        j = loop.target.id
        if j == self.var or loop_ir.reductions_of(self.outer):
            return None
        assigned = set(self.assigned) | set(self.loop_vars)
        for a in it.args[:2]:
            for n in ast.walk(a):
                if isinstance(n, ast.Name) and (n.id in assigned or n.id in self.arrays):
                    return None
                if isinstance(n, (ast.Subscript, ast.Call)):
                    return None
        # nothing may leave the loop early or skip the rest of an iteration of it
        def leaves(stmts):
            for st in stmts:
                if isinstance(st, (ast.Break, ast.Continue)):
                    return True
                if isinstance(st, ast.If) and (leaves(st.body) or leaves(st.orelse)):
                    return True
            return False
        if leaves(loop.body) or any(isinstance(n, ast.While) for n in ast.walk(loop)):
            return None
        # scalars: temporaries of one iteration
        names = []
        for n in ast.walk(loop):
            if isinstance(n, ast.Assign) and isinstance(n.targets[0], ast.Name) and n.targets[0].id not in names:
                names.append(n.targets[0].id)
            elif isinstance(n, ast.For) and n is not loop and n.target.id not in names:
                names.append(n.target.id)
        if j in names or self.var in names:
            return None
        for name in names:
            first = next((st for st in loop.body if _uses_name(st, name)), None)
            if isinstance(first, ast.For) and first.target.id == name and not any(_uses_name(a, name) for a in first.iter.args):
                continue
            if not (isinstance(first, ast.Assign) and isinstance(first.targets[0], ast.Name)
                    and first.targets[0].id == name and not _uses_name(first.value, name)):
                return None
        # arrays: iteration j stays inside its own slab of everything the loop stores to
        slab = {}       # array -> (dimension, offset)
        for n in ast.walk(loop):
            if isinstance(n, ast.Assign) and isinstance(n.targets[0], ast.Subscript):
                t = n.targets[0]
                if not (isinstance(t.value, ast.Name) and t.value.id in self.arrays):
                    return None
                where = [(d, _var_offset(e, j)) for d, e in enumerate(_elts(t)) if _var_offset(e, j) is not None]
                if len(where) != 1 or slab.setdefault(t.value.id, where[0]) != where[0]:
                    return None
        if not slab:
            return None
        for n in ast.walk(loop):
            if isinstance(n, ast.Subscript) and isinstance(n.value, ast.Name) and n.value.id in slab:
                d, off = slab[n.value.id]
                idx = _elts(n)
                if d >= len(idx) or _var_offset(idx[d], j) != off:
                    return None
                if any(_uses_name(e, j) for k, e in enumerate(idx) if k != d):
                    return None
        return loop

    def _find_strip(self):
        """``{id(loop): {scalar: op}}`` for the inner loops that a *strip* kernel
        shares out between wavefronts, or None if the loop nest does not suit that
        shape.  In a strip the 64 lanes of a wavefront take 64 consecutive outer
        iterations and the wavefronts of the workgroup form the team of each of
        them; it is the coalesced mapping when the inner loops walk down columns
        (``A[j, i]``: the parallel variable indexes the contiguous dimension).

        Shared-out loops are the ``simd`` loops and, when the body has no ``simd``
        loop, a single sequential loop that only folds values into scalars.  They
        end in workgroup barriers, so they may only stand where every lane of the
        workgroup arrives together: directly in the body or inside sequential
        loops whose bounds are the same for every outer iteration - never under
        ``if`` / ``while`` - and nothing outside them may ``break`` / ``continue``."""
        body = self.outer.body
        assigned = set(self.assigned) | {self.var}
        spread = {}

        def loop_free(stmts, allow_continue):
            stop = (ast.For, ast.While, ast.Break) if allow_continue else (ast.For, ast.While, ast.Break, ast.Continue)
            return not any(isinstance(n, stop) for st in stmts for n in ast.walk(st))

        def has_simd(node):
            return any(isinstance(n, ast.For) and n is not self.outer and "simd" in (getattr(n, "pragma", None) or {})
                       for n in ast.walk(node))

        def walk(stmts) -> bool:
            if skips_iterations(stmts):
                return False                    # some lanes would miss the barriers that follow
            for st in stmts:
                if isinstance(st, ast.For) and "simd" in (getattr(st, "pragma", None) or {}):
                    if st.orelse or not isinstance(st.target, ast.Name) or not loop_free(st.body, True):
                        return False
                    if set(st.pragma) - {"simd", "reduction"}:
                        return False
                    ops = {}
                    for key, op in loop_ir.reductions_of(st).items():
                        if not key.isidentifier():
                            return False
                        ops[key] = op
                    if any(_uses_name(a, n) for a in st.iter.args for n in ops):
                        return False
                    spread[id(st)] = ops
                elif isinstance(st, ast.For):
                    if has_simd(st):
                        if st.orelse or any(_uses_name(a, n) for a in st.iter.args for n in assigned):
                            return False        # lanes would reach the barriers inside a different number of times
                        if any(isinstance(n, ast.Break) for n in ast.walk(st)) or not walk(st.body):
                            return False
                elif isinstance(st, (ast.If, ast.While)) and has_simd(st):
                    return False
            return True

        if has_simd(self.outer):
            if not walk(body):
                return None
        else:
            parts = _find_strip_parts(body, self.var)
            if parts is None:
                return None
            for loop, ops in parts:
                for st in loop.body:
                    if isinstance(st.targets[0], ast.Name):
                        st.reduce = ops[st.targets[0].id]
                spread[id(loop)] = ops
        if not spread:
            return None
        # profitability: down the columns, never along a row of a matrix
        good = bad = False
        for n in ast.walk(self.outer):
            if isinstance(n, ast.For) and id(n) in spread:
                jv = n.target.id
                for st in n.body:
                    for sub in ast.walk(st):
                        if isinstance(sub, ast.Subscript) and isinstance(sub.value, ast.Name) and sub.value.id in self.arrays:
                            last = _elts(sub)[-1]
                            if _uses_name(last, self.var):
                                good = True
                            if _uses_name(last, jv) and self.arrays[sub.value.id].ndim >= 2:
                                bad = True
        return spread if good and not bad else None

    def __init__(self, tree: ast.Module, val_arrays: dict, val_scalars: dict):
        self.tree = tree
        self.outer = loop_ir.outer_loop(tree)
        if not (isinstance(self.outer.iter, ast.Call) and isinstance(self.outer.iter.func, ast.Name)
                and self.outer.iter.func.id in ("range", "prange") and len(self.outer.iter.args) == 3):
            raise Unsupported(f"Parallel loops iterate over range(...): {ast.unparse(self.outer.iter)}")
        if not isinstance(self.outer.target, ast.Name):
            raise Unsupported("The loop variable must be a plain name")
        self.var = self.outer.target.id
        self.pragma = getattr(self.outer, "pragma", None) or {"parallel_for": True}
        self.lo_node, self.hi_node, _ = self.outer.iter.args
        self.arrays = val_arrays      # name -> ArrayParam
        self.scalars = val_scalars    # name -> ScalarParam

        self.assigned = []            # local names in order of first assignment
        self.loop_vars = []
        self.stored = set()
        for n in ast.walk(self.outer):
            if isinstance(n, ast.Assign):
                t = n.targets[0]
                if isinstance(t, ast.Name) and t.id not in self.assigned:
                    self.assigned.append(t.id)
                elif isinstance(t, ast.Subscript) and isinstance(t.value, ast.Name):
                    self.stored.add(t.value.id)
            elif isinstance(n, ast.For):
                if isinstance(n.target, ast.Name):
                    self.loop_vars.append(n.target.id)
                else:
                    raise Unsupported("Loop variables must be plain names")
            elif isinstance(n, (ast.Return, ast.With, ast.Try, ast.FunctionDef, ast.Lambda, ast.ListComp, ast.Yield)):
                raise Unsupported(f"Statement not supported in a kernel: {type(n).__name__}")
        for name in self.stored:
            if name in self.arrays:
                self.arrays[name].stored = True
            elif name not in self.assigned:
                raise Unsupported(f"`{name}` is subscripted but is not an array argument")

        is_simd = "simd" in self.pragma
        self.kind = "flat" if (is_simd or not _has_simd_loop(self.outer.body)) else "team"

        # sequential loops that every lane of a flat kernel runs by itself; if they index the
        # contiguous dimension with the parallel variable, adjacent lanes must take adjacent iterations
        nested = [n for st in self.outer.body for n in ast.walk(st) if isinstance(n, (ast.For, ast.While))]
        self.lane_loops = self.kind == "flat" and bool(nested)
        self.lane_loops_strided = self.lane_loops and any(
            isinstance(n, ast.Subscript) and _uses_name(_elts(n)[-1], self.var)
            for lp in nested for st in lp.body for n in ast.walk(st))

        self.overwritten = self._fully_overwritten()

        # Shapes whose team spans several wavefronts (strips, workgroup teams) run statements
        # outside the shared-out loops on every wavefront but store from one of them only.
        # An array stored that way and read by another statement would need a barrier between
        # the two (the other wavefronts may read too early or too late), so such loop nests
        # keep to teams inside one wavefront, where program order is enough.
        self.multi_wave_ok = not self._leader_store_reloaded()
        self.strip = self._find_strip() if self.multi_wave_ok else None
        self.collapse = self._find_collapse() if self.kind == "team" else None
        self.strip_split = self._find_strip_split()
        self.team_split = self._find_team_split()
        self.reread = self._find_reread()
        self.row_cache = self._find_row_cache()

        # reductions of the parallel loop: constant-subscript elements of arrays
        self.outer_reductions = []
        for key, op in loop_ir.reductions_of(self.outer).items():
            try:
                node = ast.parse(key, mode="eval").body
            except SyntaxError:
                continue
            if (isinstance(node, ast.Subscript) and isinstance(node.value, ast.Name)
                    and node.value.id in self.arrays and isinstance(node.slice, ast.Constant)
                    and type(node.slice.value) is int and self.arrays[node.value.id].ndim == 1):
                arr = self.arrays[node.value.id]
                acc_ty = arr.ty
                if arr.ty.size < 4:
                    # 8- and 16-bit elements: registers and cross-lane steps work on 32 bits; sums
                    # wrap to the element type at the end exactly as they would have step by step
                    acc_ty = T.F32 if arr.ty.is_float else (T.Ty("uint32") if arr.ty.kind == "u" else T.I32)
                if arr.ty.is_bool:
                    op = {"+": "max", "*": "min"}.get(op, op)       # NumPy's bool arithmetic: or / and
                self.outer_reductions.append(
                    OuterReduction(key, op, arr.name, node.slice.value, acc_ty, f"__acc{len(self.outer_reductions)}",
                                   arr.ty)
                )

        # accesses indexed directly by the parallel loop variable: checked on
        # the host against the array extents before every launch
        # Accesses under a condition of the program are not checked (the condition is
        # their guard); those a flat kernel may want to load early are listed apart, and
        # the host picks the variant that leaves them in place when they could leave
        # their array.
        self.bound_checks = []
        self.guarded_checks = []
        # other affine subscripts of the parallel variable (`a[2 * i]`, `a[n - 1 - i]`, `a[-i]`):
        # (array, dimension, expression); the host evaluates them at both ends of the range
        self.affine_checks = []
        fixed_scalars = {k for k, p in self.scalars.items() if k not in self.assigned and p.ty.kind in "iub"}
        guarded = guarded_nodes(self.outer.body)
        for n in ast.walk(self.outer):
            if isinstance(n, ast.Subscript) and isinstance(n.value, ast.Name) and n.value.id in self.arrays:
                into = self.guarded_checks if id(n) in guarded else self.bound_checks
                for d, e in enumerate(_elts(n)):
                    off = _var_offset(e, self.var)
                    if off is not None and (n.value.id, d, off) not in into:
                        into.append((n.value.id, d, off))
                    elif (off is None and id(n) not in guarded and not isinstance(e, ast.Slice)
                          and _affine_in(e, self.var, fixed_scalars)):
                        item = (n.value.id, d, ast.unparse(e))
                        if item not in self.affine_checks:
                            self.affine_checks.append(item)
        self.ragged = self._find_ragged()
        self.grouping = self._find_grouping()


def _partial_type(ty: Ty) -> Ty:
    """Type of the per-lane partial results of a reduction: registers and cross-lane
    steps are 32 or 64 bits wide, so 16-bit floats accumulate in float32 (rounded once,
    when the team combines) and 8/16-bit integers and flags in 32-bit integers (sums wrap
    to the narrow type at the end exactly as they would have step by step)."""
    if ty.size >= 4:
        return ty
    if ty.is_float:
        return T.F32
    return Ty("uint32") if ty.kind == "u" else T.I32


def _partial_identity(op: str, ty: Ty, pty: Ty) -> str:
    """Neutral element of ``op`` over ``ty``, written in the partial type ``pty``."""
    if pty == ty or ty.is_float:
        return T.identity_literal(op, pty)
    if ty.is_bool:
        return "0" if op in ("max", "+") else "1"
    return f"(({pty.c}){T.identity_literal(op, ty)})"


def _find_strip_parts(body, var):
    """``[(loop, {scalar: op}), ...]`` if the body of a parallel loop is scalar set-up,
    then sequential loops with independent iterations - they fold values into scalars with
    a reduction operator (``s += A[j, i] * y[j]``) without looking at the running value,
    and / or store to arrays, each iteration inside its own slab (``C[j, i] = A[j, i] * f[i]``:
    the loop variable, plus a constant, in one dimension of every subscript of that array) -
    with nothing but scalar assignments between them (``mu = s / n``), then anything without
    loops: column reductions and column updates written without ``simd``.  None otherwise."""
    at = [k for k, st in enumerate(body) if isinstance(st, (ast.For, ast.While))]
    if not at or not all(isinstance(body[k], ast.For) for k in at):
        return None
    found = []
    for k in at:
        loop = body[k]
        if loop.orelse or not isinstance(loop.target, ast.Name) or (getattr(loop, "pragma", None) or {}):
            return None
        for st in loop.body:    # `continue` ends one iteration of the inner loop, wherever that runs
            if any(isinstance(n, (ast.For, ast.While, ast.Break)) for n in ast.walk(st)):
                return None
        ops = {}
        k_var = loop.target.id
        slab = {}           # array stored in the loop -> (dimension, offset) of the loop variable in its subscripts
        folds = []
        for st in loop.body:
            if not isinstance(st, ast.Assign):
                return None
            tgt = st.targets[0]
            if isinstance(tgt, ast.Name):
                op = loop_ir.reduction_operator(st)
                if op is None or ops.setdefault(tgt.id, op) != op:
                    return None
                folds.append(st)
            elif isinstance(tgt, ast.Subscript) and isinstance(tgt.value, ast.Name):
                # a store: iterations are independent when each one stays in its own slab of the array
                where = [(d, _var_offset(e, k_var)) for d, e in enumerate(_elts(tgt)) if _var_offset(e, k_var) is not None]
                if len(where) != 1 or slab.setdefault(tgt.value.id, where[0]) != where[0]:
                    return None
            else:
                return None
        for name in ops:    # the running value is not looked at inside the loop
            if any(_uses_name(loop_ir.reduction_operand(s2), name) for s2 in folds):
                return None
            if any(_uses_name(s2.value, name) for s2 in loop.body if s2 not in folds):
                return None
        for n in ast.walk(loop):
            if isinstance(n, ast.Subscript) and isinstance(n.value, ast.Name) and n.value.id in slab:
                d, off = slab[n.value.id]
                idx = _elts(n)
                if d >= len(idx) or _var_offset(idx[d], k_var) != off or any(
                        _uses_name(e, k_var) for q, e in enumerate(idx) if q != d):
                    return None
        if not (ops or slab) or any(_uses_name(a, n) for a in loop.iter.args for n in ops):
            return None
        found.append((loop, ops))
    for k, st in enumerate(body):
        if k in at:
            continue
        if any(isinstance(n, (ast.Break, ast.Continue)) for n in ast.walk(st)):
            return None
        if k < at[-1] and not (isinstance(st, ast.Assign) and isinstance(st.targets[0], ast.Name)):
            return None     # run by every wavefront of the strip: values only, no effects
    return found


class KernelBuilder:
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
            pty = _partial_type(ty)
            self.partials[name] = (p, pty)
            self.w(f"{pty.c} {p} = {_partial_identity(op, ty, pty)};")
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
            pty = _partial_type(ty)
            p = self.fresh(f"part_{name}_")
            typed[name] = (p, pty)
            self.partials[name] = (p, pty)
            self.w(f"{pty.c} {p} = {_partial_identity(op, ty, pty)};")
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

    # ---- rows binned by the trip count of their simd loop ----------------------------------------
    # Classes: 0..3 by rising trip count (thresholds are kernel arguments).  The rows of one class,
    # the base class, are taken in their natural order; the rows of the others are listed by the
    # binning kernel: `__rows[c * __m + k]`, `__counts[c]` of them.
    def _split_iteration(self, idx_code: str, guard=None, upto=None):
        """One iteration, the scalar set-up first; ``guard`` (a C condition that may use
        ``__trip``, the trip count of the simd loop) decides whether the rest runs."""
        a = self.a
        body = a.outer.body
        at = next(k for k, st in enumerate(body) if st is a.team_split)
        self.w("{")
        self.ind += 1
        self.w(f"const appy::i64 {cname(a.var)} = {idx_code};")
        self._declare_locals()
        self.block(body[:at])
        if guard is not None:
            lo, hi = self._range_args(a.team_split)
            self.w(f"const appy::i64 __trip = ({hi}) - ({lo});")
            self.w(f"if ({guard}) {{")
            self.ind += 1
        self.block(body[at:upto])
        if guard is not None:
            self.ind -= 1
            self.w("}")
        self.ind -= 1
        self.w("}")

    def _body_bins(self):
        """The kernel that sorts rows into classes: one lane per row runs the set-up, the rows of
        every class but the base class are appended to the list of their class (one reservation
        per workgroup, chunk and class).  It also clears the counters of the next launch."""
        RPT = 4
        B = self.spec.block
        var = self.a.var
        self.ex.locals[var] = T.WEAK_INT
        self.mode = "lane"
        self.w("__shared__ int __cnt[4];")
        self.w("__shared__ int __first[4];")
        self.w("if (blockIdx.x == 0 && threadIdx.x < 136) __zero[threadIdx.x] = 0;     // 8 counters, 64 part loads of 8 bytes")
        self.w(f"for (appy::i64 __c0 = __lo + (appy::i64)blockIdx.x * {B * RPT}; __c0 < __hi; __c0 += (appy::i64)gridDim.x * {B * RPT}) {{")
        self.ind += 1
        self.w("if (threadIdx.x < 4) __cnt[threadIdx.x] = 0;")
        self.w("__syncthreads();")
        self.w(f"int __cl[{RPT}], __pos[{RPT}];")
        self.w("#pragma unroll")
        self.w(f"for (int __r = 0; __r < {RPT}; ++__r) {{")
        self.ind += 1
        self.w(f"const appy::i64 __i = __c0 + (appy::i64)__r * {B} + threadIdx.x;")
        self.w("__cl[__r] = -1;")
        self.w("__pos[__r] = 0;")
        self.w("if (__i < __hi) {")
        self.ind += 1
        body = self.a.outer.body
        at = next(k for k, st in enumerate(body) if st is self.a.team_split)
        self.w(f"const appy::i64 {cname(var)} = __i;")
        self._declare_locals()
        self.block(body[:at])
        lo, hi = self._range_args(self.a.team_split)
        self.w(f"const appy::i64 __trip = ({hi}) - ({lo});")
        self.w("const int __c = __trip <= __t0 ? 0 : __trip <= __t1 ? 1 : __trip <= __t2 ? 2 : 3;")
        self.w("if (__c != __base) { __cl[__r] = __c; __pos[__r] = atomicAdd(&__cnt[__c], 1); }")
        self.ind -= 1
        self.w("}")
        self.ind -= 1
        self.w("}")
        self.w("__syncthreads();")
        self.w("if (threadIdx.x < 4) __first[threadIdx.x] = __cnt[threadIdx.x] ? atomicAdd(&__counts[threadIdx.x], __cnt[threadIdx.x]) : 0;")
        self.w("__syncthreads();")
        self.w("#pragma unroll")
        self.w(f"for (int __r = 0; __r < {RPT}; ++__r) {{")
        self.w(f"    if (__cl[__r] >= 0) __rows[(appy::i64)__cl[__r] * __m + __first[__cl[__r]] + __pos[__r]] = "
               f"(int)(__c0 + (appy::i64)__r * {B} + threadIdx.x);")
        self.w("}")
        self.w("__syncthreads();")
        self.ind -= 1
        self.w("}")

    def _body_mixed(self):
        """Rows of all classes in one kernel: the wavefronts walk a row of slots, first the rows of
        the base class in their natural order (rows of other classes are passed over), then the
        listed rows class by class; the team width of a wavefront follows the class of its slot."""
        NWB = self.spec.block // 64
        var = self.a.var
        self.ex.locals[var] = T.WEAK_INT
        self.w("const int __lid = threadIdx.x & 63;")
        self.w(f"const appy::i64 __wv = (appy::i64)blockIdx.x * {NWB} + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);")
        self.w(f"const appy::i64 __nwv = (appy::i64)gridDim.x * {NWB};")
        prev = "0"
        for c in range(4):
            skip = "__skip3" if c == 3 else "0"
            self.w(f"const appy::i64 __l{c} = (appy::i64)__counts[{c}] - {skip};")
            self.w(f"const appy::i64 __n{c} = (__base == {c}) ? (__hi - __lo) : (__l{c} > 0 ? __l{c} : 0);")
            self.w(f"const appy::i64 __e{c} = {prev} + (((__n{c} << __wl{c}) + 63) >> 6);")
            prev = f"__e{c}"
        # what the classes held this time, left where the host can see it when it stages the next launch
        # (a hint for shaping that launch: which class to take in natural order, whether long rows exist)
        self.w("if (blockIdx.x == 0 && threadIdx.x == 0) {")
        self.w("    const appy::i64 __others = (__base == 0 ? 0 : (appy::i64)__counts[0]) + (__base == 1 ? 0 : (appy::i64)__counts[1]) "
               "+ (__base == 2 ? 0 : (appy::i64)__counts[2]) + (__base == 3 ? 0 : (appy::i64)__counts[3]);")
        for c in range(4):
            self.w(f"    __hint[{c + 1}] = (__base == {c}) ? (__hi - __lo) - __others : (appy::i64)__counts[{c}];")
        self.w("    __hint[0] = 1;")
        self.w("}")
        self.w("for (appy::i64 __v = __wv; __v < __e3; __v += __nwv) {")
        self.ind += 1
        self.w("const int __c = (int)(__v >= __e0) + (int)(__v >= __e1) + (int)(__v >= __e2);")
        self.w("const int __wl = __c == 0 ? __wl0 : __c == 1 ? __wl1 : __c == 2 ? __wl2 : __wl3;")
        self.w("const int __W = 1 << __wl;")
        self.w("const int __lane = __lid & (__W - 1);")
        self.w("const appy::i64 __vb = __c == 0 ? 0 : __c == 1 ? __e0 : __c == 2 ? __e1 : __e2;")
        self.w("const appy::i64 __nc = __c == 0 ? __n0 : __c == 1 ? __n1 : __c == 2 ? __n2 : __n3;")
        self.w("const appy::i64 __t = ((__v - __vb) << (6 - __wl)) + (__lid >> __wl);")
        self.w("if (__t < __nc) {")
        self.ind += 1
        self.w("const appy::i64 __i = (__c == __base) ? (__lo + __t) : "
               "(appy::i64)__rows[(appy::i64)__c * __m + (__c == 3 ? __skip3 : 0) + __t];")
        self.mode = "team"
        self._split_iteration("__i", guard="__c != __base || (__trip > __tlo && __trip <= __thi)")
        self.mode = "lane"
        self.ind -= 1
        self.w("}")
        self.ind -= 1
        self.w("}")

    def _body_listed(self):
        """Kernels over the rows of one list whose simd loop runs in planned parts: the planning
        kernel, the kernel that runs the parts (part p on the workgroups whose number is p modulo 8:
        workgroups go to the eight XCDs in turn, so every L2 sees one stripe of the gathered
        operand), and the finishing kernel."""
        s = self.spec
        W, B, S = s.width, s.block, s.parts
        tpb = B // W
        var = self.a.var
        self.ex.locals[var] = T.WEAK_INT
        self.w(f"const int __lane = threadIdx.x & {W - 1};")
        self.w(f"const appy::i64 __team = threadIdx.x / {W};")
        self.w("const appy::i64 __listed = (appy::i64)__nrows[0];")
        self.w("const appy::i64 __n = __listed < __cap ? __listed : __cap;")
        if s.aux == "plan":
            x_name, idx_name = self.a.ragged[1]
            idx = self.a.arrays[idx_name]
            idx.loaded = True
            # elements per part over all rows: the kernel that runs the parts looks at these before it
            # ties parts to XCDs (columns that crowd into few stripes would leave most XCDs idle)
            self.w(f"__shared__ unsigned long long __work[{S}];")
            self.w(f"if (threadIdx.x < {S}) __work[threadIdx.x] = 0;")
            self.w("__syncthreads();")
            self.w("unsigned long long __mine = 0;      // elements in the part of this lane, over the rows of its team")
            self.w(f"for (appy::i64 __t = (appy::i64)blockIdx.x * {tpb} + __team; __t < __n; __t += (appy::i64)gridDim.x * {tpb}) {{")
            self.ind += 1
            self.mode = "team"
            self.w("{")
            self.ind += 1
            self.w(f"const appy::i64 {cname(var)} = (appy::i64)__rows[__t];")
            self._declare_locals()
            body = self.a.outer.body
            at = next(k for k, st in enumerate(body) if st is self.a.team_split)
            self.block(body[:at])
            lo, hi = self._range_args(self.a.team_split)
            self.w(f"const appy::i64 __rlo = {lo};")
            self.w(f"const appy::i64 __rhi = ({hi}) > __rlo ? ({hi}) : __rlo;")
            # lane p < S - 1 looks for the first position whose index reaches stripe p + 1; a running
            # maximum over the lanes keeps the cuts in order, so that every position lies in exactly
            # one part whatever the order of the indices (sorted rows are cut at the stripes)
            # (the search starts where the cut would lie if the indices were spread evenly and widens its steps from
            #  there - two or three cache lines of indices per cut instead of one per level of a bisection of the whole
            #  row; 0.14 ms of a 3 ms launch were these lines)
            self.w("appy::i64 __b = __rhi;")
            self.w(f"if (__lane < {S - 1} && __rhi > __rlo) {{")
            self.w("    const appy::i64 __target = (appy::i64)(__lane + 1) * __stripe;")
            self.w("    appy::i64 __a = __rlo, __z = __rhi;       // the cut lies in [__a, __z]: indices before __a are below the target")
            self.w(f"    const appy::i64 __guess = __rlo + ((__rhi - __rlo) * (__lane + 1)) / {S};")
            self.w("    appy::i64 __step = 16;")
            self.w(f"    if ((appy::i64){cname(idx_name)}[__guess] < __target) {{")
            self.w("        __a = __guess + 1;")
            self.w("        while (__a < __z) {")
            self.w("            const appy::i64 __p = (__a + __step - 1) < (__z - 1) ? (__a + __step - 1) : (__z - 1);")
            self.w(f"            if ((appy::i64){cname(idx_name)}[__p] < __target) {{ __a = __p + 1; __step *= 4; }} else {{ __z = __p; break; }}")
            self.w("        }")
            self.w("    } else {")
            self.w("        __z = __guess;")
            self.w("        while (__a < __z) {")
            self.w("            const appy::i64 __p = (__z - __step) > __a ? (__z - __step) : __a;")
            self.w(f"            if ((appy::i64){cname(idx_name)}[__p] < __target) {{ __a = __p + 1; break; }} else {{ __z = __p; __step *= 4; }}")
            self.w("        }")
            self.w("    }")
            self.w("    while (__a < __z) {")
            self.w("        const appy::i64 __mid = __a + ((__z - __a) >> 1);")
            self.w(f"        if ((appy::i64){cname(idx_name)}[__mid] < __target) __a = __mid + 1; else __z = __mid;")
            self.w("    }")
            self.w("    __b = __a;")
            self.w("}")
            self.w(f"__b = appy::team_running_max<{W}>(__b, __lane);")
            # (cuts are kept relative to the start of the row: 32 bits are enough whatever the array size)
            self.w("if (__lane == 0) { __bnd[__t] = 0; __start[__t] = __rlo; }")
            self.w(f"const appy::i64 __cut = (__lane < {S - 1} ? __b : __rhi) - __rlo;      // where part __lane ends")
            self.w(f"if (__lane < {S}) __bnd[(appy::i64)(__lane + 1) * __cap + __t] = (int)__cut;")
            self.w(f"const appy::i64 __before = appy::team_lane_below<{W}>(__cut, __lane);")
            self.w(f"if (__lane < {S} && __cut > (__lane ? __before : 0)) __mine += (unsigned long long)(__cut - (__lane ? __before : 0));")
            self.ind -= 1
            self.w("}")
            self.mode = "lane"
            self.ind -= 1
            self.w("}")
            self.w(f"if (__lane < {S} && __mine) atomicAdd(&__work[__lane], __mine);")
            self.w("__syncthreads();")
            self.w(f"if (threadIdx.x < {S} && __work[threadIdx.x]) atomicAdd(&__load[threadIdx.x], __work[threadIdx.x]);")
            return
        self.mode = "team"
        if s.phase == 1:
            # Part p of every row runs on the workgroups whose number is p modulo 8, i.e. on one XCD, whose L2
            # then holds stripe p of the gathered operand and nothing else of it.  That ties the work of an XCD
            # to the elements that fall into its stripes: when one XCD would get more than 1.5 times its share
            # (columns crowded into few stripes), the parts are dealt to all workgroups alike instead, stripe
            # after stripe.
            self.w("unsigned long long __tot = 0, __most = 0;")
            self.w("for (int __x = 0; __x < 8; ++__x) {")
            self.w("    unsigned long long __sum = 0;")
            self.w(f"    for (int __p = __x; __p < {S}; __p += 8) __sum += __load[__p];")
            self.w("    __tot += __sum;")
            self.w("    __most = __sum > __most ? __sum : __most;")
            self.w("}")
            self.w("const bool __even = __most * 16 <= __tot * 3;")
            self.w(f"const appy::i64 __t0 = (__even ? (appy::i64)(blockIdx.x >> 3) : (appy::i64)blockIdx.x) * {tpb} + __team;")
            self.w(f"const appy::i64 __dt = (__even ? (appy::i64)(gridDim.x >> 3) : (appy::i64)gridDim.x) * {tpb};")
            self.w(f"for (appy::i64 __pass = 0; __pass < (__even ? {S // 8} : {S}); ++__pass) {{")
            self.ind += 1
            self.w("const appy::i64 __chunk = __even ? (appy::i64)(blockIdx.x & 7) + 8 * __pass : __pass;")
            self.w("for (appy::i64 __t = __t0; __t < __n; __t += __dt) {")
            self.ind += 1
            body = self.a.outer.body
            at = next(k for k, st in enumerate(body) if st is self.a.team_split)
            self._split_iteration("(appy::i64)__rows[__t]", upto=at + 1)
            self.ind -= 1
            self.w("}")
            self.ind -= 1
            self.w("}")
        else:
            self.w(f"for (appy::i64 __t = (appy::i64)blockIdx.x * {tpb} + __team; __t < __n; __t += (appy::i64)gridDim.x * {tpb}) {{")
            self.ind += 1
            self._split_iteration("(appy::i64)__rows[__t]")
            self.ind -= 1
            self.w("}")
        self.mode = "lane"

    # ---- elements grouped by the stripe of the gathered operand they read -------------------------------
    # Blocks of `Spec.block_rows` rows, one wavefront each.  The grouping kernel writes the elements of a block -
    # the 32 bits of the carried operand, the row within the block (10 bits) and the position within the stripe
    # (22 bits) - over the block's own range of positions, stripe after stripe, and where every stripe
    # starts (`__desc`, `parts + 1` numbers per block).  A cell is one stripe of one block.
    @property
    def GROUP_ROWS(self):
        return self.spec.block_rows

    def _group_setup_types(self):
        """Walks the set-up of an iteration and the term of the sum into a buffer that is thrown away:
        the types of the locals settle as they do in the kernels that run the loop row by row.
        Returns (code of the term with `__cv` / `__cx` for the two loads, its type, partial type)."""
        a, g = self.a, self.a.grouping
        body = a.outer.body
        at = next(k for k, st in enumerate(body) if st is a.team_split)
        kept, self.lines = self.lines, []
        saved_mode, self.mode = self.mode, "lane"
        self.ex.locals[a.team_split.target.id] = T.WEAK_INT
        self.block(body[:at])
        name = g["name"]
        ty = self.ex.locals.get(name)
        if ty is None:
            raise NameError(f"reduction variable `{name}` has no value before the loop")
        jv = a.team_split.target.id
        x, idx = a.arrays[g["x"]], a.arrays[g["idx"]]
        saved = dict(self.ex.load_subst)
        self.ex.load_subst[f"{g['x']}[{g['idx']}[{jv}]]"] = ("__cx", x.ty)
        if g["carried"]:
            self.ex.load_subst[f"{g['carried']}[{jv}]"] = ("__cv", a.arrays[g["carried"]].ty)
        oc, ot = self.ex.emit(loop_ir.reduction_operand(g["stmt"]))
        self.ex.load_subst = saved
        pty = _partial_type(ty)
        self.set_local(name, T.promote(ty, ot))
        self.lines, self.mode = kept, saved_mode
        return oc, ot, pty

    def _body_group(self):
        """The grouping kernel.  Per block: the set-up of its rows (and of the first row of the next
        block) gives the rows' ranges, which must follow one another - otherwise the block is refused
        and the flag raised; a first pass over the elements counts them per stripe, a second pass
        writes each element to its place.  The rank of an element within its stripe comes from
        ballots taken in a fixed order, so the layout does not depend on timing."""
        a, g, S, R = self.a, self.a.grouping, self.spec.parts, self.GROUP_ROWS
        var = a.var
        self.ex.locals[var] = T.WEAK_INT
        self.mode = "lane"
        idx_c = cname(g["idx"])
        a.arrays[g["idx"]].loaded = True
        self._group_wide = a.arrays[g["idx"]].ty.size == 8     # 64-bit indices are narrowed as they are loaded
        car_c = f"reinterpret_cast<const int*>({cname(g['carried'])})" if g["carried"] else None
        body = a.outer.body
        at = next(k for k, st in enumerate(body) if st is a.team_split)
        U = 4       # vectors of four elements per lane and step
        w = self.w
        w("const int __lid = threadIdx.x & 63;")
        w("const int __wvl = threadIdx.x >> 6;")
        w(f"__shared__ int __lp_all[4][{R + 1}];      // where the rows of the block start; the last entry: where it ends")
        w(f"__shared__ int __hq_all[4][{R + 1}];      // where they end")
        w("int* __lp = __lp_all[__wvl];")
        w("int* __hq = __hq_all[__wvl];")
        if self.spec.skip_long:
            # the sorting kernel of this launch has counted the rows of its classes: they go where the host reads them
            # when it stages the next launch (as the kernel over rows of all classes does)
            w("if (blockIdx.x == 0 && threadIdx.x == 0) {")
            w("    const appy::i64 __others = (__base == 0 ? 0 : (appy::i64)__counts[0]) + (__base == 1 ? 0 : (appy::i64)__counts[1]) "
              "+ (__base == 2 ? 0 : (appy::i64)__counts[2]) + (__base == 3 ? 0 : (appy::i64)__counts[3]);")
            for c in range(4):
                w(f"    __hint[{c + 1}] = (__base == {c}) ? (__hi - __lo) - __others : (appy::i64)__counts[{c}];")
            w("    __hint[0] = 1;")
            w("}")
        w(f"const appy::i64 __nblk = (__hi - __lo + {R - 1}) / {R};")
        w("const int __cmask = (1 << __shiftc) - 1;")
        w("const unsigned long long __below = (1ull << __lid) - 1ull;")
        w("for (appy::i64 __b = (appy::i64)blockIdx.x * 4 + __wvl; __b < __nblk; __b += (appy::i64)gridDim.x * 4) {")
        self.ind += 1
        w(f"const appy::i64 __r0 = __lo + __b * {R};")
        w(f"const int __nr = (int)((__hi - __r0) < {R} ? (__hi - __r0) : {R});")
        w("appy::wave_fence();       // the block before this one has been read out of __lp")
        w("bool __good = true, __long = false;")
        w("#pragma unroll")
        w(f"for (int __k = 0; __k < {R // 64 + 1}; ++__k) {{      // and the first row of the next block, if there is one")
        self.ind += 1
        w("const int __r = __k * 64 + __lid;")
        w(f"if (__r <= __nr && __r0 + __r < __hi && (__k < {R // 64} || __lid == 0)) {{")
        self.ind += 1
        w(f"const appy::i64 {cname(var)} = __r0 + __r;")
        self._declare_locals()
        self.block(body[:at])
        lo, hi = self._range_args(a.team_split)
        w(f"const appy::i64 __rlo = {lo};")
        w(f"const appy::i64 __rhi = {hi};")
        w("if (__rlo < 0 || __rhi < __rlo || __rhi > __len) __good = false;")
        w("__lp[__r] = (int)__rlo;")
        w("if (__r < __nr) { __hq[__r] = (int)__rhi; __long = __long || (__rhi - __rlo > __rowmax); }")
        self.ind -= 1
        w("}")
        self.ind -= 1
        w("}")
        w("appy::wave_fence();")
        w("// every row ends where the next one starts; the block ends no later than the next one starts")
        w("#pragma unroll")
        w(f"for (int __k = 0; __k < {R // 64}; ++__k) {{")
        w("    const int __r = __k * 64 + __lid;")
        w("    if (__r < __nr - 1) __good = __good && __lp[__r + 1] == __hq[__r];")
        w("    else if (__r == __nr - 1 && __r0 + __nr < __hi) __good = __good && __lp[__nr] >= __hq[__r];")
        w("}")
        w("__good = __ballot(!__good) == 0ull;")
        if not self.spec.skip_long:
            w("if (__ballot(__long) != 0ull && __lid == 0) __hint[0] = 2;      // rows too long for this treatment: the next launch sorts them")
        w("const int __first = __good ? __lp[0] : 0, __end = __good ? __hq[__nr - 1] : 0;")
        w("appy::wave_fence();")
        w("#pragma unroll")
        w(f"for (int __k = 0; __k < {R // 64 + 1}; ++__k) {{")
        w("    const int __r = __k * 64 + __lid;")
        w(f"    if (__r >= __nr && __r <= {R} && (__k < {R // 64} || __lid == 0)) __lp[__r] = __end;")
        w("}")
        w("appy::wave_fence();")
        w("if (!__good) {")
        w("    // refused: the launch runs the loop row by row instead; the cells of this block stay empty")
        w("    if (__lid == 0) __flag[0] = 1;")
        w(f"    if (__lid <= {S}) __desc[__b * {S + 1} + __lid] = 0;")
        w("    continue;")
        w("}")
        skip = self.spec.skip_long

        def find_row(table, at):
            w(f"int __row = 0, __past = {R};       // the last row that starts at or before {at}")
            w("#pragma unroll")
            w(f"for (int __it = 0; __it < {R.bit_length() - 1}; ++__it) {{")
            w("    const int __mid = (__row + __past) >> 1;")
            w(f"    if ({table}[__mid] <= {at}) __row = __mid; else __past = __mid;")
            w("}")

        def count(k):
            w("#pragma unroll")
            w("for (int __q = 0; __q < 4; ++__q)")
            w("#pragma unroll")
            w(f"    for (int __s = 0; __s < {S}; ++__s) __cnt[__s] += __popcll(__ballot((__c[{k}][__q] >> __shiftc) == __s));")

        def starts():
            w("__at[0] = __first;")
            w("#pragma unroll")
            w(f"for (int __s = 0; __s < {S}; ++__s) __at[__s + 1] = __at[__s] + __cnt[__s];")
            w("#pragma unroll")
            w(f"for (int __s = 0; __s <= {S}; ++__s) if (__lid == __s) __desc[__b * {S + 1} + __s] = __at[__s];")

        def place_one(kc, kv):
            w(f"const int __cq = __c[{kc}][__q];")
            w("const int __sq = __cq >> __shiftc;          // negative past the end (and for negative indices: such elements are dropped)")
            w("int __pos = 0;")
            w("#pragma unroll")
            w(f"for (int __s = 0; __s < {S}; ++__s) {{")
            w("    const unsigned long long __m = __ballot(__sq == __s);")
            w("    if (__sq == __s) __pos = __at[__s] + __popcll(__m & __below);")
            w("    __at[__s] += __popcll(__m);")
            w("}")
            w(f"if (__sq >= 0 && __sq < {S})")
            w("    __ent[__pos] = (long long)(((unsigned long long)(((unsigned)__row << 22) | (unsigned)(__cq & __cmask)) << 32) "
              f"| (unsigned long long)(unsigned)__v[{kv}][__q]);")

        def unrolled(n, fn):
            w("#pragma unroll")
            w(f"for (int __k = 0; __k < {n}; ++__k) {{")
            self.ind += 1
            fn()
            self.ind -= 1
            w("}")

        w(f"int __cnt[{S}], __at[{S + 1}];")
        w("#pragma unroll")
        w(f"for (int __s = 0; __s < {S}; ++__s) __cnt[__s] = 0;")

        def load_indices(k, j0, kk):
            w(f"{{ const int __j = {j0} + {kk} * 256 + __lid * 4;")
            w(f"if (__j + 4 <= __end) __c[{k}] = {self._group_index4(idx_c + ' + __j')};")
            w("else {")
            w("#pragma unroll")
            w(f"    for (int __q = 0; __q < 4; ++__q) __c[{k}][__q] = __j + __q < __end ? {self._group_index1(idx_c + '[__j + __q]')} : -1;")
            w("} }")

        def load_carried(k, j0, kk):
            if car_c:
                w(f"{{ const int __j = {j0} + {kk} * 256 + __lid * 4;")
                w(f"if (__j + 4 <= __end) __v[{k}] = appy::vload<int, 4>({car_c} + __j);")
                w("else {")
                w("#pragma unroll")
                w(f"    for (int __q = 0; __q < 4; ++__q) __v[{k}][__q] = __j + __q < __end ? {car_c}[__j + __q] : 0;")
                w("} }")
            else:
                w(f"__v[{k}] = 0;")

        def place(kc, kv, j0, kk):
            w(f"const int __j = {j0} + {kk} * 256 + __lid * 4;")
            find_row("__lp", "__j")
            w("#pragma unroll")
            w("for (int __q = 0; __q < 4; ++__q) {")
            self.ind += 1
            w("if (__j + __q < __end) while (__lp[__row + 1] <= __j + __q) ++__row;")
            place_one(kc, kv)
            self.ind -= 1
            w("}")

        if skip:
            # the sorting kernel, which ran before this one, has counted the rows beyond the limit: where there are none,
            # every element is kept and the walk over the arrays as they lie does (the layout is the same either way)
            w("if (__counts[3] == 0) {")
            self.ind += 1
        # (indices of a whole block kept in registers between the two passes - 64 registers, half the wavefronts per
        #  SIMD - made this kernel slower: 455 us against 306 for 2^26 elements)
        w(f"for (int __j0 = __first; __j0 < __end; __j0 += {256 * U}) {{")
        self.ind += 1
        w(f"appy::vec<int, 4>::type __c[{U}];")
        unrolled(U, lambda: load_indices("__k", "__j0", "__k"))
        unrolled(U, lambda: count("__k"))
        self.ind -= 1
        w("}")
        starts()
        w(f"for (int __j0 = __first; __j0 < __end; __j0 += {256 * U}) {{")
        self.ind += 1
        w(f"appy::vec<int, 4>::type __c[{U}], __v[{U}];")
        unrolled(U, lambda: (load_indices("__k", "__j0", "__k"), load_carried("__k", "__j0", "__k")))
        unrolled(U, lambda: place("__k", "__k", "__j0", "__k"))
        self.ind -= 1
        w("}")
        if skip:
            self.ind -= 1
            w("} else {")
            self.ind += 1
            self._group_walk_kept(idx_c, car_c, U, find_row, count, starts, place_one, unrolled)
            self.ind -= 1
            w("}")
        self.ind -= 1
        w("}")

    def _group_index4(self, pointer: str) -> str:
        """Four indices of the grouping kernel from `pointer`, as 32-bit numbers (an index that does not fit
        is negative afterwards, and dropped like every negative index)."""
        if not self._group_wide:
            return f"appy::vload<int, 4>({pointer})"
        return f"appy::narrow_indices(appy::vload<long long, 4>({pointer}))"

    def _group_index1(self, value: str) -> str:
        return value if not self._group_wide else f"appy::narrow_index({value})"

    def _group_walk_kept(self, idx_c, car_c, U, find_row, count, starts, place_one, unrolled):
        """The two passes of the grouping kernel over the elements of the rows that are kept (rows
        beyond `__rowmax` elements run in planned parts): the lanes walk the kept elements of the block
        as one sequence; `__kp[r]` is where row r starts in it."""
        R = self.GROUP_ROWS
        w = self.w
        P = R // 64
        w(f"// where every row starts among the elements that are kept (rows beyond the limit hold none): lane l sums rows {P}l .. {P}l + {P - 1}")
        w("int* __kp = __hq;")
        w(f"int __kt[{P}], __mine = 0;")
        w("#pragma unroll")
        w(f"for (int __i = 0; __i < {P}; ++__i) {{")
        w(f"    const int __r = {P} * __lid + __i;")
        w("    const int __n = __r < __nr ? __hq[__r] - __lp[__r] : 0;")
        w("    __kt[__i] = __n > __rowmax ? 0 : __n;")
        w("    __mine += __kt[__i];")
        w("}")
        w("int __incl = __mine;")
        w("#pragma unroll")
        w("for (int __d = 1; __d < 64; __d <<= 1) {")
        w("    const int __o = __shfl_up(__incl, __d, 64);")
        w("    if (__lid >= __d) __incl += __o;")
        w("}")
        w("appy::wave_fence();       // the ends of the rows have been read: their table now holds the starts among the kept")
        w("{")
        w("    int __run = __incl - __mine;")
        w("#pragma unroll")
        w(f"    for (int __i = 0; __i < {P}; ++__i) {{ __kp[{P} * __lid + __i] = __run; __run += __kt[__i]; }}")
        w("}")
        w(f"if (__lid == 63) __kp[{R}] = __incl;")
        w("appy::wave_fence();")
        w(f"const int __kept = __kp[{R}];")

        def positions(k):
            """Row and array positions of the four kept elements __t .. __t + 3 of this lane."""
            w(f"const int __t = __t0 + {k} * 256 + __lid * 4;")
            find_row("__kp", "__t")
            w("int __jq[4];")
            w("#pragma unroll")
            w("for (int __q = 0; __q < 4; ++__q) {")
            w("    if (__t + __q < __kept) while (__kp[__row + 1] <= __t + __q) ++__row;")
            w("    __jq[__q] = __lp[__row] + (__t + __q - __kp[__row]);")
            w("}")
            w("const bool __run = __t + 4 <= __kept && __jq[3] == __jq[0] + 3;       // four elements in a row of the arrays")

        def load(k, both):
            w("{")
            self.ind += 1
            positions(k)
            w(f"if (__run) __c[{k}] = {self._group_index4(idx_c + ' + __jq[0]')};")
            w("else {")
            w("#pragma unroll")
            w(f"    for (int __q = 0; __q < 4; ++__q) __c[{k}][__q] = __t + __q < __kept ? {self._group_index1(idx_c + '[__jq[__q]]')} : -1;")
            w("}")
            if both:
                if car_c:
                    w(f"if (__run) __v[{k}] = appy::vload<int, 4>({car_c} + __jq[0]);")
                    w("else {")
                    w("#pragma unroll")
                    w(f"    for (int __q = 0; __q < 4; ++__q) __v[{k}][__q] = __t + __q < __kept ? {car_c}[__jq[__q]] : 0;")
                    w("}")
                else:
                    w(f"__v[{k}] = 0;")
            self.ind -= 1
            w("}")

        def place(k):
            w(f"const int __t = __t0 + {k} * 256 + __lid * 4;")
            find_row("__kp", "__t")
            w("#pragma unroll")
            w("for (int __q = 0; __q < 4; ++__q) {")
            self.ind += 1
            w("if (__t + __q < __kept) while (__kp[__row + 1] <= __t + __q) ++__row;")
            place_one(k, k)
            self.ind -= 1
            w("}")

        w(f"for (int __t0 = 0; __t0 < __kept; __t0 += {256 * U}) {{")
        self.ind += 1
        w(f"appy::vec<int, 4>::type __c[{U}];")
        unrolled(U, lambda: load("__k", False))
        unrolled(U, lambda: count("__k"))
        self.ind -= 1
        w("}")
        starts()
        w(f"for (int __t0 = 0; __t0 < __kept; __t0 += {256 * U}) {{")
        self.ind += 1
        w(f"appy::vec<int, 4>::type __c[{U}], __v[{U}];")
        unrolled(U, lambda: load("__k", True))
        unrolled(U, lambda: place("__k"))
        self.ind -= 1
        w("}")

    def _body_cells(self):
        """The kernel that runs the cells: the term of the sum is evaluated per grouped element (the carried
        operand from the element, the gathered operand from its stripe) and added to the element's row
        in LDS; the sums of a cell's rows go to the scratch table of 4-byte slots per row and stripe."""
        a, g, S, R = self.a, self.a.grouping, self.spec.parts, self.GROUP_ROWS
        self.ex.locals[a.var] = T.WEAK_INT
        self.mode = "lane"
        term, tty, pty = self._group_setup_types()
        if pty.name not in ("float32", "int32", "uint32") and not self.dirty:
            raise Unsupported(f"sums of {pty.name} are not accumulated in LDS")
        x = a.arrays[g["x"]]
        x.loaded = True
        U = 8
        w = self.w
        w("const int __lid = threadIdx.x & 63;")
        w("const int __wvl = threadIdx.x >> 6;")
        w(f"__shared__ {pty.c} __acc_all[4][{R}];        // the sums of the rows of a cell, one cell per wavefront")
        w(f"{pty.c}* __acc = __acc_all[__wvl];")
        w(f"const appy::i64 __nblk = (__hi - __lo + {R - 1}) / {R};")
        w("// workgroup g serves the stripes g mod 8, g mod 8 + 8, ...: workgroups go to the eight XCDs in turn, so every L2")
        w("// holds one stripe of the gathered operand at a time")
        w("const appy::i64 __w0 = (appy::i64)(blockIdx.x >> 3) * 4 + __wvl, __nw = (appy::i64)(gridDim.x >> 3) * 4;")
        w(f"for (int __pass = 0; __pass < {S // 8}; ++__pass) {{")
        self.ind += 1
        w("const int __s = (int)(blockIdx.x & 7) + 8 * __pass;")
        w("const appy::i64 __x0 = (appy::i64)__s << __shiftc;")
        w("for (appy::i64 __b = __w0; __b < __nblk; __b += __nw) {")
        self.ind += 1
        w(f"const int __clo = __desc[__b * {S + 1} + __s], __chi = __desc[__b * {S + 1} + __s + 1];")
        w("#pragma unroll")
        w(f"for (int __k = 0; __k < {R // 64}; ++__k) __acc[__k * 64 + __lid] = 0;")
        w("appy::wave_fence();")
        w(f"for (int __j0 = __clo; __j0 < __chi; __j0 += {64 * U}) {{")
        self.ind += 1
        w(f"long long __e[{U}];")
        w(f"{x.elem_c} __xv[{U}];")
        w("#pragma unroll")
        w(f"for (int __k = 0; __k < {U}; ++__k) {{")
        w("    const int __j = __j0 + __k * 64 + __lid;")
        w("    __e[__k] = __j < __chi ? __builtin_nontemporal_load(__ent + __j) : 0ll;")
        w("}")
        w("#pragma unroll")
        w(f"for (int __k = 0; __k < {U}; ++__k) {{")
        w("    const int __j = __j0 + __k * 64 + __lid;")
        w(f"    __xv[__k] = {cname(g['x'])}[__j < __chi ? __x0 + (appy::i64)((unsigned)((unsigned long long)__e[__k] >> 32) & 0x3fffffu) : 0];")
        w("}")
        w("#pragma unroll")
        w(f"for (int __k = 0; __k < {U}; ++__k) {{")
        self.ind += 1
        w("const int __j = __j0 + __k * 64 + __lid;")
        w("if (__j < __chi) {")
        self.ind += 1
        if g["carried"]:
            cty = a.arrays[g["carried"]].ty
            bits = "(int)(unsigned)(unsigned long long)__e[__k]"
            w(f"const {cty.c} __cv = {'__int_as_float(' + bits + ')' if cty.is_float else '(' + cty.c + ')' + bits};")
        w(f"const {x.elem_c} __cx = __xv[__k];")
        w(f"atomicAdd(&__acc[(unsigned)((unsigned long long)__e[__k] >> 54)], {cast(term, tty, pty)});")
        self.ind -= 1
        w("}")
        self.ind -= 1
        w("}")
        self.ind -= 1
        w("}")
        w("appy::wave_fence();")
        w("#pragma unroll")
        w(f"for (int __k = 0; __k < {R // 64}; ++__k) {{")
        w(f"    const appy::i64 __row = __b * {R} + __k * 64 + __lid;")
        w(f"    if (__row < __hi - __lo) reinterpret_cast<{pty.c}*>(__scratch)[(appy::i64)__s * (__hi - __lo) + __row] = __acc[__k * 64 + __lid];")
        w("}")
        w("appy::wave_fence();")
        self.ind -= 1
        w("}")
        self.ind -= 1
        w("}")

    # ---- row plans: the elements of a sum over a gathered operand, ordered once and kept ----------------
    # A plan orders the elements by cell (a block of 32768 rows x one of eight column ranges of the gathered
    # operand) and, within a cell, by the 128-byte line of the operand they read.  `rkeys` writes one (key,
    # value) pair per element, the library sorts them and works out, tile by tile, where each product goes so
    # that the tile's products lie sorted by row (include/appy_hip.h, "row plans"); `xcells` runs the result.
    PLAN_ROW_BITS = 15

    def _body_rkeys(self):
        """The kernel that writes the pairs.  Per block of 256 rows (one wavefront): the set-up of its rows
        gives the rows' ranges, which must follow one another as those of a CSR matrix do and hold indices
        inside the gathered operand - otherwise the flag is raised and no plan comes of it; then every element
        goes to its own position of the two arrays: the key (block of 32768 rows, line of the operand) and the
        value (bits of the carried operand, row within the block, column within the line)."""
        a, g, R = self.a, self.a.grouping, self.GROUP_ROWS
        var = a.var
        self.ex.locals[var] = T.WEAK_INT
        self.mode = "lane"
        idx_c = cname(g["idx"])
        a.arrays[g["idx"]].loaded = True
        car_c = f"reinterpret_cast<const int*>({cname(g['carried'])})" if g["carried"] else None
        body = a.outer.body
        at = next(k for k, st in enumerate(body) if st is a.team_split)
        U = 4
        w = self.w
        RB = self.PLAN_ROW_BITS
        w("const int __lid = threadIdx.x & 63;")
        w("const int __wvl = threadIdx.x >> 6;")
        w(f"__shared__ int __lp_all[4][{R + 1}];      // where the rows of the block start; the last entry: where it ends")
        w(f"__shared__ int __hq_all[4][{R + 1}];      // where they end")
        w("int* __lp = __lp_all[__wvl];")
        w("int* __hq = __hq_all[__wvl];")
        w(f"const appy::i64 __nblk = (__hi - __lo + {R - 1}) / {R};")
        w("for (appy::i64 __b = (appy::i64)blockIdx.x * 4 + __wvl; __b < __nblk; __b += (appy::i64)gridDim.x * 4) {")
        self.ind += 1
        w(f"const appy::i64 __r0 = __lo + __b * {R};")
        w(f"const int __nr = (int)((__hi - __r0) < {R} ? (__hi - __r0) : {R});")
        w("appy::wave_fence();       // the block before this one has been read out of __lp")
        w("bool __good = true;")
        w("#pragma unroll")
        w(f"for (int __k = 0; __k < {R // 64 + 1}; ++__k) {{      // and the first row of the next block, if there is one")
        self.ind += 1
        w("const int __r = __k * 64 + __lid;")
        w(f"if (__r <= __nr && __r0 + __r < __hi && (__k < {R // 64} || __lid == 0)) {{")
        self.ind += 1
        w(f"const appy::i64 {cname(var)} = __r0 + __r;")
        self._declare_locals()
        self.block(body[:at])
        lo, hi = self._range_args(a.team_split)
        w(f"const appy::i64 __rlo = {lo};")
        w(f"const appy::i64 __rhi = {hi};")
        w("if (__rlo < 0 || __rhi < __rlo || __rhi > __len) __good = false;")
        w("__lp[__r] = (int)__rlo;")
        w("if (__r < __nr) __hq[__r] = (int)__rhi;")
        self.ind -= 1
        w("}")
        self.ind -= 1
        w("}")
        w("appy::wave_fence();")
        w("// every row ends where the next one starts; the block ends no later than the next one starts")
        w("#pragma unroll")
        w(f"for (int __k = 0; __k < {R // 64}; ++__k) {{")
        w("    const int __r = __k * 64 + __lid;")
        w("    if (__r < __nr - 1) __good = __good && __lp[__r + 1] == __hq[__r];")
        w("    else if (__r == __nr - 1 && __r0 + __nr < __hi) __good = __good && __lp[__nr] >= __hq[__r];")
        w("}")
        w("__good = __ballot(!__good) == 0ull;")
        w("const int __first = __good ? __lp[0] : 0, __end = __good ? __hq[__nr - 1] : 0;")
        w("appy::wave_fence();")
        w("#pragma unroll")
        w(f"for (int __k = 0; __k < {R // 64 + 1}; ++__k) {{")
        w("    const int __r = __k * 64 + __lid;")
        w(f"    if (__r >= __nr && __r <= {R} && (__k < {R // 64} || __lid == 0)) __lp[__r] = __end;")
        w("}")
        w("appy::wave_fence();")
        w("if (!__good) {")
        w("    if (__lid == 0) __flag[0] = 1;")
        w("    continue;")
        w("}")
        w("// (how many positions the rows of all blocks cover: when it is every position, no key stays unset and the sort needs a bit less)")
        w("if (__lid == 0) atomicAdd(reinterpret_cast<unsigned long long*>(__flag) + 1, (unsigned long long)(__end - __first));")
        w(f"const unsigned __rel0 = (unsigned)(__b * {R});       // first row of the block, counted from the start of the range")
        w("bool __inside = true;")
        w(f"for (int __j0 = __first; __j0 < __end; __j0 += {256 * U}) {{")
        self.ind += 1
        w("#pragma unroll")
        w(f"for (int __k = 0; __k < {U}; ++__k) {{")
        self.ind += 1
        w("const int __j = __j0 + __k * 256 + __lid * 4;")
        w("if (__j >= __end) continue;")
        ic = a.arrays[g["idx"]].elem_c           # int, or long long: narrowed once it is known to lie inside the operand
        w(f"appy::vec<{ic}, 4>::type __c;")
        w("appy::vec<int, 4>::type __v;")
        w(f"if (__j + 4 <= __end) __c = appy::vload<{ic}, 4>({idx_c} + __j);")
        w("else {")
        w("#pragma unroll")
        w(f"    for (int __q = 0; __q < 4; ++__q) __c[__q] = __j + __q < __end ? {idx_c}[__j + __q] : 0;")
        w("}")
        if car_c:
            w(f"if (__j + 4 <= __end) __v = appy::vload<int, 4>({car_c} + __j);")
            w("else {")
            w("#pragma unroll")
            w(f"    for (int __q = 0; __q < 4; ++__q) __v[__q] = __j + __q < __end ? {car_c}[__j + __q] : 0;")
            w("}")
        else:
            w("__v = 0;")
        w(f"int __row = 0, __past = {R};       // the last row that starts at or before __j")
        w("#pragma unroll")
        w(f"for (int __it = 0; __it < {R.bit_length() - 1}; ++__it) {{")
        w("    const int __mid = (__row + __past) >> 1;")
        w("    if (__lp[__mid] <= __j) __row = __mid; else __past = __mid;")
        w("}")
        w("#pragma unroll")
        w("for (int __q = 0; __q < 4; ++__q) {")
        w("    if (__j + __q >= __end) break;")
        w("    while (__lp[__row + 1] <= __j + __q) ++__row;")
        w(f"    const {ic} __cq = __c[__q];")
        w("    if (__cq < 0 || __cq >= __nx) { __inside = false; continue; }")
        w("    const unsigned __rel = __rel0 + (unsigned)__row;")
        w(f"    __keys[__j + __q] = ((__rel >> {RB}) << __lbits) | ((unsigned)__cq >> 5);")
        w(f"    __vals[__j + __q] = (unsigned long long)(unsigned)__v[__q] | ((unsigned long long)((__rel & {(1 << RB) - 1}u) "
          f"| (((unsigned)__cq & 31u) << {RB})) << 32);")
        w("}")
        self.ind -= 1
        w("}")
        self.ind -= 1
        w("}")
        w("if (__ballot(!__inside) != 0ull && __lid == 0) __flag[0] = 1;      // an index outside the gathered operand: no plan")
        self.ind -= 1
        w("}")

    def _body_xcells(self):
        """The kernel that runs a row plan: workgroups of 1024 lanes (one per CU: their LDS allows no more), the
        cells of column range g on the workgroups g mod 8 (one XCD and its L2 per range); a workgroup walks the
        tiles of its cells as one sequence, so that the loads of a cell's first tiles travel while the cell before
        it is finished, and puts out the sums of a cell when its last tile is through.  Tile by tile: the lanes gather the
        operand in the order of the plan (adjacent lanes read the same lines), put the value of each term into
        its slot in LDS, and after a barrier add the slots to the sums of the cell's rows, which are in LDS
        too - first the rows with one slot, a lane per row, then the rows with a run of slots, a lane per run,
        in slot order.  A row is touched by one lane per tile and tiles are separated by barriers: the sums do
        not depend on timing.  The sums of a cell go to the scratch table of 4-byte slots per row and range.

        A wavefront instruction takes four cycles on a SIMD and only four wavefronts share one, so the loop is
        written for few instructions: every load is a per-tile base held in scalar registers plus a lane
        offset that never changes, nothing is loaded under a branch (a tile that does not exist is read at one
        position for every lane and never used), the starts of a cell come through the scalar cache, and the header
        of a tile becomes a scalar one stage after it was asked for."""
        a, g = self.a, self.a.grouping
        U = self.spec.unroll
        TILE = 1024 * U
        H = U // 2
        SEG = TILE // 2 + 4          # words of the row stream from one tile of a cell to the next
        RB = self.PLAN_ROW_BITS
        ROWS = 1 << RB
        self.ex.locals[a.var] = T.WEAK_INT
        self.mode = "lane"
        term, tty, pty = self._group_setup_types()
        if pty.name not in ("float32", "int32", "uint32") and not self.dirty:
            raise Unsupported(f"sums of {pty.name} are not accumulated in LDS")
        x = a.arrays[g["x"]]
        x.loaded = True
        xc = cname(g["x"])
        w = self.w
        P = pty.c

        def value(e, xv):
            """Code of the term for element word `e` and gathered value `xv`."""
            pre = ""
            if g["carried"]:
                cty = a.arrays[g["carried"]].ty
                bits = f"(int)(unsigned)({e})"
                pre = f"const {cty.c} __cv = {'__int_as_float(' + bits + ')' if cty.is_float else '(' + cty.c + ')' + bits}; "
            return f"{{ {pre}const {x.elem_c} __cx = {xv}; __val = {cast(term, tty, pty)}; }}"

        w("const unsigned __tid = threadIdx.x;")
        w(f"__shared__ {P} __sum[{ROWS}];        // the sums of the rows of the cell")
        w(f"__shared__ __attribute__((aligned(8))) {P} __prod[{TILE}];       // the terms of a tile, sorted by row")
        w("const appy::i64 __n = __hi - __lo;")
        w("const unsigned __cmask = (1u << __colbits) - 1u;")
        w("const unsigned __xlast = (unsigned)(__nx - 1);")
        w("const char* __xb = reinterpret_cast<const char*>(" + xc + ");")
        w("// A cell may be shared by __split workgroups, each with a run of its tiles and a slot of its own for the sums: a")
        w("// run is numbered (block * __split + part) * 8 + range.  The workgroup takes the runs that the entries blockIdx.x,")
        w("// blockIdx.x + gridDim.x, ... of __order name (dealt out on the host by size; the grid is a multiple of eight")
        w("// workgroups and all runs of a workgroup read the same range) and walks their tiles as one sequence, so that")
        w("// the loads of a run's first tiles travel while the run before it is finished.")
        w("const unsigned __nrun = (unsigned)(__ncell * __split), __spl = (unsigned)__split;")
        w("const unsigned __g = blockIdx.x & 7u;")
        w("const unsigned __x0 = __g * (unsigned)__gwidth;")
        w("#pragma unroll")
        w(f"for (int __k = 0; __k < {ROWS // 1024}; ++__k) __sum[__k * 1024 + __tid] = 0;")
        w(f"unsigned long long __e0[{U}], __e1[{U}], __e2[{U}];")
        w(f"{x.elem_c} __xv[{U}], __x1[{U}];")
        w(f"unsigned __r0[{H}], __r1[{H}];")
        w("unsigned __da0, __db0, __da1, __db1;")
        w("unsigned __h0, __h1, __hv2;        // headers of the tiles in flight (the newest as it was loaded, in a vector register)")
        w("// the tile the next load fetches: run, tile within the run; of the run: its tiles, where its elements and its row")
        w("// stream start, the elements from there to the end of the cell")
        w("unsigned __vi = blockIdx.x, __tt = 0, __nt = 0;")
        w("unsigned __vc = __vi < __norder ? __order[__vi] : 0xffffffffu;        // (no run: a number beyond them all)")
        w("appy::i64 __eb = 0, __sb = 0;      // (in bytes from the start of the elements and of the row stream)")
        w("const char* __entb = reinterpret_cast<const char*>(__ent);")
        w("const char* __rsb = reinterpret_cast<const char*>(__rstream);")
        w("appy::i64 __left = 0;")
        w("// of the tiles in flight (0: the one that is added up, 1: the one whose gathers travel, 2: the one just requested):")
        w("// whether it exists, its elements, whether it ends its run, the run, its part of the row stream")
        w("bool __in0, __in1, __in2, __end0, __end1, __end2, __any0, __any1, __any2;")
        w("unsigned __cnt0, __cnt1, __cnt2, __run0, __run1, __run2;")
        w("appy::i64 __ps0, __ps1, __ps2;")

        def enter_run():
            """Where the run __vc lies (when there is such a run)."""
            w("if (__vc < __nrun) {")
            w("    const unsigned __b = (__vc >> 3) / __spl, __part = (__vc >> 3) % __spl;")
            w("    const appy::i64 __cell = (appy::i64)__b * 8 + __g;")
            w("    const unsigned __nta = __tbase[__cell + 1] - __tbase[__cell];")
            w("    const unsigned __tlo = __part * __nta / __spl;        // (at most 32 parts, and tiles of thousands of elements)")
            w("    __nt = (__part + 1) * __nta / __spl - __tlo;")
            w(f"    const appy::i64 __cs = (appy::i64)__cstart[__cell] + (appy::i64)__tlo * {TILE};")
            w("    __left = (appy::i64)__cstart[__cell + 1] - __cs;")
            w("    __eb = __cs * 8;")
            w("    __sb = ((__cs >> 1) + 4 * ((appy::i64)__tbase[__cell] + __tlo)) * 4;")
            w("} else {")
            w("    __nt = 0;")
            w("}")

        # (a tile that does not exist - past the last run, or the one turn of a run without tiles - is read all the
        #  same: one position for every lane, so that it costs one request per instruction, and never used)
        def load_tile(dst):
            """Requests the header and the elements of the next tile of the sequence into stage 2, and steps on.
            (The header is asked for first and as a vector load, and turned into a scalar only when the tile moves on
            to stage 1: a wait for it then covers no load younger than it, and none that misses.)"""
            w("{")
            w("  __any2 = __vc < __nrun; __in2 = __any2 && __tt < __nt; __end2 = __tt + 1 >= __nt; __run2 = __vc;")
            w(f"  const char* __p = __entb + appy::uniform_i64(__in2 ? __eb + (appy::i64)__tt * {TILE * 8} : 0);")
            w(f"  __ps2 = appy::uniform_i64(__in2 ? __sb + (appy::i64)__tt * {SEG * 4} : 0);")
            w("  __hv2 = *reinterpret_cast<const unsigned*>(__rsb + __ps2 + appy::lane_offset(0u));")
            w(f"  const appy::i64 __l = __left - (appy::i64)__tt * {TILE};")
            w(f"  __cnt2 = __in2 ? (unsigned)(__l < {TILE} ? __l : {TILE}) : 0u;")
            w("#pragma unroll")
            w(f"  for (int __u = 0; __u < {U}; ++__u)")
            w(f"      {dst}[__u] = __builtin_nontemporal_load(reinterpret_cast<const unsigned long long*>(__p + appy::lane_offset(__in2 ? (unsigned)((__u * 1024 + __tid) * 8) : 0u)));")
            w("  if (__any2) {")
            w("      if (!__end2) ++__tt;")
            w("      else {")
            w("          __vi += gridDim.x; __vc = __vi < __norder ? __order[__vi] : 0xffffffffu; __tt = 0;")
            self.ind += 3
            enter_run()
            self.ind -= 3
            w("      }")
            w("  }")
            w("}")

        def load_rows(dst, da, db, hdr, inn, ps):
            """Row numbers of the slots this lane adds up, and the first run of slots it may have to walk."""
            w("{")
            w("#pragma unroll")
            w(f"  for (int __u = 0; __u < {H}; ++__u)")
            w(f"      {dst}[__u] = __builtin_nontemporal_load(reinterpret_cast<const unsigned*>(__rsb + {ps} + appy::lane_offset({inn} ? (unsigned)((1 + __u * 1024 + __tid) * 4) : 0u)));")
            w(f"  const unsigned __runs = ({hdr} >> 16);")
            w(f"  const char* __q = __rsb + ({ps} + ({inn} ? (appy::i64)(1 + ((({hdr} & 0xffffu) + 1) >> 1)) * 4 : 0));     // (the header of a tile that does not exist may hold anything)")
            w(f"  const unsigned __at = appy::lane_offset({inn} && __tid < __runs ? __tid * 4 : 0u);        // (lanes without a run: one position)")
            w(f"  {da} = *reinterpret_cast<const unsigned*>(__q + __at);")
            w(f"  {db} = *reinterpret_cast<const unsigned*>(__q + __at + 4); }}")

        def gather(dst, src, inn, first, last):
            w("{")
            w("#pragma unroll")
            w(f"  for (int __u = {first}; __u < {last}; ++__u) {{")
            w(f"    unsigned __c = __x0 + ((unsigned)({src}[__u] >> 32) & __cmask);")
            w("    __c = __c < __xlast ? __c : __xlast;        // (what was read beyond the cell may hold anything)")
            w(f"    {dst}[__u] = *reinterpret_cast<const {x.elem_c}*>(__xb + appy::lane_offset({inn} ? (unsigned)(__c << 2) : 0u));")
            w("  } }")

        def shift(frm, to):
            w(f"__in{to} = __in{frm}; __end{to} = __end{frm}; __any{to} = __any{frm}; __cnt{to} = __cnt{frm}; "
              f"__run{to} = __run{frm}; __ps{to} = __ps{frm};")

        def add_run(d, d1):
            w(f"{{ const int __row = (int)({d} & {ROWS - 1}u), __from = (int)({d} >> {RB}), __to = (int)({d1} >> {RB});")
            w(f"  {P} __acc = __sum[__row];")
            w("  for (int __k = __from; __k < __to; __k += 4) {")
            w(f"      const {P} __p0 = __prod[__k], __p1 = __k + 1 < __to ? __prod[__k + 1] : 0, "
              "__p2 = __k + 2 < __to ? __prod[__k + 2] : 0, __p3 = __k + 3 < __to ? __prod[__k + 3] : 0;")
            w("      __acc += __p0;")
            w("      if (__k + 1 < __to) __acc += __p1;")
            w("      if (__k + 2 < __to) __acc += __p2;")
            w("      if (__k + 3 < __to) __acc += __p3;")
            w("  }")
            w("  __sum[__row] = __acc; }")

        enter_run()
        load_tile("__e0")
        w("__h0 = __builtin_amdgcn_readfirstlane(__hv2);")
        shift(2, 0)
        load_tile("__e1")
        w("__h1 = __builtin_amdgcn_readfirstlane(__hv2);")
        shift(2, 1)
        load_rows("__r0", "__da0", "__db0", "__h0", "__in0", "__ps0")
        gather("__xv", "__e0", "__in0", 0, U)
        w("__syncthreads();")
        w("while (__any0) {")
        self.ind += 1
        w("const unsigned __ns = __in0 ? __h0 & 0xffffu : 0u, __nm = __in0 ? __h0 >> 16 : 0u;")
        # Where the loads of the next tiles are asked for was settled with cycle counters at the boundaries of the phases: a
        # wave that asks for a load waits until the texture addresser takes it, and with every load ahead of the first
        # barrier all waves stood in that queue together (7000 of 11300 cycles per tile) while LDS was idle, and then
        # added up together while the addresser was idle.  So the element stream of the tile after the next goes first (it
        # comes from HBM), the row numbers follow the scatter, and the gathers are asked for in two halves between the
        # phases that add up: waves that have been served go on adding while the others queue.
        load_tile("__e2")
        w(f"if (__cnt0 == {TILE}u) {{")
        w("#pragma unroll")
        w(f"    for (int __u = 0; __u < {U}; ++__u) {{")
        w(f"        {P} __val;")
        w("        " + value("__e0[__u]", "__xv[__u]"))
        w("        __prod[(unsigned)(__e0[__u] >> 32) >> __colbits] = __val;")
        w("    }")
        w("} else {")
        w("#pragma unroll")
        w(f"    for (int __u = 0; __u < {U}; ++__u) {{")
        w(f"        {P} __val;")
        w("        " + value("__e0[__u]", "__xv[__u]"))
        w("        if (__u * 1024 + __tid < __cnt0) __prod[(unsigned)(__e0[__u] >> 32) >> __colbits] = __val;")
        w("    }")
        w("}")
        load_rows("__r1", "__da1", "__db1", "__h1", "__in1", "__ps1")
        w("__syncthreads();")
        w("{")
        w(f"    {P} __sa[{H}], __sb_[{H}];")
        w(f"    appy::vec<{P}, 2>::type __pp[{H}];")
        w("#pragma unroll")
        w(f"    for (int __u = 0; __u < {H}; ++__u) {{")
        w(f"        __pp[__u] = *reinterpret_cast<const appy::vec<{P}, 2>::type*>(&__prod[2 * (__u * 1024 + __tid)]);")
        w("        __sa[__u] = __sum[__r0[__u] & 0x7fffu]; __sb_[__u] = __sum[(__r0[__u] >> 16) & 0x7fffu];")
        w("    }")
        w("#pragma unroll")
        w(f"    for (int __u = 0; __u < {H}; ++__u) {{")
        w("        const unsigned __s = 2 * (__u * 1024 + __tid);")
        w("        if (__s < __ns) __sum[__r0[__u] & 0x7fffu] = __sa[__u] + __pp[__u][0];")
        w("        if (__s + 1 < __ns) __sum[(__r0[__u] >> 16) & 0x7fffu] = __sb_[__u] + __pp[__u][1];")
        w("    }")
        w("}")
        gather("__x1", "__e1", "__in1", 0, H)
        w("if (__nm > 0) {")
        self.ind += 1
        w("if (__tid < __nm) {")
        self.ind += 1
        add_run("__da0", "__db0")
        self.ind -= 1
        w("}")
        w("if (__nm > 1024) {")
        w("    const unsigned* __runs = reinterpret_cast<const unsigned*>(__rsb + __ps0) + 1 + ((__ns + 1) >> 1);")
        w("    for (unsigned __m = __tid + 1024; __m < __nm; __m += 1024) {")
        w("        const unsigned __d = __runs[__m], __d1 = __runs[__m + 1];")
        self.ind += 2
        add_run("__d", "__d1")
        self.ind -= 2
        w("    }")
        w("}")
        self.ind -= 1
        w("}")
        gather("__x1", "__e1", "__in1", H, U)
        w("__syncthreads();")
        w("if (__end0) {")
        self.ind += 1
        w("// the run is through: its sums go out and start again at zero (every lane clears what it has read itself; the next")
        w("// tile's terms are added after the barrier that follows their scatter)")
        w("const unsigned __b = (__run0 >> 3) / __spl, __part = (__run0 >> 3) % __spl;")
        w(f"{P}* __out = reinterpret_cast<{P}*>(__scratch) + ((appy::i64)__part * 8 + __g) * __n + (appy::i64)__b * {ROWS};")
        w(f"if (((appy::i64)__b + 1) * {ROWS} <= __n) {{")
        w("#pragma unroll")
        w(f"    for (int __k = 0; __k < {ROWS // 1024}; ++__k) {{ __out[__k * 1024 + __tid] = __sum[__k * 1024 + __tid]; __sum[__k * 1024 + __tid] = 0; }}")
        w("} else {")
        w(f"    for (int __k = 0; __k < {ROWS // 1024}; ++__k) {{")
        w(f"        if ((appy::i64)__b * {ROWS} + __k * 1024 + __tid < __n) __out[__k * 1024 + __tid] = __sum[__k * 1024 + __tid];")
        w("        __sum[__k * 1024 + __tid] = 0;")
        w("    }")
        w("}")
        self.ind -= 1
        w("}")
        w("#pragma unroll")
        w(f"for (int __u = 0; __u < {U}; ++__u) {{ __e0[__u] = __e1[__u]; __e1[__u] = __e2[__u]; __xv[__u] = __x1[__u]; }}")
        w("#pragma unroll")
        w(f"for (int __u = 0; __u < {H}; ++__u) __r0[__u] = __r1[__u];")
        w("__h0 = __h1; __h1 = __builtin_amdgcn_readfirstlane(__hv2); __da0 = __da1; __db0 = __db1;")
        shift(1, 0)
        shift(2, 1)
        self.ind -= 1
        w("}")

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
            pty = _partial_type(ty)
            self.partials[name] = (p, pty)
            self.w(f"{pty.c} {p} = {_partial_identity(op, ty, pty)};")
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
