"""What the kernel generator needs to know about an annotated loop before it writes a line:
which arrays and scalars the body touches and how, the reductions of the parallel loop, and the
shapes the body allows (vector steps, teams, strips, rows binned by length, elements grouped by
the stripe they gather from, row plans).  Nothing here emits code."""
from __future__ import annotations

import ast
from dataclasses import dataclass

from ...frontend import loop_ir
from . import dtypes as T
from .dtypes import Ty


@dataclass
class OuterReduction:
    key: str             # e.g. 's[0]'
    op: str
    array: str
    index: int
    ty: Ty               # type of the register accumulators (at least 32 bits wide)
    acc: str             # register name
    elem_ty: Ty = None   # type of the array element the totals are combined into


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
