"""Inner-loop vectorisation for ``prange`` loops.

With the high-level interface (``for i in prange(...)`` without pragmas) the
compiler decides which inner loops are spread over lanes: the reference's guide
lists "Inner Loop Vectorization: APPy automatically adds the simd pragma to
innermost loops that can be vectorized" among the transformations behind
``prange`` (docs/source/developer.rst, "High-Level Programming Interface"), and
its extended reduction rule treats ``a[i] += b[i, j]`` as a reduction with
regard to loop ``j`` (same file, "Reduction Detection").  Loops annotated with
pragmas are left exactly as written.

An innermost ``for j in range(...)`` gets ``#pragma simd`` when

* it is *legal*: its iterations do not depend on each other -
  every scalar it assigns is either defined afresh in each iteration before it
  is read (and not used outside the loop), or only updated by one reduction
  operator; every array it stores to is accessed with one and the same index
  tuple throughout the loop, and that tuple contains ``j + c`` (each iteration
  owns its elements) - or does not contain ``j`` at all and is only updated by
  ``X[..] += e``, which is then rewritten to a scalar reduction around the loop;
* it is *profitable*: wherever ``j`` indexes an array directly it indexes the
  last (contiguous) dimension as ``j + c`` (loads may also gather through an
  index array, ``x[cols[j]]``) - otherwise lanes walking ``j`` would stride
  through memory while one lane per outer iteration might not.

The analysis is syntactic and conservative; anything it does not recognise
leaves the loop sequential inside its lane.
"""
from __future__ import annotations

import ast
import copy

from . import source as src

_BLOCKERS = (ast.For, ast.While, ast.Break, ast.Continue, ast.Return, ast.Try, ast.With, ast.FunctionDef, ast.Lambda)


def _elts(sub: ast.Subscript):
    return sub.slice.elts if isinstance(sub.slice, ast.Tuple) else [sub.slice]


def _uses(node, name: str) -> bool:
    return any(isinstance(n, ast.Name) and n.id == name for n in ast.walk(node))


def _uses_directly(node, name: str) -> bool:
    """``name`` occurs in ``node`` outside any nested subscript (``cols[j]`` inside
    ``x[cols[j]]`` is an indirect use)."""
    if isinstance(node, ast.Name):
        return node.id == name
    if isinstance(node, ast.Subscript):
        return False
    return any(_uses_directly(c, name) for c in ast.iter_child_nodes(node))


def _is_var_plus_const(node, var: str) -> bool:
    if isinstance(node, ast.Name) and node.id == var:
        return True
    if isinstance(node, ast.BinOp) and isinstance(node.op, (ast.Add, ast.Sub)):
        l, r = node.left, node.right
        if isinstance(l, ast.Name) and l.id == var and isinstance(r, ast.Constant) and type(r.value) is int:
            return True
        if (isinstance(node.op, ast.Add) and isinstance(r, ast.Name) and r.id == var
                and isinstance(l, ast.Constant) and type(l.value) is int):
            return True
    return False


def _reduction_op(target_text: str, value):
    """'+', '*', 'max', 'min' if ``value`` combines the target with something else."""
    same = lambda e: ast.unparse(e) == target_text   # noqa: E731
    if isinstance(value, ast.BinOp) and isinstance(value.op, (ast.Add, ast.Mult)):
        if same(value.left) != same(value.right):
            other = value.right if same(value.left) else value.left
            if not any(same(n) for n in ast.walk(other) if isinstance(n, (ast.Name, ast.Subscript))):
                return "+" if isinstance(value.op, ast.Add) else "*"
    if (isinstance(value, ast.Call) and isinstance(value.func, ast.Name) and value.func.id in ("max", "min")
            and len(value.args) == 2 and same(value.args[0]) != same(value.args[1])):
        return value.func.id
    return None


def _assign_parts(st):
    """(target, value-as-if-plain-assignment) of an Assign / AugAssign with one target."""
    if isinstance(st, ast.AugAssign):
        return st.target, ast.BinOp(left=copy.deepcopy(st.target), op=st.op, right=st.value)
    if isinstance(st, ast.Assign) and len(st.targets) == 1:
        return st.targets[0], st.value
    return None, None


class _Verdict:
    def __init__(self):
        self.ok = True
        self.hoist = []     # (statement, op): array-element reductions to turn into scalar reductions


def _count(nodes, name: str) -> int:
    return sum(1 for st in nodes for n in ast.walk(st) if isinstance(n, ast.Name) and n.id == name)


def analyse(loop: ast.For, outer: ast.For) -> _Verdict:
    """Decide whether ``loop`` (innermost, somewhere inside the parallel loop
    ``outer``) may and should become a simd loop."""
    v = _Verdict()
    outer_var = outer.target.id if isinstance(outer.target, ast.Name) else ""
    j = loop.target.id if isinstance(loop.target, ast.Name) else None
    it = loop.iter
    if (j is None or loop.orelse or not (isinstance(it, ast.Call) and isinstance(it.func, ast.Name)
                                         and it.func.id == "range" and not it.keywords and 1 <= len(it.args) <= 2)):
        v.ok = False
        return v
    if any(_uses(a, j) for a in it.args):
        v.ok = False
        return v
    for st in loop.body:
        for n in ast.walk(st):
            if isinstance(n, _BLOCKERS) or (isinstance(n, ast.Call) and not isinstance(n.func, (ast.Name, ast.Attribute))):
                v.ok = False
                return v
            if isinstance(n, ast.stmt) and not isinstance(n, (ast.Assign, ast.AugAssign, ast.If, ast.Pass)) and not (
                    isinstance(n, ast.Expr) and isinstance(n.value, ast.Constant)):
                v.ok = False            # a kind of statement this analysis does not model (annotated assignment, ...)
                return v

    # ---- assignments: scalars and array stores -------------------------------------
    scalar_kinds = {}            # name -> set of ops (None = plain)
    stores = {}                  # array -> set of index texts it is stored with
    store_stmts = []
    for st in ast.walk(ast.Module(body=loop.body, type_ignores=[])):
        if isinstance(st, (ast.Assign, ast.AugAssign)):
            tgt, val = _assign_parts(st)
            if tgt is None or isinstance(tgt, (ast.Tuple, ast.List, ast.Attribute, ast.Starred)):
                v.ok = False
                return v
            if isinstance(tgt, ast.Name):
                scalar_kinds.setdefault(tgt.id, set()).add(_reduction_op(tgt.id, val))
            elif isinstance(tgt, ast.Subscript) and isinstance(tgt.value, ast.Name):
                if any(isinstance(e, ast.Slice) for e in _elts(tgt)):
                    v.ok = False
                    return v
                stores.setdefault(tgt.value.id, set()).add(ast.unparse(tgt))
                store_stmts.append((st, tgt, val))
            else:
                v.ok = False
                return v
        elif isinstance(st, ast.NamedExpr):
            v.ok = False
            return v

    # scalars: private temporaries or reductions
    for name, kinds in scalar_kinds.items():
        if name == j or name == outer_var:
            v.ok = False
            return v
        if kinds == {None}:
            # must be written before it is read in every iteration: its first statement-level
            # occurrence is an unconditional plain assignment that does not read it
            first = None
            for st in loop.body:
                if _uses(st, name):
                    first = st
                    break
            tgt, val = _assign_parts(first) if isinstance(first, (ast.Assign, ast.AugAssign)) else (None, None)
            if not (isinstance(first, ast.Assign) and isinstance(tgt, ast.Name) and tgt.id == name
                    and not _uses(val, name)):
                v.ok = False
                return v
            if _count(outer.body, name) != _count([loop], name):
                v.ok = False            # also used outside the loop: its last value is wanted there
                return v
        elif len(kinds) == 1:
            # a reduction: the loop may mention it only in its own update statements
            expected = 0
            for st in ast.walk(ast.Module(body=loop.body, type_ignores=[])):
                if isinstance(st, (ast.Assign, ast.AugAssign)):
                    tgt, _val = _assign_parts(st)
                    if isinstance(tgt, ast.Name) and tgt.id == name:
                        expected += 1 if isinstance(st, ast.AugAssign) else 2
            if _count(loop.body, name) != expected:
                v.ok = False
                return v
        else:
            v.ok = False
            return v
    assigned = set(scalar_kinds)

    # arrays that are stored to
    for arr, texts in stores.items():
        accesses = {ast.unparse(n) for n in ast.walk(ast.Module(body=loop.body, type_ignores=[]))
                    if isinstance(n, ast.Subscript) and isinstance(n.value, ast.Name) and n.value.id == arr}
        if len(texts) != 1 or accesses != texts:
            v.ok = False                # touched with more than one index tuple
            return v
    for st, tgt, val in store_stmts:
        idx = _elts(tgt)
        if any(_uses(e, j) for e in idx):
            if not any(_is_var_plus_const(e, j) for e in idx):
                v.ok = False            # e.g. X[j // 2]: two iterations may share an element
                return v
        else:
            # the same element in every iteration: only as `X[..] += e` / `*=`, hoisted to a scalar
            op = _reduction_op(ast.unparse(tgt), val)
            top_level = any(st is s for s in loop.body)
            if op not in ("+", "*") or not top_level or any(_uses(e, a) for e in idx for a in assigned):
                v.ok = False
                return v
            # nothing else in the loop may look at the element while it is being accumulated
            text = ast.unparse(tgt)
            seen = sum(1 for n in ast.walk(ast.Module(body=loop.body, type_ignores=[]))
                       if isinstance(n, ast.Subscript) and ast.unparse(n) == text)
            mine = [s2 for s2, t2, _ in store_stmts if ast.unparse(t2) == text]
            if seen != sum(1 if isinstance(s2, ast.AugAssign) else 2 for s2 in mine):
                v.ok = False
                return v
            v.hoist.append((st, op))

    # ---- profitability: j walks the contiguous dimension -----------------------------
    indexed_by_j = 0
    for n in ast.walk(ast.Module(body=loop.body, type_ignores=[])):
        if isinstance(n, ast.Subscript) and isinstance(n.value, ast.Name):
            idx = _elts(n)
            if any(isinstance(e, ast.Slice) for e in idx):
                v.ok = False
                return v
            if any(_uses_directly(e, j) for e in idx):
                indexed_by_j += 1
                if any(_uses_directly(e, j) for e in idx[:-1]) or not _is_var_plus_const(idx[-1], j):
                    v.ok = False        # strided or computed access along j
                    return v
            elif any(_uses(e, j) for e in idx) and not isinstance(n.ctx, ast.Load):
                v.ok = False            # scatter through an index array: two iterations may hit one element
                return v
    if indexed_by_j == 0:
        v.ok = False
    return v


class _Vectorise:
    def __init__(self, outer: ast.For):
        self.outer = outer
        self.counter = 0
        self.changed = 0

    def block(self, stmts):
        out = []
        for st in stmts:
            if isinstance(st, ast.For) and not any(isinstance(n, (ast.For, ast.While)) for s in st.body for n in ast.walk(s)):
                verdict = analyse(st, self.outer)
                if verdict.ok:
                    out.extend(self._emit(st, verdict))
                    self.changed += 1
                    continue
            for f in ("body", "orelse"):
                sub = getattr(st, f, None)
                if isinstance(sub, list) and sub and isinstance(sub[0], ast.stmt):
                    setattr(st, f, self.block(sub))
            out.append(st)
        return out

    def _emit(self, loop: ast.For, verdict: _Verdict):
        pre, post = [], []
        for st, op in verdict.hoist:
            tgt, val = _assign_parts(st)
            self.counter += 1
            r = f"__appy_acc{self.counter}"
            other = val.right if ast.unparse(val.left) == ast.unparse(tgt) else val.left
            pre.append(ast.parse(f"{r} = {'0' if op == '+' else '1'}").body[0])
            binop = ast.Add() if op == "+" else ast.Mult()
            loop.body[loop.body.index(st)] = ast.AugAssign(target=ast.Name(id=r, ctx=ast.Store()), op=binop, value=other)
            post.append(ast.AugAssign(target=copy.deepcopy(tgt), op=copy.deepcopy(binop), value=ast.Name(id=r, ctx=ast.Load())))
        return pre + [src.make_pragma_stmt("#pragma simd"), loop] + post


def vectorise_inner_loops(outer: ast.For) -> int:
    """Mark the vectorisable innermost loops of a ``prange`` loop (in place).
    Returns how many loops were marked."""
    if any(src.pragma_text(n) is not None for n in ast.walk(outer) if isinstance(n, ast.stmt)):
        return 0        # the programmer has started annotating: nothing is added
    vz = _Vectorise(outer)
    outer.body = vz.block(outer.body)
    ast.fix_missing_locations(outer)
    return vz.changed
