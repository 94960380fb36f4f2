"""Decoration-time rewrite of an annotated function.

Turns every loop annotated with ``#pragma parallel for ...`` (or iterating over
``prange``) into a call of the run-time stub, keeping the rest of the function
as ordinary Python.  The observable result follows the reference's four
decoration-time passes (reference tree: appy/__init__.py:38-65,
appy/frontend/hoist_shape_attr.py:4-48, appy/frontend/process_shared.py:4-75,
appy/frontend/replace_pfor_with_stub.py:3-81):

* ``X.shape[k]`` inside a ``for`` statement becomes the name ``X_shape_k`` and
  the assignment ``X_shape_k = X.shape[k]`` is placed in front of the
  (outermost) loop;
* for ``shared(v, ...)`` the loop is bracketed by ``v = numpy.array([v])`` and
  ``v = v.item()`` and every use of ``v`` in the loop reads ``v[0]``;
* the loop is replaced by ``appy._kernel_launch(<loop text>, 'kernel_loop_N',
  locals(), globals(), {options})`` where the loop text starts with the pragma
  line and loops are numbered per function starting at 1;
* decorators of the function are dropped so that executing the new source
  does not decorate again.

The implementation works on statement lists with pragma marker statements
(see :mod:`appy_amd.frontend.source`) instead of comment nodes.
"""
from __future__ import annotations

import ast
import copy
import re

from . import auto_simd
from . import source as src
from .pragma import is_parallel_for_text

_SHARED_CLAUSE = re.compile(r"shared\(([^)]*)\)")

_BODY_FIELDS = ("body", "orelse", "finalbody")


# --------------------------------------------------------------------------
# X.shape[k] hoisting
# --------------------------------------------------------------------------
class _ShapeRefs(ast.NodeTransformer):
    def __init__(self):
        self.seen = []  # (array name, dim) in first-use order, no duplicates

    def visit_Subscript(self, node):
        self.generic_visit(node)
        v = node.value
        if (
            isinstance(v, ast.Attribute)
            and v.attr == "shape"
            and isinstance(v.value, ast.Name)
            and isinstance(node.slice, ast.Constant)
            and isinstance(node.slice.value, int)
            and isinstance(node.ctx, ast.Load)
        ):
            key = (v.value.id, node.slice.value)
            if key not in self.seen:
                self.seen.append(key)
            return ast.copy_location(ast.Name(id=f"{key[0]}_shape_{key[1]}", ctx=ast.Load()), node)
        return node


def _hoist_shapes_in_block(stmts):
    out = []
    for st in stmts:
        if isinstance(st, ast.For):
            refs = _ShapeRefs()
            st = refs.visit(st)
            for name, dim in refs.seen:
                out.append(ast.parse(f"{name}_shape_{dim} = {name}.shape[{dim}]").body[0])
            out.append(st)
            continue
        for f in _BODY_FIELDS:
            sub = getattr(st, f, None)
            if isinstance(sub, list) and sub and isinstance(sub[0], ast.stmt):
                setattr(st, f, _hoist_shapes_in_block(sub))
        if isinstance(st, ast.Try):
            for h in st.handlers:
                h.body = _hoist_shapes_in_block(h.body)
        out.append(st)
    return out


# --------------------------------------------------------------------------
# shared(...) scalars and stub replacement
# --------------------------------------------------------------------------
class _NameToElement0(ast.NodeTransformer):
    def __init__(self, names):
        self.names = set(names)

    def visit_Name(self, node):
        if node.id in self.names:
            return ast.copy_location(
                ast.Subscript(value=ast.Name(id=node.id, ctx=ast.Load()), slice=ast.Constant(value=0), ctx=node.ctx),
                node,
            )
        return node


def shared_names(pragma_text: str):
    names = []
    for group in _SHARED_CLAUSE.findall(pragma_text):
        names.extend(v.strip() for v in group.split(",") if v.strip())
    return names


def _range_flag(node: ast.For, flag: str) -> bool:
    """``range(..., flag=True)`` / ``appy.range(..., flag=True)`` as the loop's iterator."""
    it = node.iter
    if not isinstance(it, ast.Call):
        return False
    f = it.func
    is_range = (isinstance(f, ast.Name) and f.id == "range") or (
        isinstance(f, ast.Attribute) and f.attr == "range" and isinstance(f.value, ast.Name) and f.value.id == "appy")
    return is_range and any(k.arg == flag and isinstance(k.value, ast.Constant) and k.value.value is True
                            for k in it.keywords)


def _is_prange_loop(node: ast.For) -> bool:
    """``prange(...)``, ``appy.prange(...)`` or its documented spelling
    ``appy.range(..., parallel=True)`` (reference: docs/source/legacy.rst)."""
    it = node.iter
    if not isinstance(it, ast.Call):
        return False
    f = it.func
    if isinstance(f, ast.Name) and f.id == "prange":
        return True
    if isinstance(f, ast.Attribute) and f.attr == "prange" and isinstance(f.value, ast.Name) and f.value.id == "appy":
        return True
    return _range_flag(node, "parallel")


class _SimdRanges(ast.NodeTransformer):
    """``for j in appy.range(n, simd=True)`` inside a parallel loop is the
    keyword spelling of ``#pragma simd`` above ``for j in range(n)``."""

    def _fix(self, stmts):
        out = []
        for st in stmts:
            st = self.visit(st)
            if isinstance(st, ast.For) and _range_flag(st, "simd"):
                st.iter.func = ast.Name(id="range", ctx=ast.Load())
                st.iter.keywords = []
                out.append(src.make_pragma_stmt("#pragma simd"))
            out.append(st)
        return out

    def generic_visit(self, node):
        for f in _BODY_FIELDS:
            sub = getattr(node, f, None)
            if isinstance(sub, list) and sub and isinstance(sub[0], ast.stmt):
                setattr(node, f, self._fix(sub))
        return node


class _InnerPranges(ast.NodeTransformer):
    """A ``prange`` loop inside a loop that already is a kernel promises independent
    iterations and nothing more: inside the kernel it is a ``range`` loop (which the
    vectoriser may then spread over lanes)."""

    def visit_For(self, node):
        self.generic_visit(node)
        if _is_prange_loop(node):
            node.iter.func = ast.Name(id="range", ctx=ast.Load())
            node.iter.keywords = [k for k in node.iter.keywords if k.arg not in ("parallel", "shared")]
        return node


def prange_reductions(loop: ast.For):
    """Scalars that a ``prange`` loop without a pragma reduces across its
    iterations (reference behaviour as documented for ``appy.prange``,
    docs/source/getting_started.rst:51-66: "APPy automatically detects
    reductions"): names updated only by ``s += e`` / ``s *= e`` /
    ``s = max(s, e)`` / ``s = min(s, e)`` with one and the same operator, never
    assigned in any other way inside the loop (a name that is also plainly
    assigned is a per-iteration temporary) and not a loop variable."""
    ops = {}
    loop_vars = {n.target.id for n in ast.walk(loop) if isinstance(n, ast.For) and isinstance(n.target, ast.Name)}

    def note(name, op):
        ops.setdefault(name, set()).add(op)

    for n in ast.walk(loop):
        if isinstance(n, ast.AugAssign) and isinstance(n.target, ast.Name):
            note(n.target.id, {ast.Add: "+", ast.Mult: "*"}.get(type(n.op)))
        elif isinstance(n, ast.Assign):
            for t in n.targets:
                for nm in (t.elts if isinstance(t, ast.Tuple) else [t]):
                    if not isinstance(nm, ast.Name):
                        continue
                    v, op = n.value, None
                    if len(n.targets) == 1 and not isinstance(t, ast.Tuple):
                        if isinstance(v, ast.BinOp) and isinstance(v.op, (ast.Add, ast.Mult)) and any(
                                isinstance(x, ast.Name) and x.id == nm.id for x in (v.left, v.right)):
                            op = "+" if isinstance(v.op, ast.Add) else "*"
                        elif (isinstance(v, ast.Call) and isinstance(v.func, ast.Name) and v.func.id in ("max", "min")
                              and len(v.args) == 2 and any(isinstance(x, ast.Name) and x.id == nm.id for x in v.args)):
                            op = v.func.id
                    note(nm.id, op)
        elif isinstance(n, (ast.NamedExpr,)) and isinstance(n.target, ast.Name):
            note(n.target.id, None)
    return [name for name, kinds in ops.items() if len(kinds) == 1 and None not in kinds and name not in loop_vars]


class _LoopOutliner:
    def __init__(self, options):
        self.options = dict(options)
        self.count = 0
        self.pending = None  # text of the last unconsumed '#pragma parallel for' comment
        self.loops = []      # (loop name, loop text) in order, for inspection

    def _stub(self, loop_text: str, loop_name: str) -> ast.Expr:
        call = ast.Call(
            func=ast.Attribute(value=ast.Name(id="appy", ctx=ast.Load()), attr="_kernel_launch", ctx=ast.Load()),
            args=[
                ast.Constant(value=loop_text),
                ast.Constant(value=loop_name),
                ast.Call(func=ast.Name(id="locals", ctx=ast.Load()), args=[], keywords=[]),
                ast.Call(func=ast.Name(id="globals", ctx=ast.Load()), args=[], keywords=[]),
                ast.Dict(
                    keys=[ast.Constant(value=k) for k in self.options],
                    values=[ast.Constant(value=v) for v in self.options.values()],
                ),
            ],
            keywords=[],
        )
        return ast.fix_missing_locations(ast.Expr(value=call))

    def _outline(self, loop: ast.For):
        pragma, self.pending = self.pending, None
        self.count += 1
        loop_name = f"kernel_loop_{self.count}"
        pre, post = [], []
        simd_outer = False
        if _is_prange_loop(loop):
            # `prange` is `range` with the promise of independent iterations
            loop = copy.deepcopy(loop)
            simd_outer = _range_flag(loop, "simd")
            loop.iter.func = ast.Name(id="range", ctx=ast.Load())
            loop.iter.keywords = []
        loop = _SimdRanges().visit(copy.deepcopy(loop))
        loop.body = [_InnerPranges().visit(st) for st in loop.body]
        if pragma:
            if not re.search(r"\bsimd\b", pragma):
                # inner loops without annotations of their own: those that are provably independent
                # and walk the contiguous dimension are spread over lanes, as the reference's guide
                # says of loops whose `simd` was not spelled out (docs/source/legacy.rst:6)
                auto_simd.vectorise_inner_loops(loop)
            shared = shared_names(pragma)
            if shared:
                loop = _NameToElement0(shared).visit(copy.deepcopy(loop))
                for v in shared:
                    pre.append(ast.parse(f"{v} = numpy.array([{v}])").body[0])
                    post.append(ast.parse(f"{v} = {v}.item()").body[0])
            loop_text = pragma + "\n" + src.unparse(loop)
        else:
            # `for i in prange(...)` without a pragma: a parallel loop over the same range;
            # scalars it reduces are shared between the iterations.  Their buffer is float64
            # whatever the start value (a Python `total = 0` may well receive floats); a
            # start value that was an int gets an int back when the result is integral.
            reduced = prange_reductions(loop)
            pragma = "#pragma parallel for simd" if simd_outer else "#pragma parallel for"
            if not simd_outer:
                auto_simd.vectorise_inner_loops(loop)
            if reduced:
                pragma += f" shared({', '.join(reduced)})"
                loop = _NameToElement0(reduced).visit(copy.deepcopy(loop))
                for v in reduced:
                    pre.append(ast.parse(f"__appy_start_{v} = {v}").body[0])
                    pre.append(ast.parse(f"{v} = numpy.array([{v}], dtype=numpy.float64)").body[0])
                    post.append(ast.parse(f"{v} = appy._reduction_result({v}, __appy_start_{v})").body[0])
            loop_text = pragma + "\n" + src.unparse(loop)
        self.loops.append((loop_name, loop_text))
        return pre + [self._stub(loop_text, loop_name)] + post

    def block(self, stmts):
        out = []
        for st in stmts:
            text = src.pragma_text(st)
            if text is not None:
                if is_parallel_for_text(text):
                    self.pending = text
                # any other pragma outside a parallel loop has no meaning here
                continue
            if isinstance(st, ast.For) and (self.pending or _is_prange_loop(st)):
                out.extend(self._outline(st))
                continue
            for f in _BODY_FIELDS:
                sub = getattr(st, f, None)
                if isinstance(sub, list) and sub and isinstance(sub[0], ast.stmt):
                    new = self.block(sub)
                    setattr(st, f, new if new or f != "body" else [ast.Pass()])
            if isinstance(st, ast.Try):
                for h in st.handlers:
                    h.body = self.block(h.body) or [ast.Pass()]
            out.append(st)
        return out


def transform(tree: ast.Module, options) -> tuple[ast.Module, list]:
    """Rewrite a module holding one function definition.

    Returns the new module and the list of ``(loop name, loop text)`` pairs
    that were outlined.
    """
    tree.body = _hoist_shapes_in_block(tree.body)
    for node in tree.body:
        if isinstance(node, (ast.FunctionDef, ast.AsyncFunctionDef)):
            node.decorator_list = []
    outliner = _LoopOutliner(options)
    tree.body = outliner.block(tree.body) or [ast.Pass()]
    ast.fix_missing_locations(tree)
    return tree, outliner.loops
