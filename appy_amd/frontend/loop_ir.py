"""Per-loop front end: loop text -> loop IR.

The loop IR is a standard ``ast.Module`` holding one ``For`` nest in which

* every ``range`` call has the three arguments ``(start, stop, 1)``,
* tuple assignments and augmented assignments are expanded to plain ones,
* ``For`` and ``Assign`` nodes that follow a pragma carry a ``pragma`` dict,
* assignments that are reductions carry ``reduce`` (one of ``+ * max min``)
  and the annotated loop around them lists them as
  ``pragma['reduction'] = 'op:target,...'``.

This is the form the reference's back ends consume (reference tree:
appy/backends/triton/codegen.py:18-32 runs sanity_check, rewrite_tuple_assign,
rewrite_aug_assign, rewrite_range, attach_pragma and reduction_detection from
appy/frontend/ in that order); the rules below restate those passes.
"""
from __future__ import annotations

import ast
import copy

from . import source as src
from .pragma import is_pragma_text, parse_pragma

REDUCTION_OPS = ("+", "*", "max", "min")


# --------------------------------------------------------------------------
# structure checks (reference: appy/frontend/sanity_check.py:4-18)
# --------------------------------------------------------------------------
def check_structure(tree: ast.Module) -> None:
    loops = sum(isinstance(n, ast.For) for n in tree.body)
    if loops > 1:
        raise Exception(f"Input AST should only contain a single for loop while {loops} found.")
    assert tree.body and src.pragma_text(tree.body[0]) is not None, "Input AST should start with a pragma"


# --------------------------------------------------------------------------
# statement normalisation
# --------------------------------------------------------------------------
class _Normalise(ast.NodeTransformer):
    """Tuple assignment, augmented assignment and ``range`` normal forms
    (reference: appy/frontend/rewrite_tuple_assign.py:4-17,
    rewrite_aug_assign.py:5-20, rewrite_range.py:4-27)."""

    _tmp = 0

    def visit_Assign(self, node):
        self.generic_visit(node)
        if len(node.targets) > 1:
            # a = b = e  ->  a = e; b = a   (targets are assigned from left to right)
            first, rest = node.targets[0], node.targets[1:]
            out = self.visit_Assign(ast.copy_location(ast.Assign(targets=[first], value=node.value), node))
            out = out if isinstance(out, list) else [out]
            src_ = copy.deepcopy(first)
            for n in ast.walk(src_):
                if hasattr(n, "ctx"):
                    n.ctx = ast.Load()
            for t in rest:
                more = self.visit_Assign(ast.copy_location(ast.Assign(targets=[t], value=copy.deepcopy(src_)), node))
                out.extend(more if isinstance(more, list) else [more])
            return out
        if (isinstance(node.value, ast.BoolOp) and len(node.value.values) == 2
                and isinstance(node.targets[0], (ast.Name, ast.Subscript))):
            # `found = found or e` / `ok = ok and e`: a flag folded over the iterations is the
            # maximum / minimum of truth values
            key = ast.unparse(node.targets[0])
            a, b = node.value.values
            if (ast.unparse(a) == key) != (ast.unparse(b) == key):
                mine, other = (a, b) if ast.unparse(a) == key else (b, a)
                fn = "max" if isinstance(node.value.op, ast.Or) else "min"
                node.value = ast.Call(
                    func=ast.Name(id=fn, ctx=ast.Load()),
                    args=[mine, ast.Call(func=ast.Name(id="bool", ctx=ast.Load()), args=[other], keywords=[])],
                    keywords=[])
                return node
        if isinstance(node.value, ast.Tuple):
            tgt = node.targets[0]
            assert isinstance(tgt, ast.Tuple) and len(tgt.elts) == len(node.value.elts), (
                "a tuple on the right-hand side needs a tuple of the same length on the left"
            )
            written = {ast.unparse(t) for t in tgt.elts}
            reads_a_target = any(
                isinstance(n, (ast.Name, ast.Subscript)) and ast.unparse(n) in written
                for v in node.value.elts[1:] for n in ast.walk(v))
            if not reads_a_target:
                return [
                    ast.copy_location(ast.Assign(targets=[t], value=v), node)
                    for t, v in zip(tgt.elts, node.value.elts)
                ]
            # `p, q = q, p`: the right-hand side is evaluated in full before anything is stored
            out, temps = [], []
            for v in node.value.elts:
                _Normalise._tmp += 1
                name = f"__appy_t{_Normalise._tmp}"
                temps.append(name)
                out.append(ast.copy_location(ast.Assign(targets=[ast.Name(id=name, ctx=ast.Store())], value=v), node))
            for t, name in zip(tgt.elts, temps):
                out.append(ast.copy_location(ast.Assign(targets=[t], value=ast.Name(id=name, ctx=ast.Load())), node))
            return out
        return node

    def visit_AnnAssign(self, node):
        self.generic_visit(node)
        if node.value is None:
            return None                     # a bare annotation declares nothing a kernel needs
        return self.visit_Assign(ast.copy_location(ast.Assign(targets=[node.target], value=node.value), node))

    def visit_Assert(self, node):
        return None                         # as under `python -O`: kernels carry no assertions

    def visit_Subscript(self, node):
        self.generic_visit(node)
        inner = node.value
        if (isinstance(inner, ast.Subscript) and isinstance(inner.value, ast.Name)
                and not isinstance(node.slice, (ast.Slice, ast.Tuple))
                and not isinstance(inner.slice, ast.Slice)
                and not (isinstance(inner.slice, ast.Tuple) and any(isinstance(e, ast.Slice) for e in inner.slice.elts))
                and not (isinstance(inner.value, ast.Attribute))):
            # A[r][c] is A[r, c]
            first = list(inner.slice.elts) if isinstance(inner.slice, ast.Tuple) else [inner.slice]
            return ast.copy_location(
                ast.Subscript(value=inner.value, slice=ast.Tuple(elts=first + [node.slice], ctx=ast.Load()), ctx=node.ctx),
                node)
        return node

    def visit_AugAssign(self, node):
        self.generic_visit(node)
        read = copy.deepcopy(node.target)
        read.ctx = ast.Load()
        return ast.copy_location(
            ast.Assign(targets=[node.target], value=ast.BinOp(left=read, op=node.op, right=node.value)), node
        )

    def visit_Call(self, node):
        self.generic_visit(node)
        if isinstance(node.func, ast.Name) and node.func.id == "range":
            n = len(node.args)
            if n == 1:
                node.args = [ast.Constant(value=0), node.args[0], ast.Constant(value=1)]
            elif n == 2:
                node.args = [node.args[0], node.args[1], ast.Constant(value=1)]
            elif n == 3:
                step = node.args[2]
                if not (isinstance(step, ast.Constant) and step.value == 1 and not isinstance(step.value, bool)):
                    raise Exception(f"Only step 1 is supported in range, got: {ast.unparse(node)}")
            else:
                raise Exception(f"range expects 1 to 3 arguments, got: {ast.unparse(node)}")
        return node


# --------------------------------------------------------------------------
# pragma attachment (reference: appy/frontend/attach_pragma.py:4-24)
# --------------------------------------------------------------------------
def _attach_pragmas(stmts, pending):
    """A pragma belongs to the next ``For`` or ``Assign`` in program order; an
    assignment consumes it (so ``#pragma simd`` written above ``s = 0.0``
    leaves the following loop sequential).  Marker statements are removed."""
    out = []
    for st in stmts:
        text = src.pragma_text(st)
        if text is not None:
            if is_pragma_text(text):
                pending = text
            continue
        if isinstance(st, ast.For):
            if pending is not None:
                st.pragma = parse_pragma(pending)
                pending = None
            st.body, pending = _attach_pragmas(st.body, pending)
            st.orelse, pending = _attach_pragmas(st.orelse, pending)
        elif isinstance(st, ast.Assign):
            if pending is not None:
                st.pragma = parse_pragma(pending)
                pending = None
        else:
            for f in ("body", "orelse"):
                sub = getattr(st, f, None)
                if isinstance(sub, list) and sub and isinstance(sub[0], ast.stmt):
                    new, pending = _attach_pragmas(sub, pending)
                    setattr(st, f, new)
        out.append(st)
    return out, pending


# --------------------------------------------------------------------------
# reduction detection (reference: appy/frontend/reduction_detection.py:19-104)
# --------------------------------------------------------------------------
def is_scalar_location(node) -> bool:
    """A name, or an array element with a literal subscript (``s[0]``)."""
    return isinstance(node, ast.Name) or (
        isinstance(node, ast.Subscript) and isinstance(node.slice, ast.Constant)
    )


def reduction_operator(assign: ast.Assign):
    """``+``/``*`` for ``t = t + e`` / ``t = e * t``; ``max``/``min`` for
    ``t = max(t, e)``; None when the assignment is not of that shape."""
    tgt = assign.targets[0]
    if not is_scalar_location(tgt):
        return None
    key = ast.unparse(tgt)
    val = assign.value

    def same(e):
        return is_scalar_location(e) and ast.unparse(e) == key

    if isinstance(val, ast.BinOp) and isinstance(val.op, (ast.Add, ast.Mult)):
        if same(val.left) or same(val.right):
            return "+" if isinstance(val.op, ast.Add) else "*"
    elif (
        isinstance(val, ast.Call)
        and isinstance(val.func, ast.Name)
        and val.func.id in ("max", "min")
        and len(val.args) >= 2
    ):
        if same(val.args[0]) or same(val.args[1]):
            return val.func.id
    return None


def reduction_operand(assign: ast.Assign):
    """The expression combined into the target by a reduction assignment."""
    key = ast.unparse(assign.targets[0])
    val = assign.value
    if isinstance(val, ast.BinOp):
        if is_scalar_location(val.left) and ast.unparse(val.left) == key:
            return val.right
        return val.left
    a, b = val.args[0], val.args[1]
    if is_scalar_location(a) and ast.unparse(a) == key:
        return b
    return a


def _inner_parallel_loops_are_simd(tree: ast.Module) -> None:
    """``#pragma parallel for`` on a loop inside the loop that becomes the kernel promises
    independent iterations, which is what ``simd`` asks for: the inner loop is spread over
    the lanes of the team that runs the outer iteration."""
    outer = outer_loop(tree)
    for n in ast.walk(outer):
        if isinstance(n, ast.For) and n is not outer:
            pragma = getattr(n, "pragma", None)
            if pragma and "parallel_for" in pragma:
                del pragma["parallel_for"]
                pragma["simd"] = True


def _as_addition(assign: ast.Assign) -> None:
    """``t = t - e`` becomes ``t = t + (-e)`` (the same value in IEEE and in wrapping
    integer arithmetic), so that a running difference is a ``+`` reduction."""
    val = assign.value
    if (isinstance(val, ast.BinOp) and isinstance(val.op, ast.Sub) and len(assign.targets) == 1
            and isinstance(val.left, (ast.Name, ast.Subscript))
            and ast.unparse(val.left) == ast.unparse(assign.targets[0])):
        assign.value = ast.BinOp(left=val.left, op=ast.Add(), right=ast.UnaryOp(op=ast.USub(), operand=val.right))


def _element_reduction(st, loop_var: str, assigned: set, body):
    """For ``X[idx] = X[idx] op e`` / ``X[idx] = max(X[idx], e)`` at the top level of a
    simd loop, with ``idx`` the same in every iteration and ``X`` touched nowhere else in
    the loop: the operator; otherwise None."""
    if not (isinstance(st, ast.Assign) and len(st.targets) == 1):
        return None
    tgt = st.targets[0]
    if not (isinstance(tgt, ast.Subscript) and isinstance(tgt.value, ast.Name)) or is_scalar_location(tgt):
        return None
    idx = tgt.slice.elts if isinstance(tgt.slice, ast.Tuple) else [tgt.slice]
    for e in idx:
        if isinstance(e, ast.Slice):
            return None
        for n in ast.walk(e):
            if isinstance(n, ast.Name) and (n.id == loop_var or n.id in assigned):
                return None
            if isinstance(n, ast.Subscript):
                return None                 # an index read from memory: keep to the simple case
    key = ast.unparse(tgt)
    val = st.value
    same = lambda e: isinstance(e, ast.Subscript) and ast.unparse(e) == key   # noqa: E731
    if isinstance(val, ast.BinOp) and isinstance(val.op, (ast.Add, ast.Mult)) and same(val.left) != same(val.right):
        op, other = ("+" if isinstance(val.op, ast.Add) else "*"), (val.right if same(val.left) else val.left)
    elif (isinstance(val, ast.Call) and isinstance(val.func, ast.Name) and val.func.id in ("max", "min")
          and len(val.args) == 2 and not val.keywords and same(val.args[0]) != same(val.args[1])):
        op, other = val.func.id, (val.args[1] if same(val.args[0]) else val.args[0])
    else:
        return None
    # the array may appear in the loop only as the two mentions of this statement
    mentions = sum(1 for b in body for n in ast.walk(b) if isinstance(n, ast.Name) and n.id == tgt.value.id)
    if mentions != 2 or any(isinstance(n, ast.Name) and n.id == tgt.value.id for n in ast.walk(other)):
        return None
    return op, other


def _hoist_element_reductions(tree: ast.Module) -> None:
    """A ``simd`` loop inside a parallel loop that accumulates into one array element
    (``y[i] += A[i, j] * x[j]`` under ``for j``) carries a dependence through memory that
    its lanes would race on.  Such an element becomes a scalar around the loop::

        __appy_e1 = y[i]
        #pragma simd
        for j in ...: __appy_e1 = __appy_e1 + A[i, j] * x[j]
        y[i] = __appy_e1

    which the reduction detection below then treats like any local accumulator."""
    counter = [0]

    def block(stmts, inside_parallel):
        out = []
        for st in stmts:
            if isinstance(st, ast.For):
                pragma = getattr(st, "pragma", None) or {}
                var = st.target.id if isinstance(st.target, ast.Name) else ""
                if inside_parallel and "simd" in pragma and "parallel_for" not in pragma:
                    for a in st.body:
                        if isinstance(a, ast.Assign):
                            _as_addition(a)
                    assigned = {n.targets[0].id for b in st.body for n in ast.walk(b)
                                if isinstance(n, ast.Assign) and isinstance(n.targets[0], ast.Name)}
                    pre, post = [], []
                    for k, a in enumerate(list(st.body)):
                        found = _element_reduction(a, var, assigned, st.body)
                        if found is None:
                            continue
                        op, other = found
                        counter[0] += 1
                        name = f"__appy_e{counter[0]}"
                        tgt = a.targets[0]
                        read = copy.deepcopy(tgt)
                        read.ctx = ast.Load()
                        # `y[i] = 0.0` right before the loop: the accumulator starts from that literal
                        # instead of reading the element back
                        prev = out[-1] if out else None
                        if (not pre and isinstance(prev, ast.Assign) and len(prev.targets) == 1
                                and ast.unparse(prev.targets[0]) == ast.unparse(tgt)
                                and isinstance(prev.value, ast.Constant) and type(prev.value.value) in (int, float)
                                and float(prev.value.value).is_integer()):
                            read = ast.Constant(value=prev.value.value)
                        pre.append(ast.copy_location(ast.Assign(targets=[ast.Name(id=name, ctx=ast.Store())], value=read), st))
                        acc = ast.Name(id=name, ctx=ast.Load())
                        if op in ("+", "*"):
                            value = ast.BinOp(left=acc, op=ast.Add() if op == "+" else ast.Mult(), right=other)
                        else:
                            value = ast.Call(func=ast.Name(id=op, ctx=ast.Load()), args=[acc, other], keywords=[])
                        st.body[k] = ast.copy_location(ast.Assign(targets=[ast.Name(id=name, ctx=ast.Store())], value=value), a)
                        post.append(ast.copy_location(
                            ast.Assign(targets=[copy.deepcopy(tgt)], value=ast.Name(id=name, ctx=ast.Load())), st))
                    out.extend(pre + [st] + post)
                    continue
                st.body = block(st.body, inside_parallel or "parallel_for" in pragma)
            else:
                for f in ("body", "orelse"):
                    sub = getattr(st, f, None)
                    if isinstance(sub, list) and sub and isinstance(sub[0], ast.stmt):
                        setattr(st, f, block(sub, inside_parallel))
            out.append(st)
        return out

    tree.body = block(tree.body, False)


def _assignments_in(node):
    for n in ast.walk(node):
        if isinstance(n, ast.Assign):
            yield n


def _mark_all(tree: ast.Module) -> None:
    seen = set()

    def visit(node):
        for child in ast.iter_child_nodes(node):
            visit(child)
        if isinstance(node, ast.For) and id(node) not in seen:
            seen.add(id(node))
            _mark_one(node)

    def _mark_one(loop):
        if not hasattr(loop, "pragma"):
            return
        ops_of = {}
        for a in _assignments_in(loop):
            tgt = a.targets[0]
            if is_scalar_location(tgt):
                _as_addition(a)
                ops_of.setdefault(ast.unparse(tgt), set()).add(reduction_operator(a))
        found = {}
        for a in _assignments_in(loop):
            tgt = a.targets[0]
            if not is_scalar_location(tgt):
                continue
            key = ast.unparse(tgt)
            ops = ops_of.get(key, set())
            if len(ops) == 1:
                op = next(iter(ops))
                if op is not None:
                    a.reduce = op
                    found[key] = op
        pragma = loop.pragma
        if found and ("parallel_for" in pragma or "simd" in pragma):
            entries = []
            if "reduction" in pragma:
                spec = pragma["reduction"]
                entries = list(spec) if isinstance(spec, (tuple, list)) else spec.split(",")
            for key, op in found.items():
                entry = f"{op}:{key}"
                if entry not in entries:
                    entries.append(entry)
            pragma["reduction"] = ",".join(entries)

    visit(tree)


def reductions_of(loop: ast.For) -> dict:
    """``{'s[0]': '+'}`` from ``loop.pragma['reduction']``."""
    pragma = getattr(loop, "pragma", None) or {}
    out = {}
    if "reduction" in pragma:
        spec = pragma["reduction"]
        items = spec if isinstance(spec, (tuple, list)) else spec.split(",")
        for item in items:
            op, _, var = item.partition(":")
            out[var.strip()] = op.strip()
    return out


# --------------------------------------------------------------------------
# entry point
# --------------------------------------------------------------------------
def build(loop_source: str) -> ast.Module:
    """Loop text (pragma line + ``for`` statement) -> loop IR."""
    tree = src.parse(loop_source)
    check_structure(tree)
    tree = _Normalise().visit(tree)
    tree.body, _ = _attach_pragmas(tree.body, None)
    _inner_parallel_loops_are_simd(tree)
    _hoist_element_reductions(tree)
    _mark_all(tree)
    ast.fix_missing_locations(tree)
    return tree


def outer_loop(tree: ast.Module) -> ast.For:
    for n in tree.body:
        if isinstance(n, ast.For):
            return n
    raise Exception("The launch unit holds no for loop.")
