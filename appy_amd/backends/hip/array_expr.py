"""Lowering of 1-D array expressions to ``simd`` loops.

Inside a parallel loop a statement may use NumPy slice syntax over one
dimension (``y[i, :] = 0``, ``y[i, :] += a * B[k, :]``,
``s = np.sum(A[i, :] * x[:])``, ``d = u[:] @ v[:]``).  The reference hands such
statements to the un-vendored ``astpass`` passes ``vector_op_to_loop`` and
``normalize_ranges`` and then marks the produced loops ``simd`` (reference
tree: appy/backends/triton/passes/lower_array_op_to_loop.py:5-22,
rewrite_vector_dot.py:8-30); only 1-D expressions are accepted
(attach_shapes.py:19-20).  This module produces the equivalent loops directly
from NumPy's slice semantics:

    X[.., lo:hi, ..] = f(Y[.., a:b, ..], s)
        ->  for c in range(0, hi - lo):  X[.., lo + c, ..] = f(Y[.., a + c, ..], s)

    t = g(np.sum(E))
        ->  r = 0;  for c in range(0, n): r = r + E[c];  t = g(r)

Slice bounds that are omitted come from the array's shape, literal negative
bounds count from its end; the extent is the one of the assignment target (for
reductions: of the first sliced operand).
"""
from __future__ import annotations

import ast
import copy

_REDUCERS = {"sum": "+", "max": "max", "min": "min", "amax": "max", "amin": "min", "prod": "*"}
# further NumPy functions of one 1-D operand (two for the products) that come down to reductions
_DERIVED = ("mean", "average", "var", "std", "any", "all", "count_nonzero", "dot", "inner", "vdot", "argmax", "argmin")
# methods of an array expression that mean the function of the same name
_METHODS = ("sum", "max", "min", "prod", "mean", "var", "std", "any", "all", "dot", "argmax", "argmin")


def _is_array(val) -> bool:
    kind = f"{type(val).__module__}.{type(val).__name__}"
    return kind in ("numpy.ndarray", "torch.Tensor")


class _Ctx:
    def __init__(self, val_map):
        self.val_map = val_map
        self.counter = 0
        self.shape_refs = set()  # (array, dim) pairs whose extent the kernel needs

    def fresh(self, stem):
        self.counter += 1
        return f"__{stem}{self.counter}"

    def ndim(self, name):
        v = self.val_map.get(name)
        return v.ndim if _is_array(v) else None

    def shape_name(self, arr, dim):
        self.shape_refs.add((arr, dim))
        return ast.Name(id=f"{arr}_shape_{dim}", ctx=ast.Load())


def _slices_of(sub: ast.Subscript):
    elts = sub.slice.elts if isinstance(sub.slice, ast.Tuple) else [sub.slice]
    return [(d, e) for d, e in enumerate(elts) if isinstance(e, ast.Slice)]


def _has_vector_part(node, ctx: _Ctx) -> bool:
    for n in ast.walk(node):
        if isinstance(n, ast.Subscript) and _slices_of(n):
            return True
        if isinstance(n, ast.BinOp) and isinstance(n.op, ast.MatMult):
            return True
        if (
            isinstance(n, ast.Call)
            and isinstance(n.func, ast.Attribute)
            and isinstance(n.func.value, ast.Name)
            and n.func.value.id in ("np", "numpy")
            and (n.func.attr in _REDUCERS or n.func.attr in _DERIVED)
            and 1 <= len(n.args) <= 2
            and all(isinstance(a, ast.Name) and ctx.ndim(a.id) == 1 for a in n.args)
        ):
            return True
    return False


def _bounds(sub: ast.Subscript, dim: int, sl: ast.Slice, ctx: _Ctx):
    if sl.step is not None:
        raise RuntimeError(f"Step is not supported in slicing: {ast.unparse(sub)}")
    if not isinstance(sub.value, ast.Name) or ctx.ndim(sub.value.id) is None:
        raise RuntimeError(f"Only arrays defined outside of parallel region can be sliced: {ast.unparse(sub)}")
    lo = sl.lower if sl.lower is not None else ast.Constant(value=0)
    hi = sl.upper if sl.upper is not None else ctx.shape_name(sub.value.id, dim)
    return _from_end(lo, sub, dim, ctx), _from_end(hi, sub, dim, ctx)


def _negative_literal(node):
    """k for the literal ``-k`` (k > 0), else None."""
    if isinstance(node, ast.UnaryOp) and isinstance(node.op, ast.USub) and isinstance(node.operand, ast.Constant) \
            and type(node.operand.value) is int and node.operand.value > 0:
        return node.operand.value
    if isinstance(node, ast.Constant) and type(node.value) is int and node.value < 0:
        return -node.value
    return None


def _from_end(bound, sub: ast.Subscript, dim: int, ctx: _Ctx):
    """A literal negative slice bound counts from the end of the dimension
    (``A[i, 1:-1]``); bounds computed at run time are taken as they are."""
    k = _negative_literal(bound)
    if k is None:
        return bound
    return ast.BinOp(left=ctx.shape_name(sub.value.id, dim), op=ast.Sub(), right=ast.Constant(value=k))


def _extent(lo, hi):
    if isinstance(lo, ast.Constant) and lo.value == 0:
        return hi
    return ast.BinOp(left=hi, op=ast.Sub(), right=lo)


def _offset(lo, c: str):
    idx = ast.Name(id=c, ctx=ast.Load())
    if isinstance(lo, ast.Constant) and lo.value == 0:
        return idx
    return ast.BinOp(left=copy.deepcopy(lo), op=ast.Add(), right=idx)


class _Canonical(ast.NodeTransformer):
    """Spellings that mean an array expression without showing a slice: ``A[i]`` of a 2-D
    array is the row ``A[i, :]``; ``E.sum()`` is ``np.sum(E)``, ``E.astype(T)`` is ``T(E)``
    element by element, for an array expression ``E``."""

    def __init__(self, ctx: _Ctx):
        self.ctx = ctx

    def visit_Subscript(self, node):
        self.generic_visit(node)
        if isinstance(node.value, ast.Name):
            nd = self.ctx.ndim(node.value.id)
            elts = list(node.slice.elts) if isinstance(node.slice, ast.Tuple) else [node.slice]
            if nd is not None and 0 < len(elts) < nd and not any(isinstance(e, ast.Constant) and e.value is Ellipsis for e in elts):
                elts += [ast.Slice(lower=None, upper=None, step=None) for _ in range(nd - len(elts))]
                node.slice = ast.Tuple(elts=elts, ctx=ast.Load())
        return node

    def visit_Call(self, node):
        self.generic_visit(node)
        f = node.func
        # `axis=0` / `axis=-1` on a 1-D operand says nothing
        if (isinstance(f, ast.Attribute) and (f.attr in _REDUCERS or f.attr in _DERIVED or f.attr in _METHODS)
                and len(node.keywords) == 1 and node.keywords[0].arg == "axis"
                and isinstance(node.keywords[0].value, (ast.Constant, ast.UnaryOp))
                and ast.literal_eval(node.keywords[0].value) in (0, -1)):
            node.keywords = []
        if (isinstance(f, ast.Attribute) and isinstance(f.value, ast.Name) and f.value.id in ("np", "numpy")
                and f.attr in ("zeros_like", "ones_like") and len(node.args) == 1 and not node.keywords
                and (_has_vector_part(node.args[0], self.ctx)
                     or (isinstance(node.args[0], ast.Name) and self.ctx.ndim(node.args[0].id) == 1))):
            return ast.Constant(value=0 if f.attr == "zeros_like" else 1)
        if isinstance(f, ast.Attribute) and not (isinstance(f.value, ast.Name) and f.value.id in ("np", "numpy", "math")):
            vec = _has_vector_part(f.value, self.ctx) or (isinstance(f.value, ast.Name) and self.ctx.ndim(f.value.id) == 1)
            if vec and f.attr in _METHODS and not node.keywords:
                np_fn = ast.Attribute(value=ast.Name(id="np", ctx=ast.Load()), attr=f.attr, ctx=ast.Load())
                return ast.Call(func=np_fn, args=[f.value] + node.args, keywords=[])
            if vec and f.attr == "astype" and len(node.args) == 1 and not node.keywords:
                return ast.Call(func=node.args[0], args=[f.value], keywords=[])
        return node


class _Scalarise(ast.NodeTransformer):
    """Rewrite every sliced subscript / bare 1-D array in an expression to its
    element at position ``c``; records the extent of the first one seen."""

    def __init__(self, ctx: _Ctx, c: str):
        self.ctx = ctx
        self.c = c
        self.first_extent = None

    def visit_Subscript(self, node):
        sl = _slices_of(node)
        if not sl:
            # plain element access: indices may still contain expressions
            node.slice = self.visit(node.slice)
            return node
        if len(sl) > 1:
            raise RuntimeError(
                f"Using array expression of dimensionality > 1 is not supported: {ast.unparse(node)}"
            )
        dim, s = sl[0]
        lo, hi = _bounds(node, dim, s, self.ctx)
        if self.first_extent is None:
            self.first_extent = _extent(lo, hi)
        new_idx = _offset(lo, self.c)
        if isinstance(node.slice, ast.Tuple):
            elts = list(node.slice.elts)
            elts[dim] = new_idx
            node.slice = ast.Tuple(elts=elts, ctx=ast.Load())
        else:
            node.slice = new_idx
        return node

    def visit_Name(self, node):
        if isinstance(node.ctx, ast.Load) and self.ctx.ndim(node.id) == 1:
            if self.first_extent is None:
                self.first_extent = self.ctx.shape_name(node.id, 0)
            return ast.Subscript(value=node, slice=ast.Name(id=self.c, ctx=ast.Load()), ctx=ast.Load())
        return node

    def visit_Attribute(self, node):
        return node  # np.pi, X.shape: nothing to scalarise

    def visit_Call(self, node):
        node.args = [self.visit(a) for a in node.args]
        return node


def _simd_loop(c: str, extent, body, reduction=None) -> ast.For:
    loop = ast.For(
        target=ast.Name(id=c, ctx=ast.Store()),
        iter=ast.Call(
            func=ast.Name(id="range", ctx=ast.Load()),
            args=[ast.Constant(value=0), extent, ast.Constant(value=1)],
            keywords=[],
        ),
        body=body,
        orelse=[],
    )
    loop.pragma = {"simd": True}
    if reduction:
        op, var = reduction
        loop.pragma["reduction"] = f"{op}:{var}"
    loop.from_array_expr = True
    return loop


class _ReduceCalls(ast.NodeTransformer):
    """Hoist ``np.sum(E)`` / ``E1 @ E2`` out of an expression: each becomes a
    scalar temporary computed by a simd reduction loop placed before the
    statement."""

    def __init__(self, ctx: _Ctx):
        self.ctx = ctx
        self.prologue = []

    def _reduce(self, op: str, vec_expr, init=None, indexed=None):
        r = self.ctx.fresh("r")
        c = self.ctx.fresh("c")
        sc = _Scalarise(self.ctx, c)
        elem = sc.visit(copy.deepcopy(vec_expr))
        if sc.first_extent is None:
            raise RuntimeError(f"Reduction over a non-array expression: {ast.unparse(vec_expr)}")
        self.last_extent = sc.first_extent
        if indexed is not None:
            elem = indexed(elem, c, sc.first_extent)
        if init is not None:
            pass
        elif op == "+":
            init = ast.Constant(value=0)
        elif op == "*":
            init = ast.Constant(value=1)
        else:
            inf = ast.Call(func=ast.Name(id="float", ctx=ast.Load()), args=[ast.Constant(value="inf")], keywords=[])
            init = ast.UnaryOp(op=ast.USub(), operand=inf) if op == "max" else inf
        self.prologue.append(ast.Assign(targets=[ast.Name(id=r, ctx=ast.Store())], value=init))
        acc = ast.Name(id=r, ctx=ast.Load())
        if op in ("+", "*"):
            val = ast.BinOp(left=acc, op=ast.Add() if op == "+" else ast.Mult(), right=elem)
        else:
            val = ast.Call(func=ast.Name(id=op, ctx=ast.Load()), args=[acc, elem], keywords=[])
        upd = ast.Assign(targets=[ast.Name(id=r, ctx=ast.Store())], value=val)
        upd.reduce = op
        self.prologue.append(_simd_loop(c, sc.first_extent, [upd], reduction=(op, r)))
        return ast.Name(id=r, ctx=ast.Load())

    def _is_vec(self, node):
        return _has_vector_part(node, self.ctx) or self._is_vec_name(node)

    def visit_Call(self, node):
        f = node.func
        is_np = isinstance(f, ast.Attribute) and isinstance(f.value, ast.Name) and f.value.id in ("np", "numpy")
        if is_np and f.attr in _REDUCERS and len(node.args) == 1 and not node.keywords and self._is_vec(node.args[0]):
            inner = self.visit(node.args[0])  # nested reductions first
            return self._reduce(_REDUCERS[f.attr], inner)
        if is_np and f.attr in _DERIVED and node.args and not node.keywords and all(self._is_vec(a) for a in node.args):
            return self._derived(f.attr, [self.visit(a) for a in node.args], node)
        if (isinstance(f, ast.Name) and f.id == "len" and len(node.args) == 1 and _has_vector_part(node.args[0], self.ctx)):
            sc = _Scalarise(self.ctx, "__none")
            sc.visit(copy.deepcopy(node.args[0]))
            return sc.first_extent
        self.generic_visit(node)
        return node

    def _derived(self, fn: str, args, node):
        """``np.mean`` / ``var`` / ``std`` / ``any`` / ``all`` / ``count_nonzero`` / ``dot`` of
        1-D array expressions, spelled through sum / max / min reductions."""
        if fn in ("dot", "inner", "vdot"):
            if len(args) != 2:
                raise RuntimeError(f"np.{fn} takes two 1-D operands here: {ast.unparse(node)}")
            return self._reduce("+", ast.BinOp(left=args[0], op=ast.Mult(), right=args[1]))
        if len(args) != 1:
            raise RuntimeError(f"np.{fn} takes one 1-D operand here: {ast.unparse(node)}")
        e = args[0]
        if fn in ("mean", "average"):
            total = self._reduce("+", e, init=ast.Constant(value=0.0))
            return ast.BinOp(left=total, op=ast.Div(), right=copy.deepcopy(self.last_extent))
        if fn in ("var", "std"):
            total = self._reduce("+", e, init=ast.Constant(value=0.0))
            n = self.last_extent
            mean = ast.BinOp(left=total, op=ast.Div(), right=copy.deepcopy(n))
            m = self.ctx.fresh("r")
            self.prologue.append(ast.Assign(targets=[ast.Name(id=m, ctx=ast.Store())], value=mean))
            dev = ast.BinOp(left=copy.deepcopy(e), op=ast.Sub(), right=ast.Name(id=m, ctx=ast.Load()))
            sq = self._reduce("+", ast.BinOp(left=dev, op=ast.Mult(), right=copy.deepcopy(dev)), init=ast.Constant(value=0.0))
            var = ast.BinOp(left=sq, op=ast.Div(), right=copy.deepcopy(n))
            return var if fn == "var" else ast.BinOp(left=var, op=ast.Pow(), right=ast.Constant(value=0.5))
        if fn in ("argmax", "argmin"):
            # the extreme value first, then the smallest position that holds it
            best = self._reduce("max" if fn == "argmax" else "min", e)
            b = self.ctx.fresh("r")
            self.prologue.append(ast.Assign(targets=[ast.Name(id=b, ctx=ast.Store())], value=best))

            def position(elem, c, extent):
                hit = ast.Compare(left=elem, ops=[ast.Eq()], comparators=[ast.Name(id=b, ctx=ast.Load())])
                return ast.IfExp(test=hit, body=ast.Name(id=c, ctx=ast.Load()), orelse=copy.deepcopy(extent))

            first = self._reduce("min", e, init=ast.Constant(value=2 ** 62), indexed=position)
            return first
        truth = ast.Call(func=ast.Name(id="bool", ctx=ast.Load()), args=[e], keywords=[])
        if fn == "any":
            return self._reduce("max", truth, init=ast.Constant(value=False))
        if fn == "all":
            return self._reduce("min", truth, init=ast.Constant(value=True))
        assert fn == "count_nonzero"
        return self._reduce("+", ast.Call(func=ast.Name(id="int", ctx=ast.Load()), args=[truth], keywords=[]))

    def _is_vec_name(self, node):
        return isinstance(node, ast.Name) and self.ctx.ndim(node.id) == 1

    def visit_BinOp(self, node):
        self.generic_visit(node)
        if isinstance(node.op, ast.MatMult):
            prod = ast.BinOp(left=node.left, op=ast.Mult(), right=node.right)
            return self._reduce("+", prod)
        return node


def _refuse_shifted_self_reference(tgt, dim, lo, value, ctx: _Ctx):
    """``A[i, 1:] = f(A[i, :-1])``: NumPy evaluates the right-hand side before it
    stores anything; a loop whose iterations run side by side on the same row
    cannot (an element is overwritten by one lane while another still has to
    read its old value - the reference documents the same limit,
    docs/metal_simd_memory_hazards.md, "Slice with index offset").  Refused
    rather than computed wrongly."""
    if not isinstance(tgt.value, ast.Name):
        return
    t_elts = tgt.slice.elts if isinstance(tgt.slice, ast.Tuple) else [tgt.slice]
    others = [ast.unparse(e) for k, e in enumerate(t_elts) if k != dim]
    for n in ast.walk(value):
        if not (isinstance(n, ast.Subscript) and isinstance(n.value, ast.Name) and n.value.id == tgt.value.id):
            continue
        sl = _slices_of(n)
        n_elts = n.slice.elts if isinstance(n.slice, ast.Tuple) else [n.slice]
        if len(sl) != 1 or sl[0][0] != dim or len(n_elts) != len(t_elts):
            continue
        if [ast.unparse(e) for k, e in enumerate(n_elts) if k != dim] != others:
            continue
        n_lo, _ = _bounds(n, dim, sl[0][1], ctx)
        if ast.unparse(n_lo) != ast.unparse(lo):
            raise RuntimeError(
                f"`{ast.unparse(tgt)}` is updated from `{ast.unparse(n)}`, the same row at another offset: "
                "the elements cannot be updated side by side in place; write the result to another array"
            )


def _lower_assign(st: ast.Assign, ctx: _Ctx):
    out = []
    # 1. reductions inside the right-hand side become scalar temporaries
    rc = _ReduceCalls(ctx)
    st.value = rc.visit(st.value)
    out.extend(rc.prologue)
    tgt = st.targets[0]
    tgt_sliced = isinstance(tgt, ast.Subscript) and bool(_slices_of(tgt))
    if not tgt_sliced:
        if _has_vector_part(st.value, ctx):
            raise RuntimeError(f"Array expression assigned to a scalar location: {ast.unparse(st)}")
        out.append(st)
        return out
    # 2. elementwise statement over the target's extent
    sl = _slices_of(tgt)
    if len(sl) > 1:
        raise RuntimeError(f"Using array expression of dimensionality > 1 is not supported: {ast.unparse(tgt)}")
    c = ctx.fresh("c")
    dim, s = sl[0]
    lo, hi = _bounds(tgt, dim, s, ctx)
    _refuse_shifted_self_reference(tgt, dim, lo, st.value, ctx)
    new_tgt = copy.deepcopy(tgt)
    idx = _offset(lo, c)
    if isinstance(new_tgt.slice, ast.Tuple):
        elts = list(new_tgt.slice.elts)
        elts[dim] = idx
        new_tgt.slice = ast.Tuple(elts=elts, ctx=ast.Load())
    else:
        new_tgt.slice = idx
    sc = _Scalarise(ctx, c)
    new_val = sc.visit(st.value)
    body = ast.Assign(targets=[new_tgt], value=new_val)
    out.append(_simd_loop(c, _extent(lo, hi), [body]))
    return out


def _lower_block(stmts, ctx: _Ctx):
    out = []
    canon = _Canonical(ctx)
    for st in stmts:
        if isinstance(st, ast.Assign):
            st = canon.visit(st)
        if isinstance(st, ast.Assign) and (
            _has_vector_part(st, ctx)
        ):
            out.extend(_lower_assign(st, ctx))
            continue
        for f in ("body", "orelse"):
            sub = getattr(st, f, None)
            if isinstance(sub, list) and sub and isinstance(sub[0], ast.stmt):
                setattr(st, f, _lower_block(sub, ctx))
        out.append(st)
    return out


def transform(tree: ast.Module, val_map):
    """Returns the tree with array statements replaced by simd loops and the
    set of ``(array, dim)`` extents the new loops refer to as ``X_shape_d``."""
    ctx = _Ctx(val_map)
    tree.body = _lower_block(tree.body, ctx)
    ast.fix_missing_locations(tree)
    return tree, ctx.shape_refs
