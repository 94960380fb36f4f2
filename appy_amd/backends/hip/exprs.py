"""Python expressions of the loop IR -> typed HIP C++ expressions.

Every method returns ``(code, Ty)``.  Types follow NumPy >= 2 promotion with
weak Python scalars (see :mod:`.dtypes`), so a kernel computes what the
un-jitted loop computes.  Calls are restricted to the functions the reference
accepts inside kernels (reference tree:
appy/backends/triton/passes/device_passes/rewrite_np_calls.py:4-26): ``np.*`` /
``math.*`` maths, ``max min abs int float pow`` and ``float('inf')``; anything
else raises ``ValueError("Unknown function: ...")``.
"""
from __future__ import annotations

import ast
import math
from dataclasses import dataclass

import numpy as np

from . import dtypes as T
from .dtypes import Ty

RESERVED = {
    # C++ keywords and names used by the generated code itself
    "alignas", "alignof", "and", "asm", "auto", "bool", "break", "case", "catch", "char", "class", "const",
    "constexpr", "continue", "default", "delete", "do", "double", "else", "enum", "explicit", "export",
    "extern", "false", "float", "for", "friend", "goto", "if", "inline", "int", "long", "mutable",
    "namespace", "new", "not", "nullptr", "operator", "or", "private", "protected", "public", "register",
    "return", "short", "signed", "sizeof", "static", "struct", "switch", "template", "this", "throw",
    "true", "try", "typedef", "typename", "union", "unsigned", "using", "virtual", "void", "volatile",
    "while", "xor", "appy", "threadIdx", "blockIdx", "blockDim", "gridDim", "main", "abs", "min", "max",
    "pow", "floor", "ceil", "sqrt", "exp", "log", "sin", "cos", "tan", "erf", "fabs", "fmod", "y0", "y1",
    "j0", "j1", "jn", "yn", "signbit", "isnan", "isinf", "div", "remainder", "round", "trunc", "rint",
}


def cname(name: str) -> str:
    """C++ identifier for a Python identifier."""
    return name + "_" if name in RESERVED else name


@dataclass
class ArrayParam:
    name: str
    ty: Ty          # element type (bool arrays are loaded as bytes)
    ndim: int
    stored: bool = False
    loaded: bool = False

    @property
    def elem_c(self) -> str:
        return "unsigned char" if self.ty.is_bool else self.ty.c


@dataclass
class ScalarParam:
    name: str
    ty: Ty


# unary maths: python name -> (float32 function, float64 function)
_UNARY_MATH = {
    "sqrt": ("sqrtf", "sqrt"), "exp": ("expf", "exp"), "exp2": ("exp2f", "exp2"), "expm1": ("expm1f", "expm1"),
    "log": ("logf", "log"), "log2": ("log2f", "log2"), "log10": ("log10f", "log10"), "log1p": ("log1pf", "log1p"),
    "sin": ("sinf", "sin"), "cos": ("cosf", "cos"), "tan": ("tanf", "tan"),
    "arcsin": ("asinf", "asin"), "arccos": ("acosf", "acos"), "arctan": ("atanf", "atan"),
    "asin": ("asinf", "asin"), "acos": ("acosf", "acos"), "atan": ("atanf", "atan"),
    "sinh": ("sinhf", "sinh"), "cosh": ("coshf", "cosh"), "tanh": ("tanhf", "tanh"),
    "arcsinh": ("asinhf", "asinh"), "arccosh": ("acoshf", "acosh"), "arctanh": ("atanhf", "atanh"),
    "asinh": ("asinhf", "asinh"), "acosh": ("acoshf", "acosh"), "atanh": ("atanhf", "atanh"),
    "floor": ("floorf", "floor"), "ceil": ("ceilf", "ceil"), "trunc": ("truncf", "trunc"), "rint": ("rintf", "rint"),
    "fabs": ("fabsf", "fabs"), "erf": ("erff", "erf"), "erfc": ("erfcf", "erfc"),
    "cbrt": ("cbrtf", "cbrt"), "gamma": ("tgammaf", "tgamma"), "lgamma": ("lgammaf", "lgamma"),
}
_BINARY_MATH = {
    "arctan2": ("atan2f", "atan2"), "atan2": ("atan2f", "atan2"), "hypot": ("hypotf", "hypot"),
    "fmod": ("fmodf", "fmod"), "copysign": ("copysignf", "copysign"),
    "power": ("powf", "pow"), "pow": ("powf", "pow"),
}
_CONSTANTS = {"pi": math.pi, "e": math.e, "inf": math.inf, "nan": math.nan, "tau": math.tau, "Inf": math.inf,
              "infty": math.inf, "NaN": math.nan, "euler_gamma": 0.5772156649015329}
_NP_CASTS = {"float32", "float64", "float16", "int8", "int16", "int32", "int64", "uint8", "uint16", "uint32",
             "uint64", "bool_"}
_MATH_MODULE_NAMES = ("np", "numpy", "math")


def _negative_literal(node):
    """k for the literal index ``-k`` (k > 0), else None."""
    if isinstance(node, ast.UnaryOp) and isinstance(node.op, ast.USub) and isinstance(node.operand, ast.Constant) \
            and type(node.operand.value) is int and node.operand.value > 0:
        return node.operand.value
    if isinstance(node, ast.Constant) and type(node.value) is int and node.value < 0:
        return -node.value
    return None


def cast(code: str, src: Ty, dst: Ty) -> str:
    if src.c == dst.c:
        return code
    return f"(({dst.c})({code}))"


def truth(code: str, ty: Ty) -> str:
    return code if ty.is_bool else f"(({code}) != 0)"


class ExprEmitter:
    """Typing + C++ spelling of expressions over a fixed set of kernel
    parameters and the current types of local variables."""

    def __init__(self, arrays, scalars, module_names):
        self.arrays = arrays            # name -> ArrayParam
        self.scalars = scalars          # name -> ScalarParam
        self.module_names = set(module_names)
        self.locals = {}                # name -> Ty (loop variables included)
        self.load_subst = {}            # unparsed subscript -> (code, Ty)
        self.shape_scalars = set()      # 'X_shape_k' names referenced
        self.stream_arrays = set()      # arrays whose scalar loads bypass the caches (read once by the launch)
        self.checked = False            # compare every index with the extent of its dimension
        self.sites = []                 # checked kernels: source text of the subscripts, by site number

    # ---- leaves ---------------------------------------------------------------
    def name_type(self, name: str):
        if name in self.locals:
            return self.locals[name]
        if name in self.scalars:
            return self.scalars[name].ty
        return None

    def emit(self, node):
        m = getattr(self, "e_" + type(node).__name__, None)
        if m is None:
            raise NotImplementedError(f"Expression not supported in a kernel: {ast.unparse(node)}")
        code, ty = m(node)
        if isinstance(node, (ast.BinOp, ast.UnaryOp)) and ty.is_int and ty.size < 4:
            # C++ computes 8- and 16-bit integers as `int`; NumPy wraps in the operands' type
            code = f"(({ty.c})({code}))"
        return code, ty

    def e_Constant(self, node):
        v = node.value
        if isinstance(v, bool):
            return ("true" if v else "false"), T.WEAK_BOOL
        if isinstance(v, int):
            return f"{v}LL", T.WEAK_INT
        if isinstance(v, float):
            return T.float_literal(v, T.F64), T.WEAK_FLOAT
        raise NotImplementedError(f"Constant not supported in a kernel: {v!r}")

    def e_Name(self, node):
        ty = self.name_type(node.id)
        if ty is None:
            if node.id in self.arrays:
                raise NotImplementedError(f"Whole-array use of `{node.id}` is only supported in 1-D array expressions")
            raise NameError(f"name `{node.id}` is read in the kernel before it has a value")
        return cname(node.id), ty

    def e_Attribute(self, node):
        if isinstance(node.value, ast.Name) and node.value.id in _MATH_MODULE_NAMES and node.attr in _CONSTANTS:
            return T.float_literal(_CONSTANTS[node.attr], T.F64), T.WEAK_FLOAT
        if isinstance(node.value, ast.Name) and node.value.id in self.arrays:
            arr = self.arrays[node.value.id]
            if node.attr == "ndim":
                return f"{arr.ndim}LL", T.WEAK_INT
            if node.attr == "size":
                for d in range(arr.ndim):
                    self.shape_scalars.add((arr.name, d))
                dims = [cname(f"{arr.name}_shape_{d}") for d in range(arr.ndim)] or ["1LL"]
                return "(" + " * ".join(dims) + ")", T.WEAK_INT
        raise NotImplementedError(f"Attribute not supported in a kernel: {ast.unparse(node)}")

    # ---- memory -----------------------------------------------------------------
    def site(self, sub: ast.Subscript) -> int:
        text = ast.unparse(sub)
        if text not in self.sites:
            self.sites.append(text)
        return self.sites.index(text)

    def inside_code(self, arr: ArrayParam, sub: ast.Subscript) -> str:
        """Condition under which every index of ``sub`` lies inside ``arr``."""
        elts = sub.slice.elts if isinstance(sub.slice, ast.Tuple) else [sub.slice]
        conds = []
        for d, e in enumerate(elts):
            if _negative_literal(e) is not None:
                k = _negative_literal(e)
                self.shape_scalars.add((arr.name, d))
                conds.append(f"({cname(f'{arr.name}_shape_{d}')} >= {k}LL)")
                continue
            code, ty = self.emit(e)
            self.shape_scalars.add((arr.name, d))
            conds.append(f"appy::inside({cast(code, ty, T.I64)}, {cname(f'{arr.name}_shape_{d}')})")
        return " && ".join(conds)

    def index_code(self, arr: ArrayParam, sub: ast.Subscript, check=None) -> str:
        check = self.checked if check is None else check
        site = self.site(sub) if check else -1
        elts = sub.slice.elts if isinstance(sub.slice, ast.Tuple) else [sub.slice]
        if len(elts) != arr.ndim:
            raise NotImplementedError(
                f"`{ast.unparse(sub)}`: {arr.ndim}-D array `{arr.name}` needs {arr.ndim} scalar indices"
            )
        terms = []
        for d, e in enumerate(elts):
            if isinstance(e, ast.Slice):
                raise NotImplementedError(f"Slice outside an array statement: {ast.unparse(sub)}")
            neg = _negative_literal(e)
            if neg is not None:
                # X[-k] counts from the end, as in Python
                self.shape_scalars.add((arr.name, d))
                code, ty = f"({cname(f'{arr.name}_shape_{d}')} - {neg}LL)", T.I64
            else:
                code, ty = self.emit(e)
            if not (ty.is_int or ty.is_bool):
                raise TypeError(f"Array index must be an integer: {ast.unparse(sub)}")
            code = cast(code, ty, T.I64)
            if check:
                # an index outside its dimension is reported and replaced by 0, so the access itself stays legal
                self.shape_scalars.add((arr.name, d))
                code = f"appy::at({code}, {cname(f'{arr.name}_shape_{d}')}, {site}, __oob)"
            if d < arr.ndim - 1:
                terms.append(f"{code} * {cname(arr.name)}_stride_{d}")
            else:
                terms.append(code)
        return " + ".join(terms)

    def e_Subscript(self, node):
        base = node.value
        # X.shape[k] that was not hoisted
        if (isinstance(base, ast.Attribute) and base.attr == "shape" and isinstance(base.value, ast.Name)
                and isinstance(node.slice, ast.Constant)):
            nm = f"{base.value.id}_shape_{node.slice.value}"
            self.shape_scalars.add((base.value.id, node.slice.value))
            return cname(nm), T.WEAK_INT
        if not isinstance(base, ast.Name) or base.id not in self.arrays:
            raise NotImplementedError(f"Subscript of a non-array in a kernel: {ast.unparse(node)}")
        key = ast.unparse(node)
        if key in self.load_subst:
            return self.load_subst[key]
        arr = self.arrays[base.id]
        arr.loaded = True
        code = f"{cname(arr.name)}[{self.index_code(arr, node)}]"
        if arr.name in self.stream_arrays and not arr.stored:
            code = f"__builtin_nontemporal_load(&{code})"
        if arr.ty.is_bool:
            code = f"({code} != 0)"
        return code, arr.ty

    # ---- operators ----------------------------------------------------------------
    def e_UnaryOp(self, node):
        code, ty = self.emit(node.operand)
        if isinstance(node.op, ast.USub):
            if ty.is_bool:
                ty2 = T.WEAK_INT if ty.weak else T.I64
                return f"(-{cast(code, ty, ty2)})", ty2
            return f"(-{code})", ty
        if isinstance(node.op, ast.UAdd):
            return code, ty
        if isinstance(node.op, ast.Not):
            return f"(!{truth(code, ty)})", T.BOOL
        if isinstance(node.op, ast.Invert):
            if ty.is_bool:
                return f"(!{code})", ty
            if ty.is_int:
                return f"(~{code})", ty
        raise NotImplementedError(f"Operator not supported in a kernel: {ast.unparse(node)}")

    def e_BinOp(self, node):
        lc, lt = self.emit(node.left)
        rc, rt = self.emit(node.right)
        op = node.op
        if isinstance(op, (ast.Add, ast.Sub, ast.Mult)):
            t = T.promote(lt, rt)
            if t.is_bool:
                if isinstance(op, ast.Add):
                    return f"({lc} || {rc})", t
                if isinstance(op, ast.Mult):
                    return f"({lc} && {rc})", t
                raise TypeError("boolean subtract is not defined")
            sym = {ast.Add: "+", ast.Sub: "-", ast.Mult: "*"}[type(op)]
            if t.name == "bfloat16":    # computed in float32 and rounded once, as PyTorch does
                return f"((__bf16)({cast(lc, lt, T.F32)} {sym} {cast(rc, rt, T.F32)}))", t
            return f"({cast(lc, lt, t)} {sym} {cast(rc, rt, t)})", t
        if isinstance(op, ast.Div):
            t = T.true_divide(lt, rt)
            if t.name == "bfloat16":
                return f"((__bf16)({cast(lc, lt, T.F32)} / {cast(rc, rt, T.F32)}))", t
            return f"({cast(lc, lt, t)} / {cast(rc, rt, t)})", t
        if isinstance(op, ast.FloorDiv):
            t = T.promote(lt, rt)
            if t.is_bool:
                t = T.WEAK_INT if t.weak else T.from_dtype(np.int8)
            a, b = cast(lc, lt, t), cast(rc, rt, t)
            if t.is_float:
                if t.size == 2:     # 16-bit floats: computed in float32, rounded once
                    return cast(f"appy::floordiv_float({cast(lc, lt, T.F32)}, {cast(rc, rt, T.F32)})", T.F32, t), t
                return f"appy::floordiv_float({a}, {b})", t
            if t.kind == "u":
                return f"appy::div_unsigned<{t.c}>({a}, {b})", t
            return f"appy::floordiv_int<{t.c}>({a}, {b})", t
        if isinstance(op, ast.Mod):
            t = T.promote(lt, rt)
            if t.is_bool:
                t = T.WEAK_INT if t.weak else T.from_dtype(np.int8)
            a, b = cast(lc, lt, t), cast(rc, rt, t)
            if t.is_float:
                if t.size == 2:     # 16-bit floats: computed in float32, rounded once
                    return cast(f"appy::mod_float({cast(lc, lt, T.F32)}, {cast(rc, rt, T.F32)})", T.F32, t), t
                return f"appy::mod_float({a}, {b})", t
            if t.kind == "u":
                return f"appy::mod_unsigned<{t.c}>({a}, {b})", t
            return f"appy::mod_int<{t.c}>({a}, {b})", t
        if isinstance(op, ast.Pow):
            t = T.promote(lt, rt)
            if isinstance(node.right, ast.Constant) and type(node.right.value) is int and node.right.value == 2:
                # x ** 2 is x * x exactly (one rounding either way); higher powers go through
                # pow like NumPy's, where repeated multiplication would round differently
                a = cast(lc, lt, t)
                return f"({a} * {a})", t
            if t.is_float:
                fn = "powf" if t.name == "float32" else "pow"
                return f"{fn}({cast(lc, lt, t)}, {cast(rc, rt, t)})", t
            if t.is_bool:
                t = T.WEAK_INT
            return f"appy::ipow<{t.c}>({cast(lc, lt, t)}, {cast(rc, rt, T.I64)})", t
        if isinstance(op, (ast.BitAnd, ast.BitOr, ast.BitXor)):
            t = T.promote(lt, rt)
            if t.is_float:
                raise TypeError(f"bitwise operator on floats: {ast.unparse(node)}")
            if t.is_bool:
                sym = {ast.BitAnd: "&&", ast.BitOr: "||", ast.BitXor: "!="}[type(op)]
            else:
                sym = {ast.BitAnd: "&", ast.BitOr: "|", ast.BitXor: "^"}[type(op)]
            return f"({cast(lc, lt, t)} {sym} {cast(rc, rt, t)})", t
        if isinstance(op, (ast.LShift, ast.RShift)):
            t = T.promote(lt, rt)
            if not t.is_int:
                raise TypeError(f"shift needs integers: {ast.unparse(node)}")
            sym = "<<" if isinstance(op, ast.LShift) else ">>"
            return f"({cast(lc, lt, t)} {sym} {cast(rc, rt, t)})", t
        raise NotImplementedError(f"Operator not supported in a kernel: {ast.unparse(node)}")

    def e_Compare(self, node):
        if (len(node.ops) == 1 and isinstance(node.ops[0], (ast.In, ast.NotIn))
                and isinstance(node.comparators[0], (ast.Tuple, ast.List, ast.Set)) and node.comparators[0].elts):
            # `x in (1, 2, 3)`: one of the values equals x
            tests = [ast.Compare(left=node.left, ops=[ast.Eq()], comparators=[e]) for e in node.comparators[0].elts]
            code, ty = self.e_BoolOp(ast.BoolOp(op=ast.Or(), values=tests))
            return (f"(!{code})" if isinstance(node.ops[0], ast.NotIn) else code), ty
        parts = []
        lc, lt = self.emit(node.left)
        for op, right in zip(node.ops, node.comparators):
            rc, rt = self.emit(right)
            sym = {ast.Lt: "<", ast.LtE: "<=", ast.Gt: ">", ast.GtE: ">=", ast.Eq: "==", ast.NotEq: "!="}.get(type(op))
            if sym is None:
                raise NotImplementedError(f"Comparison not supported in a kernel: {ast.unparse(node)}")
            t = T.promote(lt, rt)
            if t.is_int and lt.weak != rt.weak and (lt.is_int or lt.is_bool) and (rt.is_int or rt.is_bool) \
                    and t.name != "uint64":
                # a Python integer next to a typed one is compared by value (`u8 > -2` is true), not
                # squeezed into the other operand's type first
                t = T.I64
            parts.append(f"({cast(lc, lt, t)} {sym} {cast(rc, rt, t)})")
            lc, lt = rc, rt
        return ("(" + " && ".join(parts) + ")" if len(parts) > 1 else parts[0]), T.BOOL

    def e_BoolOp(self, node):
        sym = " && " if isinstance(node.op, ast.And) else " || "
        parts = []
        for v in node.values:
            c, t = self.emit(v)
            parts.append(truth(c, t))
        return "(" + sym.join(parts) + ")", T.BOOL

    def e_IfExp(self, node):
        tc, tt = self.emit(node.test)
        bc, bt = self.emit(node.body)
        oc, ot = self.emit(node.orelse)
        t = T.join(bt, ot)
        return f"({truth(tc, tt)} ? {cast(bc, bt, t)} : {cast(oc, ot, t)})", t

    # ---- calls ---------------------------------------------------------------------
    def _float_fn(self, names, args):
        """Apply a float function pair to already emitted ``(code, ty)`` args."""
        t = None
        for _, at in args:
            t = T.join(t, T.to_float(at)) if t is not None else T.to_float(at)
        half = t if t.size == 2 else None      # 16-bit floats: evaluated in float32, rounded back
        if half is not None:
            t = T.F32
        fn = names[0] if t.name == "float32" else names[1]
        code = f"{fn}({', '.join(cast(c, at, t) for c, at in args)})"
        if half is not None and half.name == "bfloat16":
            return cast(code, t, half), half
        return code, t

    def e_Call(self, node):
        f = node.func
        if node.keywords:
            raise NotImplementedError(f"Keyword arguments are not supported in a kernel: {ast.unparse(node)}")
        if isinstance(f, ast.Name):
            return self._builtin_call(f.id, node)
        if isinstance(f, ast.Attribute) and isinstance(f.value, ast.Name) and f.value.id in _MATH_MODULE_NAMES:
            return self._module_call(f.value.id, f.attr, node)
        raise ValueError(f"Unknown function: {ast.unparse(f)}")

    def _minmax(self, which, node):
        if len(node.args) < 2:
            raise NotImplementedError(f"{which}() of a single argument is not supported in a kernel")
        code, ty = self.emit(node.args[0])
        for a in node.args[1:]:
            c2, t2 = self.emit(a)
            t = T.join(ty, t2)
            op = "OpMax" if which == "max" else "OpMin"
            code = f"appy::{op}::f<{t.c}>({cast(code, ty, t)}, {cast(c2, t2, t)})"
            ty = t
        return code, ty

    def _builtin_call(self, name, node):
        args = node.args
        if name in ("max", "min"):
            return self._minmax(name, node)
        if name == "abs" and len(args) == 1:
            c, t = self.emit(args[0])
            if t.is_float:
                fn = "fabsf" if t.name == "float32" else "fabs"
                return f"{fn}({c})", t
            if t.kind == "u" or t.is_bool:
                return c, t
            return f"(({c}) < 0 ? -({c}) : ({c}))", t
        if name == "float" and len(args) == 1:
            a = args[0]
            if isinstance(a, ast.Constant) and isinstance(a.value, str):
                try:
                    v = float(a.value)
                except ValueError:
                    raise ValueError(f"Unknown function: {ast.unparse(node)}")
                return T.float_literal(v, T.F64), T.WEAK_FLOAT
            c, t = self.emit(a)
            return cast(c, t, T.WEAK_FLOAT), T.WEAK_FLOAT
        if name == "int" and len(args) == 1:
            c, t = self.emit(args[0])
            return cast(c, t, T.WEAK_INT), T.WEAK_INT
        if name == "bool" and len(args) == 1:
            c, t = self.emit(args[0])
            return truth(c, t), T.BOOL
        if name == "pow" and len(args) == 2:
            return self.e_BinOp(ast.BinOp(left=args[0], op=ast.Pow(), right=args[1]))
        if name == "len" and len(args) == 1 and isinstance(args[0], ast.Name) and args[0].id in self.arrays:
            self.shape_scalars.add((args[0].id, 0))
            return cname(f"{args[0].id}_shape_0"), T.WEAK_INT
        if name == "round" and len(args) == 1:       # Python's round(): half to even, an int
            c, t = self.emit(args[0])
            if not t.is_float:
                return c, t
            fn = "rintf" if t.name == "float32" else "rint"
            return f"((long long){fn}({c}))", T.WEAK_INT
        if name in _UNARY_MATH and len(args) == 1:        # `from math import sqrt`
            return self._float_fn(_UNARY_MATH[name], [self.emit(args[0])])
        raise ValueError(f"Unknown function: {name}")

    def _module_call(self, mod, attr, node):
        args = node.args
        is_math = mod == "math"
        if attr in _UNARY_MATH and len(args) == 1:
            c, t = self.emit(args[0])
            if is_math:  # math.* works on Python floats
                code, _ = self._float_fn(_UNARY_MATH[attr], [(cast(c, t, T.F64), T.F64)])
                if attr in ("floor", "ceil", "trunc"):
                    return cast(code, T.F64, T.WEAK_INT), T.WEAK_INT
                return code, T.WEAK_FLOAT
            if attr in ("floor", "ceil", "trunc", "rint", "fabs") and not t.is_float:
                t2 = T.to_float(t)
                return self._float_fn(_UNARY_MATH[attr], [(cast(c, t, t2), t2)])
            return self._float_fn(_UNARY_MATH[attr], [(c, t)])
        if attr in _BINARY_MATH and len(args) == 2:
            a = self.emit(args[0])
            b = self.emit(args[1])
            if attr in ("power", "pow") and not is_math:
                return self.e_BinOp(ast.BinOp(left=args[0], op=ast.Pow(), right=args[1]))
            if is_math:
                code, _ = self._float_fn(_BINARY_MATH[attr], [(cast(a[0], a[1], T.F64), T.F64), (cast(b[0], b[1], T.F64), T.F64)])
                return code, T.WEAK_FLOAT
            return self._float_fn(_BINARY_MATH[attr], [a, b])
        if attr in ("maximum", "fmax") and len(args) == 2:
            return self._minmax("max", node)
        if attr in ("minimum", "fmin") and len(args) == 2:
            return self._minmax("min", node)
        if attr in ("abs", "absolute") and len(args) == 1:
            return self._builtin_call("abs", node)
        if attr == "where" and len(args) == 3:
            return self.e_IfExp(ast.IfExp(test=args[0], body=args[1], orelse=args[2]))
        if attr == "square" and len(args) == 1:
            return self.e_BinOp(ast.BinOp(left=args[0], op=ast.Mult(), right=args[0]))
        if attr in _NP_CASTS and len(args) == 1 and not is_math:
            c, t = self.emit(args[0])
            dst = T.from_dtype("bool" if attr == "bool_" else attr)
            return cast(c, t, dst), dst
        if attr in ("isnan", "isinf") and len(args) == 1:
            c, t = self.emit(args[0])
            if not t.is_float:
                return "false", T.BOOL
            return f"(__builtin_{attr}({c}) != 0)", T.BOOL
        if attr == "isfinite" and len(args) == 1:
            c, t = self.emit(args[0])
            if not t.is_float:
                return "true", T.BOOL
            return f"(__builtin_isfinite({c}) != 0)", T.BOOL
        # the rest are spelled through operators and functions that exist already
        P = ast.parse
        call = lambda fn, *xs: ast.Call(func=P(fn, mode="eval").body, args=list(xs), keywords=[])   # noqa: E731
        num = lambda v: ast.Constant(value=v)                                                          # noqa: E731
        if attr == "clip" and len(args) == 3:
            return self._minmax("min", call("min", call("max", args[0], args[1]), args[2]))
        if attr in ("mod", "remainder") and len(args) == 2:
            return self.e_BinOp(ast.BinOp(left=args[0], op=ast.Mod(), right=args[1]))
        if attr == "floor_divide" and len(args) == 2:
            return self.e_BinOp(ast.BinOp(left=args[0], op=ast.FloorDiv(), right=args[1]))
        if attr in ("divide", "true_divide") and len(args) == 2:
            return self.e_BinOp(ast.BinOp(left=args[0], op=ast.Div(), right=args[1]))
        if attr in ("add", "subtract", "multiply") and len(args) == 2:
            op = {"add": ast.Add(), "subtract": ast.Sub(), "multiply": ast.Mult()}[attr]
            return self.e_BinOp(ast.BinOp(left=args[0], op=op, right=args[1]))
        if attr == "negative" and len(args) == 1:
            return self.e_UnaryOp(ast.UnaryOp(op=ast.USub(), operand=args[0]))
        if attr == "reciprocal" and len(args) == 1:
            return self.e_BinOp(ast.BinOp(left=num(1.0), op=ast.Div(), right=args[0]))
        if attr in ("deg2rad", "radians", "rad2deg", "degrees") and len(args) == 1:
            f = math.pi / 180.0 if attr in ("deg2rad", "radians") else 180.0 / math.pi
            if is_math:
                c, t = self.emit(args[0])
                return f"({cast(c, t, T.F64)} * {T.float_literal(f, T.F64)})", T.WEAK_FLOAT
            c, t = self.emit(args[0])
            ft = T.to_float(t)
            return f"({cast(c, t, ft)} * {T.float_literal(f, ft.strong() if not ft.weak else T.F64)})", ft
        if attr in ("round", "around", "round_") and len(args) == 1 and not is_math:
            return self._module_call(mod, "rint", call("np.rint", args[0]))   # half to even, like NumPy
        if attr == "sign" and len(args) == 1:
            c, t = self.emit(args[0])
            if t.is_bool or t.kind == "u":
                return f"(({t.c})(({c}) != 0))", t
            zero = "0" if t.is_int else T.float_literal(0.0, t if not t.weak else T.F64)
            return f"(({t.c})((({c}) > {zero}) - (({c}) < {zero})))", t
        if attr == "heaviside" and len(args) == 2:
            test_neg = ast.Compare(left=args[0], ops=[ast.Lt()], comparators=[num(0.0)])
            test_zero = ast.Compare(left=args[0], ops=[ast.Eq()], comparators=[num(0.0)])
            return self.e_IfExp(ast.IfExp(test=test_neg, body=num(0.0),
                                          orelse=ast.IfExp(test=test_zero, body=args[1], orelse=num(1.0))))
        raise ValueError(f"Unknown function: {mod}.{attr}")
