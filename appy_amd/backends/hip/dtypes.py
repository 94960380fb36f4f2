"""Scalar types of generated kernels and NumPy's promotion rules.

HIP C++ needs a static type for every value.  The rules follow what the
un-jitted loop computes under NumPy >= 2 (NEP 50): array elements and NumPy
scalars are *strong* (they carry their dtype), Python ``int``/``float``/
``bool`` values and literals are *weak* (they adopt the dtype of a strong
operand of the same or a higher kind, otherwise they are int64 / float64).
"""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np

_C_NAMES = {
    "bool": "bool",
    "int8": "signed char",
    "uint8": "unsigned char",
    "int16": "short",
    "uint16": "unsigned short",
    "int32": "int",
    "uint32": "unsigned int",
    "int64": "long long",
    "uint64": "unsigned long long",
    "float16": "_Float16",
    "bfloat16": "__bf16",       # tensors only: NumPy has no such dtype
    "float32": "float",
    "float64": "double",
}


@dataclass(frozen=True)
class Ty:
    """A scalar type: NumPy dtype name plus the weak flag."""

    name: str
    weak: bool = False

    @property
    def dtype(self) -> np.dtype:
        return np.dtype(self.name)

    @property
    def kind(self) -> str:
        if self.name == "bfloat16":
            return "f"
        return self.dtype.kind  # 'b', 'i', 'u', 'f'

    @property
    def is_float(self) -> bool:
        return self.kind == "f"

    @property
    def is_int(self) -> bool:
        return self.kind in "iu"

    @property
    def is_bool(self) -> bool:
        return self.kind == "b"

    @property
    def size(self) -> int:
        if self.name == "bfloat16":
            return 2
        return self.dtype.itemsize

    @property
    def c(self) -> str:
        return _C_NAMES[self.name]

    def strong(self) -> "Ty":
        return Ty(self.name, False)

    def __str__(self):
        return ("weak " if self.weak else "") + self.name


BOOL = Ty("bool")
I32 = Ty("int32")
I64 = Ty("int64")
F32 = Ty("float32")
F64 = Ty("float64")
WEAK_INT = Ty("int64", True)
WEAK_FLOAT = Ty("float64", True)
WEAK_BOOL = Ty("bool", True)


BF16 = Ty("bfloat16")


def _dtype_name(dtype) -> str:
    return "bfloat16" if isinstance(dtype, str) and dtype == "bfloat16" else np.dtype(dtype).name


def supported(dtype) -> bool:
    return _dtype_name(dtype) in _C_NAMES


def from_dtype(dtype) -> Ty:
    name = _dtype_name(dtype)
    if name not in _C_NAMES:
        raise TypeError(f"dtype {name} is not supported in generated kernels")
    return Ty(name)


_WEAK_SAMPLE = {"b": True, "i": 1, "u": 1, "f": 1.0}


def promote(a: Ty, b: Ty) -> Ty:
    """Type of ``a (op) b`` for an arithmetic operator."""
    if "bfloat16" in (a.name, b.name):
        # PyTorch's rules (the type only exists for tensors): Python scalars, integers and
        # booleans adopt bfloat16, float16 meets it in float32, wider floats win
        o = b if a.name == "bfloat16" else a
        if o.weak or not o.is_float or o.name == "bfloat16":
            return BF16
        return F32 if o.name == "float16" else o.strong()
    if a.weak and b.weak:
        if a.is_float or b.is_float:
            return WEAK_FLOAT
        if a.is_int or b.is_int:
            return WEAK_INT
        return WEAK_BOOL
    if a.weak or b.weak:
        w, s = (a, b) if a.weak else (b, a)
        res = np.result_type(s.dtype, _WEAK_SAMPLE[w.kind])
        return from_dtype(res)
    return from_dtype(np.result_type(a.dtype, b.dtype))


def join(a: Ty | None, b: Ty | None) -> Ty | None:
    """Type of a variable that is assigned values of type ``a`` and ``b``."""
    if a is None:
        return b
    if b is None:
        return a
    if a == b:
        return a
    return promote(a, b)


def true_divide(a: Ty, b: Ty) -> Ty:
    t = promote(a, b)
    if t.is_float:
        return t
    return WEAK_FLOAT if t.weak else F64


def to_float(t: Ty) -> Ty:
    """Result type of a NumPy floating-point ufunc (``np.sqrt``) applied to ``t``."""
    if t.is_float:
        return t
    if t.weak:
        return WEAK_FLOAT
    return from_dtype(np.sqrt(np.ones(1, dtype=t.dtype)).dtype)


def of_python_value(v) -> Ty | None:
    """Type of a by-value kernel argument; None if ``v`` is not a scalar."""
    if isinstance(v, bool):
        return WEAK_BOOL
    if isinstance(v, int):
        return WEAK_INT
    if isinstance(v, float):
        return WEAK_FLOAT
    if isinstance(v, np.generic):
        if supported(v.dtype):
            return from_dtype(v.dtype)
    return None


def float_literal(v: float, t: Ty) -> str:
    """C++ spelling of the Python float ``v`` in type ``t``."""
    import math

    if math.isnan(v):
        base = "__builtin_nan(\"\")"
    elif math.isinf(v):
        base = "__builtin_inf()" if v > 0 else "(-__builtin_inf())"
    else:
        base = repr(float(v))
        if "e" not in base and "." not in base:
            base += ".0"
    if t.name == "float64":
        return base
    return f"(({t.c}){base})"


def identity_literal(op: str, t: Ty) -> str:
    """Neutral element of a reduction operator in type ``t``."""
    if op == "+":
        return f"(({t.c})0)"
    if op == "*":
        return f"(({t.c})1)"
    if t.is_float:
        inf = "__builtin_inf()"
        return f"(({t.c})(-{inf}))" if op == "max" else f"(({t.c}){inf})"
    if t.is_bool:
        return "false" if op == "max" else "true"
    info = np.iinfo(t.dtype)
    val = info.min if op == "max" else info.max
    if t.name == "int64" and op == "max":
        return "((long long)(-9223372036854775807LL - 1))"
    suffix = "ULL" if t.kind == "u" else "LL"
    return f"(({t.c}){val}{suffix})"


def partial_type(ty: Ty) -> Ty:
    """Type of the per-lane partial results of a reduction: registers and cross-lane
    steps are 32 or 64 bits wide, so 16-bit floats accumulate in float32 (rounded once,
    when the team combines) and 8/16-bit integers and flags in 32-bit integers (sums wrap
    to the narrow type at the end exactly as they would have step by step)."""
    if ty.size >= 4:
        return ty
    if ty.is_float:
        return F32
    return Ty("uint32") if ty.kind == "u" else I32


def partial_identity(op: str, ty: Ty, pty: Ty) -> str:
    """Neutral element of ``op`` over ``ty``, written in the partial type ``pty``."""
    if pty == ty or ty.is_float:
        return identity_literal(op, pty)
    if ty.is_bool:
        return "0" if op in ("max", "+") else "1"
    return f"(({pty.c}){identity_literal(op, ty)})"
