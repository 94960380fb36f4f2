"""appy_amd - annotated Python loops on AMD MI355X (gfx950).

``@jit`` rewrites every loop annotated with ``#pragma parallel for ...`` into a
call of :func:`_kernel_launch`, which generates a HIP C++ kernel for the loop,
compiles it with hiprtc and launches it through ``libappy_hip.so``.  The user
surface (decorator, pragma grammar, by-value scalars, ``shared()`` scalars,
NumPy arrays copied in and out, GPU tensors used in place) is the one of the
reference package (reference tree: appy/__init__.py:18-151).
"""
from __future__ import annotations

import ast
import builtins as _builtins
import inspect
import os
import sys
import textwrap

__version__ = "0.1.0"  # of this package, not of the reference it is compatible with
from . import dispatcher
from .residency import invalidate, resident, sync_host  # noqa: F401 - part of the public interface
from .graphs import graph  # noqa: F401
from .frontend import source as _source
from .frontend import static_rewrite as _static_rewrite

_DEFAULT_OPTIONS = (
    ("backend", None),
    ("dry_run", False),
    ("dump_code", False),
    ("dump_code_to_file", None),
    ("verbose_static_rewrite", False),
    ("verbose_block_loop", False),
)


def _kernel_launch(loop_source, loop_name, scope, global_scope, options):
    """Run-time stub that stands where an annotated loop stood.

    ``loop_source`` is the pragma line followed by the loop, ``loop_name`` is
    ``kernel_loop_N``, ``scope``/``global_scope`` are ``locals()``/``globals()``
    of the calling function (reference: appy/__init__.py:18-35)."""
    dispatcher.codegen(options.get("backend"), loop_source, loop_name, scope, global_scope, options)


def _reduction_result(buffer, start):
    """Value of a scalar that a ``prange`` loop reduced in a float64 buffer: the
    type the un-jitted loop would most plausibly have produced - an ``int`` when
    the start value was an ``int`` and the result is integral, else a ``float``."""
    value = buffer.item()
    if type(start) in (int, bool) and value == int(value) and abs(value) < 2.0 ** 53:
        return int(value)
    return value


def release():
    """Give back the device memory the compiled loops hold between launches - scratch buffers of launches made of
    several kernels, row plans (the kept order of the elements of CSR-like loops) - and what the pooled
    allocator has cached.  Waits for the launches that use that memory.  The loops stay compiled; the next
    launch of a loop allocates again what it needs."""
    from .backends.hip import codegen as _cg
    from .backends.hip import runtime as _rt

    for _f, _src in list(_cg.code_cache.values()):
        _f.release()
    _rt.check(_rt.lib().appy_hip_pool_trim())


def set_default_options(options):
    for key, val in _DEFAULT_OPTIONS:
        options.setdefault(key, val)
    if os.environ.get("APPY_HIP_CHECK_BOUNDS") == "1":
        # a whole program under device-side index checks, without touching its decorators
        options.setdefault("check_bounds", True)


def rewrite_loops(fn, **options):
    """Source of ``fn`` -> rewritten function object (reference:
    appy/__init__.py:38-65)."""
    source = textwrap.dedent(inspect.getsource(fn))
    tree = _source.parse(source)
    if options.get("shader", False):
        raise NotImplementedError("shader loops are not part of the HIP execution path")
    # carried to the code generator through the stub: names the device kernels
    # after the function they come from, which keeps profiles readable
    options.setdefault("fn_name", fn.__name__)
    tree, _loops = _static_rewrite.transform(tree, options)
    new_source = ast.unparse(tree)
    if options["verbose_static_rewrite"]:
        print("[Static Rewrite] new code:\n", new_source)
    import numpy

    g = fn.__globals__
    g["numpy"] = numpy
    # The stub is spelled `appy._kernel_launch`; make that name resolve even if
    # the caller imported this package under another name.
    g.setdefault("appy", sys.modules[__name__])
    free = fn.__code__.co_freevars
    if free and fn.__closure__:
        new_fn = _with_closure(fn, new_source, g)
    else:
        namespace = {}
        exec(compile(new_source, filename=f"<appy:{fn.__name__}>", mode="exec"), g, namespace)
        new_fn = namespace[fn.__name__]
    new_fn.__appy_source__ = new_source
    return new_fn


def _with_closure(fn, new_source, g):
    """The rewritten function bound to the cells ``fn`` closes over, so that names of
    an enclosing function (constants, helper functions defined next to the kernel)
    stay visible, late binding included.  The loops have become strings, so each free
    variable is mentioned once at the top of the body: that keeps it a free variable of
    the new code object and puts it into the ``locals()`` the launch stub looks names up in."""
    import types

    free = fn.__code__.co_freevars
    tree = ast.parse(new_source)
    fdef = next(n for n in tree.body if isinstance(n, (ast.FunctionDef, ast.AsyncFunctionDef)) and n.name == fn.__name__)
    mention = ast.Expr(value=ast.Tuple(elts=[ast.Name(id=v, ctx=ast.Load()) for v in free], ctx=ast.Load()))
    at = 1 if (fdef.body and isinstance(fdef.body[0], ast.Expr) and isinstance(fdef.body[0].value, ast.Constant)
               and isinstance(fdef.body[0].value.value, str)) else 0
    fdef.body.insert(at, mention)
    factory = ast.FunctionDef(
        name="__appy_factory", args=ast.arguments(posonlyargs=[], args=[], kwonlyargs=[], kw_defaults=[], defaults=[]),
        body=[ast.Assign(targets=[ast.Name(id=v, ctx=ast.Store()) for v in free], value=ast.Constant(value=None)),
              fdef, ast.Return(value=ast.Name(id=fn.__name__, ctx=ast.Load()))],
        decorator_list=[])
    module = ast.fix_missing_locations(ast.Module(body=[factory], type_ignores=[]))
    namespace = {}
    exec(compile(module, filename=f"<appy:{fn.__name__}>", mode="exec"), g, namespace)
    shell = namespace["__appy_factory"]()
    cells = dict(zip(free, fn.__closure__))
    new_fn = types.FunctionType(shell.__code__, g, fn.__name__, shell.__defaults__,
                                tuple(cells[v] for v in shell.__code__.co_freevars))
    new_fn.__kwdefaults__ = shell.__kwdefaults__
    new_fn.__dict__.update(shell.__dict__)
    return new_fn


def jit(fn=None, **options):
    set_default_options(options)
    if fn:
        return rewrite_loops(fn, **options)

    def jit_with_args(fn1):
        return rewrite_loops(fn1, **options)

    return jit_with_args


def shader(fn=None, **options):
    """Shader-style kernels (one function body per work-item) are an experiment of the
    reference's Metal and Numba back ends (reference: appy/__init__.py:84-92); the HIP
    execution path runs annotated loops only."""
    raise NotImplementedError("shader functions are not part of the HIP execution path; annotate a loop with "
                              "`#pragma parallel for` instead")


cpu_shader = shader


# ---- names usable inside annotated functions -------------------------------
def vidx(start, stepsize, bound=None):
    """Slice of at most ``stepsize`` indices from ``start``, clipped at
    ``bound`` (reference: appy/__init__.py:95-100)."""
    stop = start + stepsize
    if bound:
        stop = min(bound, stop)
    return slice(start, stop)


class prange(object):
    """Parallel range: identical to ``range`` when executed by the interpreter
    (reference: appy/__init__.py:105-110)."""

    def __new__(cls, *args, shared=None):
        return _builtins.range(*args)


built_in_range = _builtins.range


def range(*args, parallel=False, simd=False):  # noqa: A001 - mirrors the reference's name
    return _builtins.range(*args)


# ---- explicit data placement -------------------------------------------------
def _to_gpu(a):
    import torch

    kind = f"{type(a).__module__}.{type(a).__name__}"
    if kind == "numpy.ndarray":
        return torch.from_numpy(a).to("cuda")
    if isinstance(a, torch.Tensor):
        return a.to("cuda")
    if isinstance(a, list):
        return torch.tensor(a).to("cuda")
    if type(a) in (int, float):
        return a
    raise AssertionError("Unsupported type to transfer to GPU")


def to_gpu(*args):
    """NumPy arrays / tensors / lists -> tensors resident in HBM (reference:
    appy/__init__.py:118-135; 'cuda' is the device name of ROCm builds of
    PyTorch as well)."""
    if len(args) == 1:
        return _to_gpu(args[0])
    return [_to_gpu(a) for a in args]


def _to_cpu(a):
    import torch

    if isinstance(a, torch.Tensor):
        if a.ndim == 0:
            return a.item()
        return a.to("cpu").numpy()
    return a


def to_cpu(*args):
    if len(args) == 1:
        return _to_cpu(args[0])
    return [_to_cpu(a) for a in args]
