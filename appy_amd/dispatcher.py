"""Per-execution dispatch of an outlined loop.

Collects the run-time values of the names the loop uses, asks the HIP code
generator for a launcher (cached per loop text and argument types) and calls
it.  Mirrors the reference's dispatcher (reference tree:
appy/dispatcher.py:12-60) with one back end instead of a platform switch.
"""
from __future__ import annotations

import math
import types as _types
import warnings

import numpy as np

from .frontend.names import used_names

_warned_alias = set()


def _resolve_backend(name):
    if name is None or name == "hip":
        return "hip"
    if name == "triton":
        # Programs written for the reference name its GPU back end explicitly;
        # there is a single GPU back end here, so the name is taken as "the GPU".
        if name not in _warned_alias:
            _warned_alias.add(name)
            warnings.warn("backend='triton' runs on the HIP back end of appy_amd", stacklevel=4)
        return "hip"
    raise NotImplementedError("Unknown backend:" + str(name))


def _by_value(v):
    """A 0-d array or tensor (``np.array(2.0)``, ``torch.tensor(2.0)``, the result of a
    ``.sum()``) enters a kernel as the scalar it holds, in its own dtype."""
    if isinstance(v, np.ndarray):
        return v[()]
    host = v.detach().cpu()
    try:
        return host.numpy()[()]
    except TypeError:           # a dtype NumPy does not have (bfloat16)
        return host.item()


def build_val_map(loop_source, local_scope, global_scope):
    val_map = {}
    for k in used_names(loop_source):      # locals shadow globals; no copy of either scope
        if k in local_scope:
            v = local_scope[k]
        elif k in global_scope:
            v = global_scope[k]
        else:
            continue
        if getattr(v, "ndim", 1) == 0 and not isinstance(v, np.generic) and hasattr(v, "dtype"):
            v = _by_value(v)
        val_map[k] = v
    val_map.setdefault("np", np)
    val_map.setdefault("math", math)
    return val_map


def codegen(backend_name, loop_source, loop_name, local_scope, global_scope, options):
    _resolve_backend(backend_name)
    val_map = build_val_map(loop_source, local_scope, global_scope)

    from .backends.hip.codegen import codegen as hip_codegen

    f, _code_src = hip_codegen(loop_source, loop_name, val_map, options)

    if options.get("dry_run"):
        # Code generation has run (its errors surface); now interpret the loop
        # text itself with the caller's values (reference: appy/dispatcher.py:46-53).
        # The caller's locals take precedence over its globals; results travel
        # through in-place mutation of arrays, exactly as for a kernel launch.
        try:
            code_obj = compile(loop_source, filename=f"<{loop_name}>", mode="exec")
            scope = dict(global_scope)
            scope.update(local_scope)
            exec(code_obj, scope)
        except Exception as e:
            raise RuntimeError(f"Error executing loop {loop_name} in dry_run mode: {e}")
        return

    args = [v for v in val_map.values() if not isinstance(v, _types.ModuleType)]
    f(*args)
