"""Names a loop text refers to.

The run-time stub receives ``locals()``/``globals()`` of the caller and has to
pick the values the loop needs.  The reference delegates this to the
un-vendored ``astpass.passes.get_used_names.analyze(tree, no_funcname=True)``
(reference tree: appy/dispatcher.py:13-17); its contract as seen from that call
site is: every identifier that occurs in the loop text, except identifiers
that are only used as the callee of a call (``range``, ``max``, ``float``).
Here the order is the order of first occurrence in the source, which fixes the
positional argument order of the generated launcher.
"""
from __future__ import annotations

import ast
from functools import lru_cache

from . import source as src


def _ordered_nodes(node):
    yield node
    for child in ast.iter_child_nodes(node):
        yield from _ordered_nodes(child)


def used_names_of_tree(tree: ast.AST):
    callee_only = set()
    order = []
    seen = set()
    callee_nodes = set()
    for n in _ordered_nodes(tree):
        if isinstance(n, ast.Call) and isinstance(n.func, ast.Name):
            callee_nodes.add(id(n.func))
    for n in _ordered_nodes(tree):
        if isinstance(n, ast.Name):
            if id(n) in callee_nodes:
                callee_only.add(n.id)
                continue
            if n.id == src.MARKER:
                continue
            if n.id not in seen:
                seen.add(n.id)
                order.append(n.id)
    return order


@lru_cache(maxsize=4096)
def used_names(loop_source: str):
    """Tuple of identifiers used by ``loop_source`` (cached per text, so the
    loop is not re-parsed on every execution)."""
    return tuple(used_names_of_tree(src.parse(loop_source)))
