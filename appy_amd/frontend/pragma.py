"""Pragma grammar of the APPy annotations.

Behaviour follows the reference parser (appy/utils.py:97-150 in the reference
tree): a pragma is a sequence of whitespace separated clauses, each either a
bare word (``simd``) or a word with a parenthesised, comma separated argument
list (``shared(a, b)``).  ``parallel`` directly followed by ``for`` forms the
single clause ``parallel_for``.  ``shared``/``to``/``from`` always carry a
list, any other clause with arguments carries a string (one argument) or a
tuple (several).  A clause outside the recognised set is an error whose
message names the clause (pinned by the reference's
tests/unit/general/pragma/test_invalid_pragma.py:37-42).
"""
from __future__ import annotations

import re
from collections import OrderedDict

PRAGMA_PREFIX = "#pragma"

RECOGNISED_CLAUSES = frozenset(
    {"parallel_for", "simd", "block", "reduction", "shared", "to", "from", "atomic"}
)
_LIST_CLAUSES = frozenset({"shared", "to", "from"})

_CLAUSE_WITH_ARGS = re.compile(r"(\w+)\s*\(([^)]*)\)")
_BARE_WORD = re.compile(r"\w+")


def is_pragma_text(text: str) -> bool:
    """True for comment text that the per-loop passes treat as a pragma
    (reference: appy/frontend/attach_pragma.py:9, note the trailing blank)."""
    return text.startswith(PRAGMA_PREFIX + " ")


def is_parallel_for_text(text: str) -> bool:
    """True for the comments the decoration-time passes react to
    (reference: appy/frontend/process_shared.py:22)."""
    return text.startswith(PRAGMA_PREFIX + " parallel for")


def _clauses(body: str):
    pos = 0
    n = len(body)
    while pos < n:
        if body[pos].isspace():
            pos += 1
            continue
        m = _CLAUSE_WITH_ARGS.match(body, pos)
        if m:
            args = tuple(a.strip() for a in m.group(2).split(",") if a.strip())
            yield m.group(1), args
            pos = m.end()
            continue
        m = _BARE_WORD.match(body, pos)
        if not m:
            raise ValueError(f"Unexpected syntax at: {body[pos:]}")
        yield m.group(0), None
        pos = m.end()


def parse_pragma(text: str) -> "OrderedDict[str, object]":
    """``'#pragma parallel for simd shared(s)'`` ->
    ``{'parallel_for': True, 'simd': True, 'shared': ['s']}``."""
    body = text.strip()
    if body.startswith(PRAGMA_PREFIX):
        body = body[len(PRAGMA_PREFIX):]
    body = body.strip()

    raw = list(_clauses(body))
    out: "OrderedDict[str, object]" = OrderedDict()
    k = 0
    while k < len(raw):
        key, args = raw[k]
        if key == "parallel" and args is None and k + 1 < len(raw) and raw[k + 1][0] == "for":
            out["parallel_for"] = True
            k += 2
            continue
        if args is None:
            out[key] = True
        elif key in _LIST_CLAUSES:
            out[key] = list(args)
        elif len(args) == 1:
            out[key] = args[0]
        elif len(args) == 0:
            raise ValueError(f"Clause `{key}` needs at least one argument in `{body}`")
        else:
            out[key] = args
        k += 1

    for key in out:
        if key not in RECOGNISED_CLAUSES:
            raise ValueError(f"Unrecognized pragma clause: `{key}` in `{body}`")
    return out


def format_pragma(clauses) -> str:
    """Inverse of :func:`parse_pragma` (reference: appy/utils.py:153-172)."""
    words = []
    if clauses.get("parallel_for"):
        words += ["parallel", "for"]
    for key, val in clauses.items():
        if key == "parallel_for":
            continue
        if val is True:
            words.append(key)
        elif isinstance(val, (tuple, list)):
            words.append(f"{key}({', '.join(val)})")
        else:
            words.append(f"{key}({val})")
    return PRAGMA_PREFIX + " " + " ".join(words)
