"""Comment-aware parsing for annotated Python source.

The standard ``ast`` module drops comments, and the annotations of this
programming model are comments (``#pragma parallel for simd``).  The reference
relies on the third-party ``ast_comments`` package for ``Comment`` nodes
(appy/__init__.py:5,41 in the reference tree).  Here a pragma comment that
stands alone on its line is turned, before parsing, into an expression
statement that calls a marker name, so it survives as an ordinary AST node:

    #pragma simd            ->     __appy_pragma__('#pragma simd')

and :func:`unparse` maps such statements back to comment lines.  Only
comments starting with ``#pragma`` are kept; every other comment is dropped,
which is invisible to the passes (none of them reads ordinary comments).
"""
from __future__ import annotations

import ast
import io
import re
import tokenize

MARKER = "__appy_pragma__"

_MARKER_LINE = re.compile(r"^(\s*)" + re.escape(MARKER) + r"\((.*)\)\s*$")


def _pragma_comment_lines(source: str):
    """Line numbers (1-based) -> comment text for comments alone on a line."""
    found = {}
    code_lines = set()
    try:
        toks = list(tokenize.generate_tokens(io.StringIO(source).readline))
    except (tokenize.TokenError, IndentationError):
        toks = []
    skip = {tokenize.COMMENT, tokenize.NL, tokenize.NEWLINE, tokenize.INDENT,
            tokenize.DEDENT, tokenize.ENDMARKER, tokenize.ENCODING}
    for t in toks:
        if t.type not in skip:
            for ln in range(t.start[0], t.end[0] + 1):
                code_lines.add(ln)
    for t in toks:
        if t.type == tokenize.COMMENT and t.string.startswith("#pragma") and t.start[0] not in code_lines:
            found[t.start[0]] = t.string.rstrip()
    return found


def _indent_of(line: str) -> str:
    return line[: len(line) - len(line.lstrip())]


def mark_pragmas(source: str) -> str:
    """Replace stand-alone pragma comment lines by marker statements.

    A comment may be indented arbitrarily; the marker statement takes the
    indentation of the next line that holds code, so that it lands in the same
    block as the statement it annotates.
    """
    comments = _pragma_comment_lines(source)
    if not comments:
        return source
    lines = source.split("\n")

    def next_code_indent(idx: int) -> str:
        for j in range(idx + 1, len(lines)):
            s = lines[j].strip()
            if s and not s.startswith("#"):
                return _indent_of(lines[j])
        return _indent_of(lines[idx])

    for ln, text in comments.items():
        idx = ln - 1
        lines[idx] = f"{next_code_indent(idx)}{MARKER}({text!r})"
    return "\n".join(lines)


def parse(source: str) -> ast.Module:
    """``ast.parse`` that keeps ``#pragma`` comments as marker statements."""
    return ast.parse(mark_pragmas(source))


def pragma_text(node) -> str | None:
    """The comment text if ``node`` is a pragma marker statement, else None."""
    if (
        isinstance(node, ast.Expr)
        and isinstance(node.value, ast.Call)
        and isinstance(node.value.func, ast.Name)
        and node.value.func.id == MARKER
        and len(node.value.args) == 1
        and isinstance(node.value.args[0], ast.Constant)
        and isinstance(node.value.args[0].value, str)
    ):
        return node.value.args[0].value
    return None


def make_pragma_stmt(text: str) -> ast.Expr:
    node = ast.Expr(
        value=ast.Call(func=ast.Name(id=MARKER, ctx=ast.Load()), args=[ast.Constant(value=text)], keywords=[])
    )
    return ast.fix_missing_locations(node)


def unparse(node) -> str:
    """``ast.unparse`` that turns marker statements back into comment lines."""
    if isinstance(node, list):
        text = "\n".join(ast.unparse(ast.fix_missing_locations(n)) for n in node)
    else:
        text = ast.unparse(ast.fix_missing_locations(node))
    out = []
    for line in text.split("\n"):
        m = _MARKER_LINE.match(line)
        if m:
            try:
                comment = ast.literal_eval(m.group(2))
            except (ValueError, SyntaxError):
                comment = None
            if isinstance(comment, str):
                out.append(m.group(1) + comment)
                continue
        out.append(line)
    return "\n".join(out)
