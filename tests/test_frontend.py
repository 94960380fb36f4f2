"""Decoration-time rewrite and per-loop IR.

Expected forms are the worked rewrites of the reference's passes
(appy/frontend/process_shared.py:59-74, replace_pfor_with_stub.py:4-13,
hoist_shape_attr.py:19-48, reduction_detection.py:1-9)."""
import ast

import numpy as np
import pytest

import appy_amd as appy
from appy_amd.frontend import loop_ir, names, source, static_rewrite


def rewrite(src, **options):
    appy.set_default_options(options)
    tree, loops = static_rewrite.transform(source.parse(src), options)
    return ast.unparse(tree), loops


VEC_SUM = '''
@appy.jit
def vector_sum(A):
    s = 0.0
    #pragma parallel for simd shared(s)
    for i in range(A.shape[0]):
        s += A[i]
    return s
'''


def test_shared_rewrite_and_stub():
    text, loops = rewrite(VEC_SUM)
    lines = [l.strip() for l in text.splitlines()]
    assert lines[0] == "def vector_sum(A):"            # decorator removed
    assert "A_shape_0 = A.shape[0]" in lines
    assert "s = numpy.array([s])" in lines
    assert "s = s.item()" in lines
    assert lines.index("s = numpy.array([s])") < lines.index("s = s.item()")
    assert loops == [("kernel_loop_1",
                      "#pragma parallel for simd shared(s)\nfor i in range(A_shape_0):\n    s[0] += A[i]")]
    assert "appy._kernel_launch(" in text and "locals(), globals()" in text


def test_inner_pragmas_stay_in_the_loop_text_and_numbering():
    src = '''
def f(A, x, y, z):
    #pragma parallel for
    for i in range(A.shape[0]):
        yi = 0.0
        #pragma simd
        for j in range(A.shape[1]):
            yi += A[i, j] * x[j]
        y[i] = yi
    #pragma parallel for simd

    for i in range(z.shape[0]):
        z[i] = 0
'''
    text, loops = rewrite(src)
    assert [n for n, _ in loops] == ["kernel_loop_1", "kernel_loop_2"]
    assert "#pragma simd" in loops[0][1]
    assert loops[0][1].startswith("#pragma parallel for\nfor i in range(A_shape_0):")
    assert "A_shape_1" in loops[0][1]
    assert loops[1][1].startswith("#pragma parallel for simd\n")   # blank line after the pragma is fine
    assert "__appy_pragma__" not in text


def test_options_are_embedded_as_literals():
    text, _ = rewrite(VEC_SUM, dump_code=True)
    assert "'dump_code': True" in text and "'backend': None" in text


def test_function_without_pragma_is_unchanged_in_behaviour():
    @appy.jit
    def passthrough(x):
        return x

    @appy.jit
    def bump(x):
        for i in range(x.shape[0]):
            x[i] += 1
        return x

    @appy.jit
    def total(x):
        s = 0
        for i in range(x.shape[0]):
            s += x[i]
        return s

    assert passthrough([1, 2, 3]) == [1, 2, 3]
    assert all(bump(np.zeros(10)) == np.ones(10))
    assert total(np.arange(10)) == 45


def test_prange_loop_is_outlined():
    src = '''
def f(a):
    for i in appy.prange(a.shape[0]):
        a[i] = 1
'''
    _, loops = rewrite(src)
    assert loops == [("kernel_loop_1", "#pragma parallel for\nfor i in range(a_shape_0):\n    a[i] = 1")]

    @appy.jit(dry_run=True)
    def fill(a):
        for i in appy.prange(a.shape[0]):
            a[i] = 1
        return a

    assert all(fill(np.zeros(5)) == 1)


# ---- per-loop IR ---------------------------------------------------------------
def test_ir_vec_add():
    tree = loop_ir.build("#pragma parallel for simd\nfor i in range(a_shape_0):\n    c[i] = a[i] + b[i]")
    loop = loop_ir.outer_loop(tree)
    assert dict(loop.pragma) == {"parallel_for": True, "simd": True}
    assert ast.unparse(loop.iter) == "range(0, a_shape_0, 1)"
    assert "reduction" not in loop.pragma


def test_ir_shared_sum_is_a_reduction():
    tree = loop_ir.build("#pragma parallel for simd shared(b)\nfor i in range(n):\n    b[0] += a[i]")
    loop = loop_ir.outer_loop(tree)
    assert loop.pragma["reduction"] == "+:b[0]"
    assert loop.body[0].reduce == "+"
    assert ast.unparse(loop.body[0]) == "b[0] = b[0] + a[i]"
    assert loop_ir.reductions_of(loop) == {"b[0]": "+"}


def test_ir_max_min_and_product():
    for fn in ("max", "min"):
        tree = loop_ir.build(f"#pragma parallel for simd shared(m)\nfor i in range(n):\n    m[0] = {fn}(m[0], a[i])")
        assert loop_ir.outer_loop(tree).pragma["reduction"] == f"{fn}:m[0]"
    tree = loop_ir.build("#pragma parallel for simd shared(p)\nfor i in range(n):\n    p[0] = a[i] * p[0]")
    assert loop_ir.outer_loop(tree).pragma["reduction"] == "*:p[0]"


def test_ir_gemv_inner_reduction_only():
    tree = loop_ir.build(
        "#pragma parallel for\nfor i in range(A_shape_0):\n    yi = 0.0\n    #pragma simd\n"
        "    for j in range(A_shape_1):\n        yi += A[i, j] * x[j]\n    y[i] = yi")
    outer = loop_ir.outer_loop(tree)
    inner = outer.body[1]
    assert "reduction" not in outer.pragma          # yi has both a plain and a '+' assignment out here
    assert dict(inner.pragma) == {"simd": True, "reduction": "+:yi"}


def test_ir_tuple_assignment_split():
    tree = loop_ir.build("#pragma parallel for\nfor i in range(M):\n    start, end = p[i], p[i + 1]\n    y[i] = end - start")
    body = loop_ir.outer_loop(tree).body
    assert [ast.unparse(s) for s in body[:2]] == ["start = p[i]", "end = p[i + 1]"]


def test_ir_pragma_is_consumed_by_an_assignment():
    # '#pragma simd' above 's = 0.0' annotates the assignment; the loop after it stays sequential
    tree = loop_ir.build(
        "#pragma parallel for\nfor i in range(n):\n    #pragma simd\n    s = 0.0\n"
        "    for j in range(m):\n        s += a[i, j]\n    b[i] = s")
    outer = loop_ir.outer_loop(tree)
    assert hasattr(outer.body[0], "pragma") and not hasattr(outer.body[1], "pragma")


def test_ir_step_must_be_one():
    with pytest.raises(Exception) as e:
        loop_ir.build("#pragma parallel for simd\nfor i in range(0, n, 2):\n    c[i] = a[i]")
    assert "range" in str(e.value) and "step" in str(e.value)


def test_ir_structure_checks():
    with pytest.raises(AssertionError):
        loop_ir.build("for i in range(n):\n    c[i] = a[i]")
    with pytest.raises(Exception) as e:
        loop_ir.build("#pragma parallel for\nfor i in range(n):\n    c[i] = 0\nfor j in range(n):\n    c[j] = 1")
    assert "single for loop" in str(e.value)


def test_used_names_order_and_callees():
    text = "#pragma parallel for\nfor i in range(M):\n    s = max(A[i], x[idx[i]])\n    y[i] = np.sqrt(s)"
    assert names.used_names(text) == ("i", "M", "s", "A", "x", "idx", "y", "np")


def test_prange_loops_share_the_scalars_they_reduce():
    from appy_amd.frontend.static_rewrite import prange_reductions

    src = '''
def f(a, N):
    total = 0
    big = -1.0
    for i in prange(N):
        t = a[i] * 2
        total += t
        big = max(big, a[i])
    return total, big
'''
    new, loops = rewrite(src)
    assert loops[0][1].startswith("#pragma parallel for shared(total, big)\nfor i in range(N):")
    assert "total[0] += t" in loops[0][1] and "big[0] = max(big[0], a[i])" in loops[0][1]
    assert "total = numpy.array([total], dtype=numpy.float64)" in new
    assert "total = appy._reduction_result(total, __appy_start_total)" in new
    loop = ast.parse("for i in prange(n):\n    s += 1\n    t = 0\n    t += 2\n    u = u * a[i]\n    v += 1\n    v -= 1").body[0]
    assert prange_reductions(loop) == ["s", "u"]

    @appy.jit(dry_run=True)
    def sum_vector(a, N):
        sum = 0
        for i in appy.prange(N):
            sum += a[i]
        return sum

    r = sum_vector(np.ones(10), 10)
    assert r == 10 and type(r) is int                  # the documented example: "sum is now 10"
    r = sum_vector(np.full(4, 0.25), 3)
    assert r == 0.75 and type(r) is float


def test_keyword_spellings_of_parallel_and_simd_loops():
    src = '''
def f(A, x, y):
    for i in appy.range(A.shape[0], parallel=True):
        s = 0.0
        for j in appy.range(A.shape[1], simd=True):
            s += A[i, j] * x[j]
        y[i] = s
'''
    _, loops = rewrite(src)
    assert loops[0][1] == ("#pragma parallel for\nfor i in range(A_shape_0):\n    s = 0.0\n    #pragma simd\n"
                           "    for j in range(A_shape_1):\n        s += A[i, j] * x[j]\n    y[i] = s")
    tree = loop_ir.build(loops[0][1])
    inner = [n for n in ast.walk(tree) if isinstance(n, ast.For)][1]
    assert "simd" in inner.pragma and inner.pragma["reduction"] == "+:s"

    @appy.jit(dry_run=True)
    def rowdot_kw(A, x, y):
        for i in appy.range(A.shape[0], parallel=True):
            s = 0.0
            for j in appy.range(A.shape[1], simd=True):
                s += A[i, j] * x[j]
            y[i] = s
        return y

    A = np.arange(12.0).reshape(3, 4)
    assert np.allclose(rowdot_kw(A, np.ones(4), np.zeros(3)), A.sum(axis=1))
    _, loops = rewrite("def g(a):\n    for i in range(a.shape[0], parallel=True, simd=True):\n        a[i] = 0\n")
    assert loops[0][1].startswith("#pragma parallel for simd\nfor i in range(a_shape_0):")


def test_prange_loops_get_their_vectorisable_inner_loops_marked():
    def loop_text(body_src):
        return rewrite(body_src)[1][0][1]

    gemv = loop_text('''
def f(A, x, y, alpha):
    for i in prange(A.shape[0]):
        for j in range(A.shape[1]):
            y[i] += alpha * A[i, j] * x[j]
''')
    assert gemv == ("#pragma parallel for\nfor i in range(A_shape_0):\n    __appy_acc1 = 0\n    #pragma simd\n"
                    "    for j in range(A_shape_1):\n        __appy_acc1 += alpha * A[i, j] * x[j]\n    y[i] += __appy_acc1")
    spmv = loop_text('''
def f(data, indptr, indices, x, y):
    for i in prange(y.shape[0]):
        s = 0.0
        for j in range(indptr[i], indptr[i + 1]):
            s += data[j] * x[indices[j]]
        y[i] = s
''')
    assert "#pragma simd\n    for j in range(indptr[i], indptr[i + 1]):" in spmv
    spmm = loop_text('''
def f(data, indptr, indices, B, C):
    for i in prange(C.shape[0]):
        for k in range(indptr[i], indptr[i + 1]):
            for c in range(C.shape[1]):
                C[i, c] += data[k] * B[indices[k], c]
''')
    assert "    for k in range(indptr[i], indptr[i + 1]):\n        #pragma simd\n        for c in range(C_shape_1):" in spmm
    not_marked = [
        # lanes walking j would stride through A
        "def f(A, y):\n    for i in prange(A.shape[1]):\n        s = 0.0\n        for j in range(A.shape[0]):\n            s += A[j, i]\n        y[i] = s\n",
        # iteration j reads what iteration j - 1 wrote
        "def f(A):\n    for i in prange(A.shape[0]):\n        for j in range(1, A.shape[1]):\n            A[i, j] = A[i, j - 1] + 1\n",
        # a scalar carried from one iteration to the next that is not a reduction
        "def f(A, y):\n    for i in prange(A.shape[0]):\n        t = 0.0\n        for j in range(A.shape[1]):\n            t = t * 0.5 + A[i, j]\n        y[i] = t\n",
        # the last value of a temporary is used after the loop
        "def f(A, y):\n    for i in prange(A.shape[0]):\n        for j in range(A.shape[1]):\n            t = A[i, j]\n            A[i, j] = t * 2\n        y[i] = t\n",
        # the accumulated element is read inside the loop
        "def f(A, y, z):\n    for i in prange(A.shape[0]):\n        for j in range(A.shape[1]):\n            y[i] += A[i, j]\n            z[i, j] = y[i]\n",
        # scatter through an index array
        "def f(A, p, out):\n    for i in prange(A.shape[0]):\n        for j in range(A.shape[1]):\n            out[i, p[j]] = A[i, j]\n",
    ]
    for text in not_marked:
        assert "#pragma simd" not in loop_text(text), text
    # under `#pragma parallel for` the same happens as long as no inner loop carries an annotation of its own
    # (the reference's guide: vectorisable patterns are found "even if simd is not specified", docs/source/legacy.rst:6)
    marked = loop_text("def f(A, y):\n    #pragma parallel for\n    for i in range(A.shape[0]):\n        for j in range(A.shape[1]):\n            A[i, j] = 0\n")
    assert "#pragma simd\n    for j in range(A_shape_1)" in marked
    kept = loop_text("def f(A, y):\n    #pragma parallel for\n    for i in range(A.shape[0]):\n        for j in range(A.shape[1]):\n            A[i, j] = 0\n"
                     "        #pragma simd\n        for j in range(A.shape[1]):\n            y[i] = A[i, j]\n")
    assert kept.count("#pragma simd") == 1


def test_ir_simd_loops_accumulating_into_one_element_use_a_scalar():
    """`y[i] += ...` under an inner simd loop carries a dependence through memory; the
    element is accumulated in a scalar around the loop (the reference's detection only knows
    names and literal subscripts, appy/frontend/reduction_detection.py:12-13)."""
    tree = loop_ir.build(
        "#pragma parallel for\nfor i in range(n):\n    y[i] = 0.0\n    #pragma simd\n"
        "    for j in range(m):\n        y[i] += A[i, j] * x[j]\n        z[i] = max(z[i], A[i, j])\n        w[i] -= x[j]")
    body = loop_ir.outer_loop(tree).body
    text = [ast.unparse(s) for s in body]
    # (the literal stored just before the loop is where the first accumulator starts)
    assert text[:4] == ["y[i] = 0.0", "__appy_e1 = 0.0", "__appy_e2 = z[i]", "__appy_e3 = w[i]"]
    assert text[5:] == ["y[i] = __appy_e1", "z[i] = __appy_e2", "w[i] = __appy_e3"]
    inner = body[4]
    assert [ast.unparse(s) for s in inner.body] == [
        "__appy_e1 = __appy_e1 + A[i, j] * x[j]", "__appy_e2 = max(__appy_e2, A[i, j])", "__appy_e3 = __appy_e3 + -x[j]"]
    assert inner.pragma["reduction"] == "+:__appy_e1,max:__appy_e2,+:__appy_e3"
    # an element that depends on the loop variable, or an array the loop also reads elsewhere, is left alone
    tree = loop_ir.build(
        "#pragma parallel for\nfor i in range(n):\n    #pragma simd\n    for j in range(m):\n"
        "        y[j] += A[i, j]\n        v[i] += v[j]")
    inner = loop_ir.outer_loop(tree).body[0]
    assert [ast.unparse(s) for s in inner.body] == ["y[j] = y[j] + A[i, j]", "v[i] = v[i] + v[j]"]


def test_ir_running_difference_is_a_sum_reduction():
    tree = loop_ir.build(
        "#pragma parallel for\nfor i in range(n):\n    s = 0.0\n    #pragma simd\n"
        "    for j in range(m):\n        s -= A[i, j]\n    y[i] = s")
    inner = loop_ir.outer_loop(tree).body[1]
    assert ast.unparse(inner.body[0]) == "s = s + -A[i, j]" and inner.pragma["reduction"] == "+:s"


def test_decorated_functions_keep_their_closure():
    """Free variables of the decorated function stay bound to the enclosing scope's cells
    (late binding included); the reference executes the rewritten source at module level,
    where such names are lost (appy/__init__.py:60-64)."""
    def make(k):
        @appy.jit(dry_run=True)
        def f(a, out, beta=1.0):
            """doc"""
            #pragma parallel for simd
            for i in range(a.shape[0]):
                out[i] = k * a[i] + beta
        return f

    a, out = np.arange(10.0), np.zeros(10)
    f = make(2.5)
    f(a, out)
    assert np.array_equal(out, 2.5 * a + 1.0)
    f(a, out, beta=2.0)
    assert np.array_equal(out, 2.5 * a + 2.0) and f.__name__ == "f"


def test_ir_parallel_for_on_an_inner_loop_counts_as_simd():
    tree = loop_ir.build(
        "#pragma parallel for\nfor i in range(n):\n    #pragma parallel for\n    for j in range(m):\n        B[i, j] = A[i, j] + 1")
    outer = loop_ir.outer_loop(tree)
    assert dict(outer.pragma) == {"parallel_for": True} and dict(outer.body[0].pragma) == {"simd": True}
