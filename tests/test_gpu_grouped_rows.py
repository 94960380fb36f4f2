"""Loops over short rows that sum terms gathered from an operand larger than an L2 (CSR SpMV with
a few to a hundred elements per row): the elements of every 256 rows are grouped by the stripe of the
operand they read, the groups run with one stripe per XCD, and the sums of a row are added up
afterwards.  The form of a launch follows from the sizes of its arrays; what the launch before it
reported about the rows only leaves out kernels that would run empty, and never changes a bit of the result.  Every result is compared with the float64 oracle to the bar
of the parity tests (``|out - oracle| <= 1e-5 * sum(|terms|)`` per output).

Pattern: the CSR loop of the reference's examples/03-spmv.py:5-16 and
tests/integration/triton/tutorial/test_spmv.py:10-30."""
import numpy as np
import pytest

import appy_amd as appy
from appy_amd.backends.hip import codegen as cg
from appy_amd.backends.hip import selfcheck
from oracle import vectorised as vo
from oracle import workloads as wl

pytestmark = pytest.mark.gpu

TOL = 1e-5


@pytest.fixture(scope="module")
def k(gpu):
    return selfcheck.kernels()


FULL = ["clear", "bins", "group", "cells", "sums", "plan", "parts", "fold", "rowwise"]


def _steps(launch):
    return [step[0].src.name.rsplit("_", 1)[-1] if step[0] else "clear" for step in (launch.sequence or [])]


def _loop(name, index_type="int32", reuse=True):
    hits = [v[0] for kk, v in cg.code_cache.items() if kk[-1] == name and v[0].options.get("hip_bins", True)
            and v[0].options.get("hip_group", True) and getattr(v[0], "last_launch", None) is not None
            and bool(v[0].options.get("hip_reuse", True)) == reuse
            and (name != "spmv" or ("A_indptr" in v[0].analysis.arrays and v[0].analysis.arrays["A_indptr"].ty.name == index_type
                                   and v[0].analysis.arrays["x"].ty.name == "float32"))]
    return max(hits, key=lambda lp: lp.last_launch.serial if getattr(lp, "last_launch", None) is not None else -1)


def _forget(name="spmv"):
    for kk, v in cg.code_cache.items():
        if kk[-1] == name:
            for _addr, view in v[0]._hints.values():
                view[0] = 0


def _grouped(launch):
    return launch.sequence is not None and launch.spec.aux == "cells"


@appy.jit
def windows(data, start, end, indices, x, y, beta, m):
    #pragma parallel for
    for i in range(m):
        s = 0.0
        #pragma simd
        for j in range(start[i], end[i]):
            s += data[j] * x[indices[j]]
        y[i] = beta * y[i] + s


def _matrix(lengths, n, seed):
    rng = np.random.default_rng(seed)
    data, indptr, indices = wl.csr_matrix(np.asarray(lengths, dtype=np.int64), n, rng)
    x = rng.standard_normal(n, dtype=np.float32)
    return data, indptr, indices, x


@pytest.mark.parametrize("m,n,lengths", [
    (50_000, 1 << 20, "16"),                 # the uniform matrix of the benchmark, scaled down
    (40_003, (1 << 22) - 12345, "1..31"),    # a ragged last block, a last stripe that is not full
    (70_000, 3 << 20, "0,10,20"),            # empty rows; stripes that are not a power of two of the operand
    (33_000, 7 << 20, "8"),                  # sixteen stripes, two per XCD
    (36_000, 1 << 21, "1..127"),             # rows of the three classes that qualify
])
def test_short_rows_are_grouped_and_earlier_launches_change_no_bit(k, m, n, lengths):
    rng = np.random.default_rng(m)
    if lengths == "0,10,20":
        ln = rng.integers(0, 3, m) * 10
    elif ".." in lengths:
        a, b = lengths.split("..")
        ln = rng.integers(int(a), int(b) + 1, m)
    else:
        ln = np.full(m, int(lengths))
    data, indptr, indices, x = _matrix(ln, n, seed=m + 1)
    ref, budget = vo.spmv_csr(data, indptr, indices, x, (m, n))
    _forget()
    y0 = k.spmv(data, indptr, indices, x, m, n)
    first = _loop("spmv").last_launch
    # nothing is believed about the rows yet: grouped, with the kernels for rows beyond the limit set up as well
    assert _grouped(first) and _steps(first) == FULL and first.nsplit == (16 if n > (8 << 19) else 8)
    ok, worst = vo.within_budget(y0, ref, budget, TOL)
    assert ok, worst
    y1 = k.spmv(data, indptr, indices, x, m, n)
    second = _loop("spmv").last_launch
    # the first launch found no row beyond the limit: the kernels that would run empty are left out
    assert _grouped(second) and _steps(second) == ["clear", "group", "cells", "sums", "rowwise"]
    assert np.all(y1[ln == 0] == 0.0)
    # the same bits from the first launch on: neither what earlier launches reported nor timing changes the order
    # in which the terms of a row are added
    assert np.array_equal(y0, y1)
    assert np.array_equal(y1, k.spmv(data, indptr, indices, x, m, n))


def test_matrices_with_long_rows_group_their_short_rows_and_cut_the_long_ones(k):
    """What a launch reported is believed only by a launch over the same arrays.  Rows of up to 512 elements have
    their elements grouped, longer rows run in parts cut at the stripes, in one launch, from the first launch on."""
    m, n = 40_000, 1 << 20
    short = _matrix(np.full(m, 12), n, seed=1)
    rng = np.random.default_rng(2)
    ln = np.clip(rng.zipf(1.5, m), 1, 4096)
    long_ = _matrix(ln, n, seed=3)
    _forget()
    k.spmv(*short, m, n)
    k.spmv(*short, m, n)
    launch = _loop("spmv").last_launch
    assert _grouped(launch) and len(launch.sequence) == 5
    ref, budget = vo.spmv_csr(*long_, (m, n))
    results = []
    for _ in range(3):
        y = k.spmv(*long_, m, n)
        launch = _loop("spmv").last_launch
        assert _grouped(launch) and _steps(launch) == FULL       # other arrays: the report on the short rows is not theirs
        cut = launch.bin["rowmax"]
        assert cut == 512 and (ln > cut).sum() > 100 and (ln <= cut).sum() > 100
        ok, worst = vo.within_budget(y, ref, budget, TOL)
        assert ok, worst
        results.append(y)
    assert np.array_equal(results[0], results[1]) and np.array_equal(results[1], results[2])
    # and back: the matrix of short rows after the one with long rows
    ref, budget = vo.spmv_csr(*short, (m, n))
    y = k.spmv(*short, m, n)
    assert len(_loop("spmv").last_launch.sequence) == 9
    ok, worst = vo.within_budget(y, ref, budget, TOL)
    assert ok, worst
    assert np.array_equal(y, k.spmv(*short, m, n)) and len(_loop("spmv").last_launch.sequence) == 5


def test_longest_rows_just_below_and_above_the_limit_settle_on_one_form(k):
    """One limit decides between grouped and cut rows in every form of the launch: a matrix whose longest rows
    hold 257..512 elements (or 513..600) takes the same form, with the same bits, from its second launch on."""
    m, n = 40_000, 1 << 20
    for longest, steps in ((300, 5), (512, 5), (600, 9)):
        rng = np.random.default_rng(longest)
        ln = rng.integers(1, 20, m)
        ln[::97] = longest
        data, indptr, indices, x = _matrix(ln, n, seed=longest + 1)
        ref, budget = vo.spmv_csr(data, indptr, indices, x, (m, n))
        _forget()
        seen, ys = [], []
        for _ in range(5):
            ys.append(k.spmv(data, indptr, indices, x, m, n))
            seen.append(len(_loop("spmv").last_launch.sequence))
            assert _grouped(_loop("spmv").last_launch)
        assert seen == [9, steps, steps, steps, steps], (longest, seen)
        assert all(np.array_equal(ys[0], y) for y in ys[1:]), longest
        ok, worst = vo.within_budget(ys[-1], ref, budget, TOL)
        assert ok, worst


def test_rows_of_every_length_around_the_cut(k):
    """Row lengths on both sides of the limit between grouped and cut rows, empty rows, blocks made of
    long rows only, and a last block that is not full."""
    rng = np.random.default_rng(14)
    m, n = 36_001, 1 << 21
    pool = np.array([0, 1, 3, 4, 5, 31, 128, 129, 511, 512, 513, 700, 2000, 4096], dtype=np.int64)
    ln = pool[rng.integers(0, len(pool), m)]
    ln[1024:1024 + 512] = 3000              # two whole blocks of long rows
    ln[4096:4096 + 256] = 0                 # an empty block
    data, indptr, indices, x = _matrix(ln, n, seed=15)
    ref, budget = vo.spmv_csr(data, indptr, indices, x, (m, n))
    _forget()
    tags, ys = [], []
    for _ in range(3):
        y = k.spmv(data, indptr, indices, x, m, n)
        launch = _loop("spmv").last_launch
        tags.append(len(launch.sequence) if _grouped(launch) else 0)
        ok, worst = vo.within_budget(y, ref, budget, TOL)
        assert ok, worst
        assert np.all(y[ln == 0] == 0.0)
        ys.append(y)
    assert tags == [9, 9, 9]
    assert np.array_equal(ys[0], ys[1]) and np.array_equal(ys[1], ys[2])


@pytest.mark.parametrize("with_long_rows", [False, True])
def test_blocks_whose_elements_end_on_step_boundaries(k, with_long_rows):
    """The grouping kernel walks a block's elements 1024 at a time, four per lane: blocks with exactly one or
    two steps' worth of elements, one more, one fewer, long rows first, last and in between (their elements
    are passed over, so four consecutive kept elements need not be consecutive in the arrays), single rows."""
    rng = np.random.default_rng(30 + with_long_rows)
    R = 256
    L = 1000 if with_long_rows else 100          # a row beyond the cut / a long row that is still grouped
    blocks = []

    def block(lengths):
        b = np.zeros(R, dtype=np.int64)
        b[:len(lengths)] = lengths
        blocks.append(b)

    block([4] * 256)                               # 1024
    block([4] * 255 + [3])                         # 1023
    block([4] * 255 + [5])                         # 1025
    block([8] * 256)                               # 2048
    block([L] + [4] * 255)                         # long row first
    block([4] * 255 + [L])                         # long row last
    block([L if r % 2 else 3 for r in range(256)])  # every other row long
    block([])                                      # nothing
    block([512 if with_long_rows else 256])        # one row, exactly at the cut / at the end of the third class
    block([513] if with_long_rows else [128])      # one row just beyond it
    block([1] * 256)                               # one element per row
    block([0, 0, 7, 0, L, 0, 2, 1, 0, 0, 3] * 23)  # gaps of empty rows around long ones
    block([L] * 256 if with_long_rows else [96] * 256)
    for _ in range(3):
        block(rng.integers(0, 9, 256))
    ln = np.concatenate([blocks[i] for i in rng.permutation(len(blocks) * 9) % len(blocks)])
    ln = np.concatenate([ln, rng.integers(1, 6, 77)])          # a last block that is not full
    m, n = len(ln), 1 << 20
    assert m >= cg.BIN_MIN_ROWS
    data, indptr, indices, x = _matrix(ln, n, seed=32)
    ref, budget = vo.spmv_csr(data, indptr, indices, x, (m, n))
    _forget()
    forms, ys = [], []
    for _ in range(3):
        y = k.spmv(data, indptr, indices, x, m, n)
        launch = _loop("spmv").last_launch
        forms.append(len(launch.sequence) if _grouped(launch) else 0)
        ok, worst = vo.within_budget(y, ref, budget, TOL)
        assert ok, (forms, worst)
        assert np.all(y[ln == 0] == 0.0)
        ys.append(y)
    assert forms == ([9, 9, 9] if with_long_rows else [9, 5, 5])
    assert np.array_equal(ys[0], ys[1]) and np.array_equal(ys[1], ys[2])


def test_row_ranges_that_do_not_follow_one_another_run_row_by_row(gpu):
    """`range(start[i], end[i])` need not describe a CSR matrix.  Ranges out of order, ranges that overlap
    and ranges with gaps are legal loops; the grouping kernel refuses them and the launch runs the loop
    as written - once: the statement after the loop updates `y` in place."""
    rng = np.random.default_rng(4)
    m, n, per = 40_000, 1 << 20, 16
    data, indptr, indices, x = _matrix(np.full(m, per), n, seed=5)

    def run(start, end, expect_grouped=True):
        y = np.ones(m, dtype=np.float32)
        windows(data, start, end, indices, x, y, 0.5, m)
        assert _grouped(_loop("windows").last_launch) == expect_grouped
        terms = data.astype(np.float64) * x.astype(np.float64)[indices]
        cs = np.concatenate([[0.0], np.cumsum(terms)])
        ca = np.concatenate([[0.0], np.cumsum(np.abs(terms))])
        ln = np.maximum(end.astype(np.int64) - start, 0)
        ref = 0.5 + cs[start + ln] - cs[start]
        budget = 0.5 + ca[start + ln] - ca[start]
        assert np.all(np.abs(y - ref) <= TOL * budget + 1e-9 * ca[-1]), np.max(np.abs(y - ref))

    start, end = indptr[:-1].copy(), indptr[1:].copy()
    _forget("windows")
    run(start, end)                             # a CSR matrix in two arrays: grouped, from the first launch on
    run(start, end)
    # two rows swapped: ranges out of order
    s2, e2 = start.copy(), end.copy()
    s2[[1000, 1001]] = s2[[1001, 1000]]
    e2[[1000, 1001]] = e2[[1001, 1000]]
    run(s2, e2)
    # a range that reaches into its neighbour's, a range that ends before its own start, a gap
    s3, e3 = start.copy(), end.copy()
    e3[5] += 7
    e3[20_000] = s3[20_000] - 3
    s3[30_000] += 2
    run(s3, e3)
    # a range that ends beyond the arrays' extent would be refused as well; within it, the last row may stop short
    e4 = end.copy()
    e4[-1] -= 5
    run(start, e4)


def test_refused_ranges_in_a_launch_that_also_cuts_long_rows(gpu):
    """Long and short rows, and ranges out of order: nothing of the launch but the row-by-row kernel may
    touch `y`, which the statement after the loop updates in place."""
    m, n = 40_000, 1 << 20
    rng = np.random.default_rng(16)
    ln = np.where(rng.random(m) < 0.02, rng.integers(600, 3000, m), rng.integers(1, 40, m))
    data, indptr, indices, x = _matrix(ln, n, seed=17)
    start, end = indptr[:-1].copy(), indptr[1:].copy()
    terms = data.astype(np.float64) * x.astype(np.float64)[indices]
    cs = np.concatenate([[0.0], np.cumsum(terms)])
    ca = np.concatenate([[0.0], np.cumsum(np.abs(terms))])

    def run(start, end, steps):
        y = np.ones(m, dtype=np.float32)
        windows(data, start, end, indices, x, y, 0.5, m)
        launch = _loop("windows").last_launch
        assert (len(launch.sequence) if _grouped(launch) else 0) == steps
        lens = np.maximum(end.astype(np.int64) - start, 0)
        ref = 0.5 + cs[start + lens] - cs[start]
        budget = 0.5 + ca[start + lens] - ca[start]
        assert np.all(np.abs(y - ref) <= TOL * budget + 1e-9 * ca[-1]), np.max(np.abs(y - ref))

    _forget("windows")
    run(start, end, 9)
    run(start, end, 9)
    long_row = int(np.flatnonzero(ln > 600)[5])
    s2, e2 = start.copy(), end.copy()
    s2[[long_row, 7]] = s2[[7, long_row]]
    e2[[long_row, 7]] = e2[[7, long_row]]
    run(s2, e2, 9)
    run(start, end, 9)


def test_terms_with_a_scalar_factor_integer_values_and_no_second_operand(gpu):
    rng = np.random.default_rng(6)
    m, n = 40_000, 1 << 20
    ln = rng.integers(4, 24, m)
    data, indptr, indices, x = _matrix(ln, n, seed=7)
    nnz = len(indices)
    w = rng.integers(-5, 6, nnz).astype(np.int32)
    xi = rng.integers(-100, 100, n).astype(np.int32)

    @appy.jit
    def scaled(data, indptr, indices, x, y, alpha, m):
        #pragma parallel for
        for i in range(m):
            s = 0.0
            #pragma simd
            for j in range(indptr[i], indptr[i + 1]):
                s += alpha * (data[j] * x[indices[j]])
            y[i] = s

    @appy.jit
    def weighted_counts(w, indptr, indices, x, y, m):
        #pragma parallel for
        for i in range(m):
            s = 0
            #pragma simd
            for j in range(indptr[i], indptr[i + 1]):
                s += w[j] * x[indices[j]]
            y[i] = s

    @appy.jit
    def gathered(indptr, indices, x, y, m):
        #pragma parallel for
        for i in range(m):
            s = 0.0
            #pragma simd
            for j in range(indptr[i], indptr[i + 1]):
                s += x[indices[j]]
            y[i] = s

    rows = np.repeat(np.arange(m), ln)
    x64 = x.astype(np.float64)
    cases = (
        ("scaled", lambda y: scaled(data, indptr, indices, x, y, 0.25, m), 0.25 * data * x64[indices], np.float32),
        ("weighted_counts", lambda y: weighted_counts(w, indptr, indices, xi, y, m), (w.astype(np.int64) * xi[indices]).astype(np.float64), np.int32),
        ("gathered", lambda y: gathered(indptr, indices, x, y, m), x64[indices], np.float32),
    )
    for name, call, terms, dtype in cases:
        ref = np.bincount(rows, weights=terms, minlength=m)
        budget = np.bincount(rows, weights=np.abs(terms), minlength=m)
        _forget(name)
        for launch_no in range(2):
            y = np.zeros(m, dtype=dtype)
            call(y)
            assert _grouped(_loop(name).last_launch), name
            if dtype is np.int32:
                assert np.array_equal(y, ref.astype(np.int64)), name
            else:
                assert np.all(np.abs(y - ref) <= TOL * budget), name


def test_loops_that_do_not_qualify_keep_their_rows_sorted(k):
    """Terms that read a value of their row, sums of float64, operands that fit an L2, and the option."""
    rng = np.random.default_rng(8)
    m, n = 40_000, 1 << 20
    data, indptr, indices, x = _matrix(np.full(m, 10), n, seed=9)
    scale = rng.standard_normal(m).astype(np.float32)

    @appy.jit
    def row_scaled(data, indptr, indices, x, scale, y, m):
        #pragma parallel for
        for i in range(m):
            f = scale[i]
            s = 0.0
            #pragma simd
            for j in range(indptr[i], indptr[i + 1]):
                s += f * data[j] * x[indices[j]]
            y[i] = s

    y = np.empty(m, dtype=np.float32)
    for _ in range(2):
        row_scaled(data, indptr, indices, x, scale, y, m)
        launch = _loop("row_scaled").last_launch
        assert launch.spec.rows == "mixed" and launch.loop.analysis.grouping is None
    ref, budget = vo.spmv_csr(data, indptr, indices, x, (m, n))
    assert np.all(np.abs(y - scale * ref) <= TOL * np.abs(scale) * budget)
    # float64 sums
    x64 = x.astype(np.float64)
    for _ in range(2):
        y64 = k.spmv(data.astype(np.float64), indptr, indices, x64, m, n)
        assert not _grouped([v[0] for kk, v in cg.code_cache.items() if kk[-1] == "spmv"
                             and "A_indptr" in v[0].analysis.arrays and v[0].analysis.arrays["x"].ty.name == "float64"][-1].last_launch)
    assert np.all(np.abs(y64 - ref) <= 1e-12 * budget)
    # an operand of 2 MiB stays in every L2 anyway
    small = _matrix(np.full(m, 10), 1 << 19, seed=10)
    _forget()
    for _ in range(2):
        k.spmv(*small, m, 1 << 19)
        assert _loop("spmv").last_launch.spec.rows == "mixed"
    # hip_group=False
    off = selfcheck.kernels(hip_group=False)
    for _ in range(2):
        y = off.spmv(data, indptr, indices, x, m, n)
    last = [v[0] for kk, v in cg.code_cache.items() if kk[-1] == "spmv" and not v[0].options.get("hip_group", True)
            and "A_indptr" in v[0].analysis.arrays and v[0].analysis.arrays["x"].ty.name == "float32"
            and v[0].analysis.arrays["A_indptr"].ty.name == "int32"][-1].last_launch
    assert last.spec.rows == "mixed"
    assert vo.within_budget(y, ref, budget, TOL)[0]


def test_grouped_launches_on_gpu_tensors_follow_changes_of_the_matrix(gpu):
    """With `hip_reuse=False` nothing about the matrix is kept between launches: the same tensors with other
    contents give the other matrix's product."""
    import torch

    k = selfcheck.kernels(hip_reuse=False)
    m, n = 60_000, 1 << 20
    a = _matrix(np.full(m, 16), n, seed=11)
    b = _matrix(np.full(m, 16), n, seed=13)
    d = [torch.from_numpy(v).cuda() for v in a]
    _forget()
    for _ in range(2):
        y = k.spmv(*d, m, n)
    assert _grouped(_loop("spmv", reuse=False).last_launch)
    ref, budget = vo.spmv_csr(*a, (m, n))
    assert vo.within_budget(y.cpu().numpy(), ref, budget, TOL)[0]
    for t, v in zip(d, b):
        t.copy_(torch.from_numpy(v))
    y = k.spmv(*d, m, n)
    assert _grouped(_loop("spmv", reuse=False).last_launch)
    ref, budget = vo.spmv_csr(*b, (m, n))
    ok, worst = vo.within_budget(y.cpu().numpy(), ref, budget, TOL)
    assert ok, worst


@pytest.mark.parametrize("lengths", ["16", "zipf"])
def test_column_indices_of_64_bits_are_narrowed_by_the_grouping_kernels(gpu, lengths):
    """Column indices (and row starts) of 64 bits: both walks of the grouping kernel - over the arrays as they lie and
    over the kept rows of a matrix with long rows - load them as pairs of 16-byte vectors and narrow them."""
    import torch

    k = selfcheck.kernels(hip_reuse=False)
    m, n = 60_000, 1 << 20
    rng = np.random.default_rng(31)
    ln = np.full(m, 16) if lengths == "16" else np.clip(rng.zipf(1.5, m), 1, 4096)
    data, indptr, indices, x = _matrix(ln, n, seed=33)
    d = [torch.from_numpy(v).cuda() for v in (data, indptr.astype(np.int64), indices.astype(np.int64), x)]
    ref, budget = vo.spmv_csr(data, indptr, indices, x, (m, n))
    _forget()
    ys = []
    for it in range(3):
        y = k.spmv(*d, m, n)
        launch = _loop("spmv", index_type="int64", reuse=False).last_launch
        assert _grouped(launch)
        assert (_steps(launch) == FULL) == (it == 0 or lengths == "zipf")
        ok, worst = vo.within_budget(y.cpu().numpy(), ref, budget, TOL)
        assert ok, worst
        ys.append(y)
    assert torch.equal(ys[0], ys[1]) and torch.equal(ys[1], ys[2])


def test_calls_with_the_same_tensors_repeat_the_staged_kernels_until_the_rows_change_class(gpu):
    """A call whose tensors and scalars are those of an earlier call repeats that call's kernels without staging them
    again, once the form has settled (it was chosen from what a launch over these arrays reported).  The kernels read
    the arrays themselves: other contents give the other product; rows that change class are reported by the kernels,
    and the next call is staged anew."""
    import torch

    k = selfcheck.kernels(hip_reuse=False)
    m, n = 60_000, 1 << 20
    a = _matrix(np.full(m, 16), n, seed=21)
    data, indptr, indices, x = a
    d = [torch.from_numpy(v).cuda() for v in a]
    y = torch.empty(m, device="cuda")

    @appy.jit(hip_reuse=False)
    def into(data, indptr, indices, x, y, m):
        #pragma parallel for
        for i in range(m):
            s = 0.0
            #pragma simd
            for j in range(indptr[i], indptr[i + 1]):
                s += data[j] * x[indices[j]]
            y[i] = s

    def staged_by(call):
        before = cg.Launch.serial
        call()
        return cg.Launch.serial - before

    call = lambda: into(*d, y, m)
    assert staged_by(call) == 1 and _steps(_loop("into", reuse=False).last_launch) == FULL      # nothing known yet
    assert staged_by(call) == 1 and _steps(_loop("into", reuse=False).last_launch) == ["clear", "group", "cells", "sums", "rowwise"]
    y.zero_()
    assert staged_by(call) == 0                                                                 # repeated as staged
    ref, budget = vo.spmv_csr(*a, (m, n))
    assert vo.within_budget(y.cpu().numpy(), ref, budget, TOL)[0]
    # other values and columns in the same tensors: the repeated kernels read them
    b = _matrix(np.full(m, 16), n, seed=23)
    for t, v in zip(d, b):
        t.copy_(torch.from_numpy(v))
    assert staged_by(call) == 0
    ref, budget = vo.spmv_csr(*b, (m, n))
    assert vo.within_budget(y.cpu().numpy(), ref, budget, TOL)[0]
    # rows beyond the limit appear (same sizes of the arrays): the kernels report them, the call after is staged in full
    ln = np.full(m, 16)
    ln[:100] = 16 + 2000
    ln[100:100 + 100 * 125] = 0
    assert ln.sum() == 16 * m
    c = _matrix(ln, n, seed=25)
    for t, v in zip(d, c):
        t.copy_(torch.from_numpy(v))
    ref, budget = vo.spmv_csr(*c, (m, n))
    assert staged_by(call) == 0                                                                 # still the short form: right, and reports
    assert vo.within_budget(y.cpu().numpy(), ref, budget, TOL)[0]
    torch.cuda.synchronize()
    assert staged_by(call) == 1 and _steps(_loop("into", reuse=False).last_launch) == FULL
    assert vo.within_budget(y.cpu().numpy(), ref, budget, TOL)[0]
    assert staged_by(call) == 1 and _steps(_loop("into", reuse=False).last_launch) == FULL      # long rows: the form with kernels for them
    assert staged_by(call) == 0
    assert vo.within_budget(y.cpu().numpy(), ref, budget, TOL)[0]
    appy.release()


@pytest.mark.parametrize("rows_per_block", [512, 1024])
def test_larger_blocks_of_rows(gpu, rows_per_block):
    """`hip_group_rows` sets the rows per block of the grouped form (256 unless told otherwise)."""
    kk = selfcheck.kernels(hip_group_rows=rows_per_block)
    rng = np.random.default_rng(40)
    m, n = 40_000 + rows_per_block // 2 + 3, 1 << 20
    ln = np.where(rng.random(m) < 0.01, rng.integers(600, 3000, m), rng.integers(0, 12, m))
    data, indptr, indices, x = _matrix(ln, n, seed=41)
    ref, budget = vo.spmv_csr(data, indptr, indices, x, (m, n))
    for launch_no in range(3):
        y = kk.spmv(data, indptr, indices, x, m, n)
        ok, worst = vo.within_budget(y, ref, budget, TOL)
        assert ok, (launch_no, worst)
    launch = max((v[0] for key, v in cg.code_cache.items() if key[-1] == "spmv" and v[0].options.get("hip_group_rows") == rows_per_block
                  and getattr(v[0], "last_launch", None) is not None), key=lambda lp: lp.last_launch.serial).last_launch
    assert _grouped(launch) and launch.spec.block_rows == rows_per_block and len(launch.sequence) == 9
    short = _matrix(np.full(m, 9), n, seed=42)
    ref, budget = vo.spmv_csr(*short, (m, n))
    for _ in range(3):
        y = kk.spmv(*short, m, n)
        assert vo.within_budget(y, ref, budget, TOL)[0]


def test_launches_recorded_into_a_graph_keep_their_rows_sorted(gpu):
    """The grouped form clears a flag with a memory-set node, and a kept order of the elements would be that of
    the values at the time of the recording; recorded launches use the kernels over sorted rows instead, and
    every replay follows the contents of the tensors."""
    import torch

    k = selfcheck.kernels()
    m, n = 50_000, 1 << 20
    a = _matrix(np.full(m, 16), n, seed=21)
    d = [torch.from_numpy(v).cuda() for v in a]
    y = torch.zeros(m, device="cuda", dtype=torch.float32)

    @appy.jit
    def spmv_into(A_data, A_indptr, A_indices, x, y, M):
        #pragma parallel for
        for i in range(M):
            s = 0.0
            #pragma simd
            for j in range(A_indptr[i], A_indptr[i + 1]):
                s += A_data[j] * x[A_indices[j]]
            y[i] = s

    _forget("spmv_into")
    spmv_into(*d, y, m)
    assert _grouped(_loop("spmv_into").last_launch)
    spmv_into(*d, y, m)
    assert _loop("spmv_into").last_launch.plan is not None      # GPU tensors seen twice: their order is kept
    with appy.graph() as g:
        spmv_into(*d, y, m)
    assert _loop("spmv_into").last_launch.spec.rows == "mixed"
    for replay in range(3):
        d[0].mul_(1.5)
        y.zero_()
        spmv_into(*d, torch.empty_like(y), m)             # eager launches between the replays
        g.launch()
        g.synchronize()
        ref, budget = vo.spmv_csr(d[0].cpu().numpy(), a[1], a[2], a[3], (m, n))
        ok, worst = vo.within_budget(y.cpu().numpy(), ref, budget, TOL)
        assert ok, (replay, worst)
    g.close()
