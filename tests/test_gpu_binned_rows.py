"""Loops whose rows differ widely in length (CSR rows): the rows are sorted into classes by the
trip count of their simd loop before they run, and long rows that gather from a large operand are
walked one stripe of that operand at a time.  Every result is compared with the float64 oracle
to the bar of the parity tests (``|out - oracle| <= 1e-5 * sum(|terms|)`` per output), and with the
same loop run without binning.

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


@pytest.fixture(scope="module")
def plain(gpu):
    return selfcheck.kernels(hip_bins=False)


@pytest.fixture(scope="module")
def sorted_only(gpu):
    """Rows sorted by length, but never the form that groups the elements of short rows by stripe."""
    return selfcheck.kernels(hip_group=False)


def _loop(name, bins=True, index_type="int32", group=True):
    """The compiled loop of function ``name`` (for `spmv`: the one for row pointers of ``index_type``)."""
    hits = [v[0] for kk, v in cg.code_cache.items() if kk[-1] == name and bool(v[0].options.get("hip_bins", True)) == bins
            and bool(v[0].options.get("hip_group", True)) == group
            and (name != "spmv" or ("A_indptr" in v[0].analysis.arrays and v[0].analysis.arrays["A_indptr"].ty.name == index_type
                                   and v[0].analysis.arrays["x"].ty.name == "float32"))]
    return max(hits, key=lambda lp: lp.last_launch.serial if getattr(lp, "last_launch", None) is not None else -1)


def _forget(name="spmv"):
    """Drop what earlier launches of the loop have reported about their rows (the hint that shapes
    the next launch), so that a test sees the launch of a loop that knows nothing yet."""
    for kk, v in cg.code_cache.items():
        if kk[-1] == name:
            for _addr, view in v[0]._hints.values():
                view[0] = 0


def _powerlaw(m, n, clip, seed, exponent=1.5):
    rng = np.random.default_rng(seed)
    lengths = np.clip(rng.zipf(exponent, m), 1, clip).astype(np.int64)
    data, indptr, indices = wl.csr_matrix(lengths, n, rng)
    x = rng.standard_normal(n, dtype=np.float32)
    return data, indptr, indices, x, lengths


@pytest.mark.parametrize("m,n,clip", [(40_000, 1 << 20, 4096), (33_000, 5_000_000, 3000), (100_000, 1 << 19, 700)])
def test_spmv_powerlaw_rows_are_binned_and_striped(sorted_only, plain, m, n, clip):
    k = sorted_only
    data, indptr, indices, x, lengths = _powerlaw(m, n, clip, seed=m)
    ref, budget = vo.spmv_csr(data, indptr, indices, x, (m, n))
    _forget()
    y = k.spmv(data, indptr, indices, x, m, n)
    launch = _loop("spmv", group=False).last_launch
    assert launch.spec.rows == "mixed" and launch.sequence is not None
    striped = 4 * n > cg.STRIPE_MIN_BYTES
    assert len(launch.sequence) == (6 if striped else 3)
    if striped:
        assert launch.nsplit % 8 == 0 and launch.nsplit * cg.STRIPE_BYTES >= 4 * n
    ok, worst = vo.within_budget(y, ref, budget, TOL)
    assert ok, worst
    y0 = plain.spmv(data, indptr, indices, x, m, n)
    ok, worst = vo.within_budget(y0, ref, budget, TOL)
    assert ok, worst
    # rows that are not cut into parts are summed in the same order either way
    short = lengths <= 4
    assert np.array_equal(y[short], y0[short])


def test_spmv_uniform_rows_stay_in_their_natural_order(sorted_only, plain):
    k = sorted_only
    m = 50_000
    data, indptr, indices, x = wl.spmv_uniform(m, 1 << 20, 16)
    ref, budget = vo.spmv_csr(data, indptr, indices, x, (m, 1 << 20))
    _forget()
    y = k.spmv(data, indptr, indices, x, m, 1 << 20)
    launch = _loop("spmv", group=False).last_launch
    assert launch.spec.rows == "mixed" and launch.bin["base"] == 1      # 16 per row: the class of teams of four
    assert len(launch.sequence) == 6                                    # nothing known yet: set up for long rows too
    # the launch has reported what its classes held: the next one sets nothing up for long rows
    y2 = k.spmv(data, indptr, indices, x, m, 1 << 20)
    again = _loop("spmv", group=False).last_launch
    assert len(again.sequence) == 3 and again.bin["base"] == 1 and np.array_equal(y, y2)
    assert vo.within_budget(y, ref, budget, TOL)[0]
    assert np.array_equal(y, plain.spmv(data, indptr, indices, x, m, 1 << 20))


def test_spmv_rows_of_every_class_and_empty_rows(k):
    """Row lengths that sit on both sides of every class boundary, empty rows, and one class missing."""
    rng = np.random.default_rng(5)
    m, n = 36_000, 1 << 20
    pool = np.array([0, 1, 3, 4, 5, 31, 32, 33, 127, 128, 129, 500, 2000, 4096], dtype=np.int64)
    lengths = pool[rng.integers(0, len(pool), m)]
    data, indptr, indices = wl.csr_matrix(lengths, n, rng)
    x = rng.standard_normal(n, dtype=np.float32)
    ref, budget = vo.spmv_csr(data, indptr, indices, x, (m, n))
    y = k.spmv(data, indptr, indices, x, m, n)
    ok, worst = vo.within_budget(y, ref, budget, TOL)
    assert ok, worst
    assert np.all(y[lengths == 0] == 0.0)
    # no row of the longest class at all
    lengths = np.minimum(lengths, 100)
    data, indptr, indices = wl.csr_matrix(lengths, n, rng)
    ref, budget = vo.spmv_csr(data, indptr, indices, x, (m, n))
    assert vo.within_budget(k.spmv(data, indptr, indices, x, m, n), ref, budget, TOL)[0]


def test_spmv_all_rows_long(k):
    rng = np.random.default_rng(6)
    m, n = 33_000, 1 << 21
    lengths = rng.integers(900, 1400, m)
    data, indptr, indices = wl.csr_matrix(lengths, n, rng)
    x = rng.standard_normal(n, dtype=np.float32)
    ref, budget = vo.spmv_csr(data, indptr, indices, x, (m, n))
    y = k.spmv(data, indptr, indices, x, m, n)
    ok, worst = vo.within_budget(y, ref, budget, TOL)
    assert ok, worst


def test_spmv_columns_in_any_order_and_int64_indices(k):
    """The cuts of a long row follow its column order when the columns are sorted; any other order
    still has every element in exactly one part."""
    data, indptr, indices, x, lengths = _powerlaw(40_000, 1 << 20, 4096, seed=9)
    rng = np.random.default_rng(10)
    shuffled = indices.copy()
    vals = data.copy()
    for r in np.flatnonzero(lengths > 100)[:400]:
        s, e = indptr[r], indptr[r + 1]
        p = rng.permutation(e - s)
        shuffled[s:e] = indices[s:e][p]
        vals[s:e] = data[s:e][p]
    ref, budget = vo.spmv_csr(vals, indptr, shuffled, x, (40_000, 1 << 20))
    y = k.spmv(vals, indptr.astype(np.int64), shuffled.astype(np.int64), x, 40_000, 1 << 20)
    ok, worst = vo.within_budget(y, ref, budget, TOL)
    assert ok, worst


def test_the_hint_of_an_earlier_launch_shapes_the_next_one_and_never_its_results(sorted_only):
    """The kernel over the binned rows reports the sizes of its classes in page-locked memory.  The next
    launch over the same arrays takes the most populous class in natural order and leaves out the kernels
    for long rows when there were none; a launch over other arrays believes nothing of it.  The bits of the
    result are the same either way."""
    k = sorted_only
    m, n = 40_000, 1 << 20
    short = wl.spmv_uniform(m, n, 3)                        # every row in the class of single lanes
    data, indptr, indices, x, lengths = _powerlaw(m, n, 4096, seed=77)
    _forget()
    y = k.spmv(*short, m, n)
    first = _loop("spmv", group=False).last_launch
    assert first.bin["base"] == 0 and len(first.sequence) == 6
    ref, budget = vo.spmv_csr(*short, (m, n))
    assert vo.within_budget(y, ref, budget, TOL)[0]
    y_again = k.spmv(*short, m, n)
    again = _loop("spmv", group=False).last_launch
    assert len(again.sequence) == 3 and again.bin["skip"] == 0 and np.array_equal(y, y_again)
    ref, budget = vo.spmv_csr(data, indptr, indices, x, (m, n))
    y1 = k.spmv(data, indptr, indices, x, m, n)             # other arrays: set up for long rows whatever was reported
    second = _loop("spmv", group=False).last_launch
    assert len(second.sequence) == 6
    ok, worst = vo.within_budget(y1, ref, budget, TOL)
    assert ok, worst
    y2 = k.spmv(data, indptr, indices, x, m, n)             # now it is known which class holds most rows
    third = _loop("spmv", group=False).last_launch
    assert len(third.sequence) == 6 and third.bin["base"] == int(np.argmax(np.bincount(np.digitize(lengths, [4, 32, 256], right=True), minlength=4)))
    assert np.array_equal(y1, y2)


def test_spmv_columns_crowded_into_one_stripe(k):
    """Every long row has its columns in the first eighth of the vector: the parts of the other seven
    stripes are empty, and the parts are dealt to all workgroups instead of one XCD per stripe."""
    rng = np.random.default_rng(31)
    m, n = 40_000, 1 << 21
    lengths = np.clip(rng.zipf(1.4, m), 1, 3000).astype(np.int64)
    data, indptr, indices = wl.csr_matrix(lengths, n // 8, rng)          # columns below n / 8 only
    x = rng.standard_normal(n, dtype=np.float32)
    ref, budget = vo.spmv_csr(data, indptr, indices, x, (m, n))
    _forget()
    y = k.spmv(data, indptr, indices, x, m, n)
    assert _loop("spmv").last_launch.nsplit == 8
    ok, worst = vo.within_budget(y, ref, budget, TOL)
    assert ok, worst
    # and columns in the last two stripes only
    indices2 = (indices.astype(np.int64) * 2 + (n - n // 4)).astype(np.int32)
    ref, budget = vo.spmv_csr(data, indptr, indices2, x, (m, n))
    ok, worst = vo.within_budget(k.spmv(data, indptr, indices2, x, m, n), ref, budget, TOL)
    assert ok, worst


def test_more_long_rows_than_the_streamed_arrays_account_for(k):
    """Row pointers that overlap (not a CSR matrix, but a legal loop): more rows of the longest class
    than nnz / threshold.  The rows beyond the room set aside for parts run whole."""
    rng = np.random.default_rng(12)
    m, n, nnz = 40_000, 1 << 20, 200_000
    start = rng.integers(0, nnz - 3000, m).astype(np.int32)
    length = rng.integers(0, 3000, m).astype(np.int32)
    data = rng.standard_normal(nnz, dtype=np.float32)
    indices = np.sort(rng.integers(0, n, nnz)).astype(np.int32)
    x = rng.standard_normal(n, dtype=np.float32)

    @appy.jit(hip_group=False)
    def windows(data, start, length, indices, x, y, m):
        #pragma parallel for
        for i in range(m):
            a = start[i]
            b = a + length[i]
            s = 0.0
            #pragma simd
            for j in range(a, b):
                s += data[j] * x[indices[j]]
            y[i] = s

    y = np.empty(m, dtype=np.float32)
    windows(data, start, length, indices, x, y, m)
    launch = _loop("windows", group=False).last_launch
    assert len(launch.sequence) == 6
    assert launch.sequence is not None and launch.bin["cap"] < int((length > launch.bin["threshold"][2]).sum())
    terms = data.astype(np.float64) * x.astype(np.float64)[indices]
    cs = np.concatenate([[0.0], np.cumsum(terms)])
    ca = np.concatenate([[0.0], np.cumsum(np.abs(terms))])
    ref = cs[start + length] - cs[start]
    budget = ca[start + length] - ca[start]
    # the prefix sums of the check cancel: allow for their own rounding
    assert np.all(np.abs(y - ref) <= TOL * budget + 1e-9 * ca[-1])


def test_ragged_rows_without_a_gather_and_with_statements_after_the_loop(k):
    """Row sums and row maxima of CSR values (no gathered operand: no parts), float64 values, and a
    body that goes on after the loop."""
    rng = np.random.default_rng(13)
    m = 60_000
    lengths = np.clip(rng.zipf(1.6, m), 0, 3000).astype(np.int64)
    lengths[::7] = 0
    indptr = np.zeros(m + 1, dtype=np.int64)
    np.cumsum(lengths, out=indptr[1:])
    vals = rng.standard_normal(int(indptr[-1]))

    @appy.jit
    def row_stats(vals, indptr, total, top, scale, m):
        #pragma parallel for
        for i in range(m):
            s = 0.0
            t = -1e300
            #pragma simd
            for j in range(indptr[i], indptr[i + 1]):
                s += vals[j]
                t = max(t, vals[j])
            total[i] = scale * s + total[i]
            top[i] = t

    total = np.ones(m)
    top = np.empty(m)
    row_stats(vals, indptr, total, top, 0.5, m)
    launch = _loop("row_stats").last_launch
    assert launch.sequence is not None and len(launch.sequence) == 3
    ref = np.ones(m)
    ref_top = np.full(m, -1e300)
    nz = lengths > 0
    ref[nz] += 0.5 * np.add.reduceat(vals, indptr[:-1][nz])
    ref_top[nz] = np.maximum.reduceat(vals, indptr[:-1][nz])
    budget = np.ones(m)
    budget[nz] += 0.5 * np.add.reduceat(np.abs(vals), indptr[:-1][nz])
    assert np.all(np.abs(total - ref) <= 1e-12 * budget)
    assert np.array_equal(top, ref_top)


def test_binned_launches_on_gpu_tensors_and_repeated_calls(gpu):
    """GPU tensors stay in place; a second call on a changed matrix of the same shape sorts its rows
    afresh (nothing about the rows is kept between calls)."""
    import torch

    k = selfcheck.kernels()
    data, indptr, indices, x, lengths = _powerlaw(40_000, 1 << 20, 4096, seed=21)
    d = [torch.from_numpy(a).cuda() for a in (data, indptr, indices, x)]
    y = k.spmv(*d, 40_000, 1 << 20)
    ref, budget = vo.spmv_csr(data, indptr, indices, x, (40_000, 1 << 20))
    assert vo.within_budget(y.cpu().numpy(), ref, budget, TOL)[0]
    # the same tensors with other contents: rows reversed in length order
    data2, indptr2, indices2, x2, _ = _powerlaw(40_000, 1 << 20, 4096, seed=22)
    n2 = min(len(data2), len(data))
    # keep the shapes: cut the second matrix down to the first one's nnz
    ip = np.minimum(indptr2, n2).astype(np.int32)
    d[0][:n2].copy_(torch.from_numpy(data2[:n2]))
    d[1].copy_(torch.from_numpy(ip))
    d[2][:n2].copy_(torch.from_numpy(indices2[:n2]))
    y2 = k.spmv(*d, 40_000, 1 << 20)
    ref2, budget2 = vo.spmv_csr(d[0].cpu().numpy(), ip, d[2].cpu().numpy(), x, (40_000, 1 << 20))
    ok, worst = vo.within_budget(y2.cpu().numpy(), ref2, budget2, TOL)
    assert ok, worst
