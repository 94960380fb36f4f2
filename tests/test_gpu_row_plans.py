"""Row plans: a CSR-like loop whose arrays come back unchanged launch after launch has the order of its
elements worked out once (the second time the arrays are seen) and kept; later launches run two kernels
over that order.  Every result is compared with the float64 oracle to the bar of the parity tests
(``|out - oracle| <= 1e-5 * sum(|terms|)`` per output), and a plan must never outlive the contents it
was built from: values or indices changed in place, arrays stored to by another loop, other arrays at the
same addresses.

Pattern: the CSR loop of the reference's examples/03-spmv.py:5-16 and
tests/integration/triton/tutorial/test_spmv.py:10-30."""
import gc

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
def env(gpu):
    import torch

    return torch, selfcheck.kernels()


def _loop(name="spmv", **opts):
    hits = [v[0] for kk, v in cg.code_cache.items() if kk[-1] == name and getattr(v[0], "last_launch", None) is not None
            and all(v[0].options.get(o, True) == val for o, val in opts.items())]
    return max(hits, key=lambda lp: lp.last_launch.serial)


def _names(launch):
    return [step[0].src.name.rsplit("_", 1)[-1] if step[0] else "clear" for step in (launch.sequence or [])]


def _planned(launch):
    return launch.plan is not None and _names(launch) == ["xcells", "sums"]


def _matrix(lengths, n, seed):
    rng = np.random.default_rng(seed)
    data, indptr, indices = wl.csr_matrix(np.asarray(lengths, dtype=np.int64), n, rng)
    x = rng.standard_normal(n, dtype=np.float32)
    return data, indptr, indices, x


def _gpu(torch, *arrays):
    return tuple(torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in arrays)


def _check(y, data, indptr, indices, x, m, n):
    ref, budget = vo.spmv_csr(data, indptr, indices, x, (m, n))
    ok, worst = vo.within_budget(y.cpu().numpy(), ref, budget, TOL)
    assert ok, worst


def _lengths(kind, m, rng):
    if kind == "0,10,20":
        return rng.integers(0, 3, m) * 10
    if kind == "zipf":
        return np.clip(rng.zipf(1.5, m), 1, 4096)
    if ".." in kind:
        a, b = kind.split("..")
        return rng.integers(int(a), int(b) + 1, m)
    return np.full(m, int(kind))


@pytest.mark.parametrize("m,n,lengths", [
    (50_000, 1 << 20, "16"),                 # the uniform matrix of the benchmark, scaled down; two blocks of rows
    (40_003, (1 << 22) - 12345, "1..31"),    # a last block that is not full, column ranges that are not a power of two
    (70_000, 3 << 20, "0,10,20"),            # empty rows; three blocks of rows
    (33_000, 7 << 20, "8"),                  # an operand of 28 MiB: 20 bits of column per range, tiles of 4096
    (36_000, 1 << 21, "1..127"),
    (40_000, 1 << 20, "zipf"),               # rows of up to 4096 elements: runs of slots within a tile
])
def test_a_plan_is_built_on_the_second_launch_and_run_from_then_on(env, m, n, lengths):
    torch, k = env
    ln = _lengths(lengths, m, np.random.default_rng(m))
    data, indptr, indices, x = _matrix(ln, n, seed=m + 1)
    td, tp, ti, tx = _gpu(torch, data, indptr, indices, x)
    y0 = k.spmv(td, tp, ti, tx, m, n)
    first = _loop().last_launch
    assert first.plan is None and first.spec.aux == "cells"         # seen once: a form that keeps nothing
    _check(y0, data, indptr, indices, x, m, n)
    y1 = k.spmv(td, tp, ti, tx, m, n)
    second = _loop().last_launch
    assert _planned(second) and second.plan.inspector_ms > 0
    assert second.plan.tile == (4096 if n > (1 << 22) else 6144)
    _check(y1, data, indptr, indices, x, m, n)
    assert bool((y1[torch.from_numpy(ln == 0).cuda()] == 0).all())
    y2 = k.spmv(td, tp, ti, tx, m, n)
    third = _loop().last_launch
    assert _planned(third) and third.plan is second.plan            # nothing rebuilt
    # the same bits from launch to launch: no sum is touched by two lanes at once
    assert torch.equal(y1, y2)
    # another operand with the same matrix: the plan does not depend on it
    x2 = np.random.default_rng(5).standard_normal(n, dtype=np.float32)
    y3 = k.spmv(td, tp, ti, torch.from_numpy(x2).cuda(), m, n)
    assert _loop().last_launch.plan is second.plan
    _check(y3, data, indptr, indices, x2, m, n)


@pytest.mark.parametrize("ptr_type,idx_type", [(np.int64, np.int64), (np.int32, np.int64), (np.int64, np.int32)])
def test_index_arrays_of_64_bits(env, ptr_type, idx_type):
    """Row starts and column indices of 64 bits (what torch's CSR tensors hold): the kernel that writes the pairs
    narrows them once it has checked that they lie inside the operand, and so do the kernels that group the
    elements in the launch before the plan exists."""
    torch, k = env
    m, n = 50_000, 1 << 21
    data, indptr, indices, x = _matrix(np.full(m, 12), n, seed=9)
    td, tx = _gpu(torch, data, x)
    tp, ti = _gpu(torch, indptr.astype(ptr_type), indices.astype(idx_type))
    for it in range(3):
        y = k.spmv(td, tp, ti, tx, m, n)
        _check(y, data, indptr, indices, x, m, n)
        launch = max((v[0] for kk, v in cg.code_cache.items() if kk[-1] == "spmv" and getattr(v[0], "last_launch", None) is not None),
                     key=lambda lp: lp.last_launch.serial).last_launch
        assert _planned(launch) == (it >= 1)
        assert it >= 1 or launch.spec.aux == "cells"


def test_values_and_indices_changed_in_place_give_the_new_result(env):
    torch, k = env
    m, n = 45_000, 1 << 20
    data, indptr, indices, x = _matrix(np.random.default_rng(1).integers(4, 30, m), n, seed=2)
    td, tp, ti, tx = _gpu(torch, data, indptr, indices, x)
    for _ in range(3):
        y = k.spmv(td, tp, ti, tx, m, n)
    plan = _loop().last_launch.plan
    assert plan is not None
    _check(y, data, indptr, indices, x, m, n)
    # values changed through torch: the version counter of the tensor moves, the plan is not used again
    td.mul_(-2.0)
    y = k.spmv(td, tp, ti, tx, m, n)
    assert _loop().last_launch.plan is None
    _check(y, -2.0 * data, indptr, indices, x, m, n)
    y = k.spmv(td, tp, ti, tx, m, n)
    assert _loop().last_launch.plan not in (None, plan)             # seen twice in the new state: a new plan
    _check(y, -2.0 * data, indptr, indices, x, m, n)
    # indices changed in place (the columns of every row mirrored: still sorted rows)
    mirrored = (n - 1 - indices).astype(np.int32)
    ti.copy_(torch.from_numpy(mirrored).cuda())
    for _ in range(3):
        y = k.spmv(td, tp, ti, tx, m, n)
        _check(y, -2.0 * data, indptr, mirrored, x, m, n)
    assert _planned(_loop().last_launch)
    # a slice assignment through a view moves the counter of the base tensor as well
    td[1000:2000] = 0.0
    d3 = -2.0 * data
    d3[1000:2000] = 0.0
    y = k.spmv(td, tp, ti, tx, m, n)
    assert _loop().last_launch.plan is None
    _check(y, d3, indptr, mirrored, x, m, n)


@appy.jit
def scale_values(v, f):
    #pragma parallel for simd
    for i in range(v.shape[0]):
        v[i] = v[i] * f


def test_arrays_stored_to_by_another_loop_drop_the_plan(env):
    """A kernel of this package that writes into the values does not move the tensor's version counter:
    the launcher itself drops every plan built from memory a launch stores into."""
    torch, k = env
    m, n = 45_000, 1 << 20
    data, indptr, indices, x = _matrix(np.full(m, 12), n, seed=3)
    td, tp, ti, tx = _gpu(torch, data, indptr, indices, x)
    for _ in range(3):
        y = k.spmv(td, tp, ti, tx, m, n)
    plan = _loop().last_launch.plan
    assert plan is not None and plan.valid
    version = td._version
    scale_values(td, 3.0)
    assert td._version == version and not plan.valid
    y = k.spmv(td, tp, ti, tx, m, n)
    assert _loop().last_launch.plan is None
    _check(y, 3.0 * data, indptr, indices, x, m, n)
    for _ in range(2):
        y = k.spmv(td, tp, ti, tx, m, n)
    assert _planned(_loop().last_launch)
    _check(y, 3.0 * data, indptr, indices, x, m, n)
    # a store into a part of the array, through a view
    scale_values(td[5000:6000], 0.0)
    d2 = 3.0 * data
    d2[5000:6000] = 0.0
    y = k.spmv(td, tp, ti, tx, m, n)
    assert _loop().last_launch.plan is None
    _check(y, d2, indptr, indices, x, m, n)
    # storing into the operand or the result touches no plan
    for _ in range(2):
        y = k.spmv(td, tp, ti, tx, m, n)
    plan = _loop().last_launch.plan
    scale_values(tx, 2.0)
    assert plan.valid
    y = k.spmv(td, tp, ti, tx, m, n)
    assert _loop().last_launch.plan is plan
    _check(y, d2, indptr, indices, 2.0 * x, m, n)


def test_a_launch_over_a_kept_order_is_repeated_without_staging_while_the_plan_stands(env):
    """With the same tensors and scalars as the call before, the two kernels that run a plan are launched again as
    they were staged; the repeat stops as soon as the plan may not be true any more: a value changed in place, a
    store by another loop, other tensors at the same addresses, memory given back."""
    torch, k = env
    m, n = 45_000, 1 << 20
    data, indptr, indices, x = _matrix(np.full(m, 12), n, seed=6)
    td, tp, ti, tx = _gpu(torch, data, indptr, indices, x)
    y = torch.empty(m, device="cuda")

    @appy.jit
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

    for _ in range(3):
        into(td, tp, ti, tx, y, m)
    assert _planned(_loop("into").last_launch)
    _check(y, data, indptr, indices, x, m, n)
    y.zero_()
    assert staged_by(lambda: into(td, tp, ti, tx, y, m)) == 0          # repeated as it was
    _check(y, data, indptr, indices, x, m, n)
    tx.mul_(2.0)                                                         # the operand is not part of the plan
    assert staged_by(lambda: into(td, tp, ti, tx, y, m)) == 0
    _check(y, data, indptr, indices, 2.0 * x, m, n)
    td.mul_(3.0)                                                         # a value changed in place: staged anew
    assert staged_by(lambda: into(td, tp, ti, tx, y, m)) == 1
    assert _loop("into").last_launch.plan is None
    _check(y, 3.0 * data, indptr, indices, 2.0 * x, m, n)
    for _ in range(2):
        into(td, tp, ti, tx, y, m)
    assert _planned(_loop("into").last_launch)
    assert staged_by(lambda: into(td, tp, ti, tx, y, m)) == 0
    scale_values(td, 0.5)                                                # a store by another loop
    assert staged_by(lambda: into(td, tp, ti, tx, y, m)) == 1
    _check(y, 1.5 * data, indptr, indices, 2.0 * x, m, n)
    for _ in range(2):
        into(td, tp, ti, tx, y, m)
    assert staged_by(lambda: into(td, tp, ti, tx, y, m)) == 0
    appy.release()                                                       # the memory the staged launch names is gone
    assert staged_by(lambda: into(td, tp, ti, tx, y, m)) == 1
    _check(y, 1.5 * data, indptr, indices, 2.0 * x, m, n)
    # other tensors at the same addresses
    for _ in range(2):
        into(td, tp, ti, tx, y, m)
    assert staged_by(lambda: into(td, tp, ti, tx, y, m)) == 0
    ptr = td.data_ptr()
    del td
    gc.collect()
    data2 = (data * -1.0).astype(np.float32)
    td2 = torch.from_numpy(data2).cuda()
    if td2.data_ptr() == ptr:
        assert staged_by(lambda: into(td2, tp, ti, tx, y, m)) == 1
        _check(y, data2, indptr, indices, 2.0 * x, m, n)
    appy.release()


def test_stores_that_are_not_staged_again_drop_the_plan_too(env):
    """A call with the same tensors and scalars as an earlier one repeats that call's launch without staging it
    again, and a graph replays what was recorded: both must drop the plans built from what they store into."""
    torch, k = env
    m, n = 45_000, 1 << 20
    data, indptr, indices, x = _matrix(np.full(m, 12), n, seed=4)
    td, tp, ti, tx = _gpu(torch, data, indptr, indices, x)
    scale_values(td, 2.0)
    scale_values(td, 2.0)                           # from here on this call is a repeated launch
    loop = [v[0] for kk, v in cg.code_cache.items() if kk[-1] == "scale_values"][-1]
    assert loop._replays
    for _ in range(3):
        y = k.spmv(td, tp, ti, tx, m, n)
    plan = _loop().last_launch.plan
    assert plan is not None and plan.valid
    _check(y, 4.0 * data, indptr, indices, x, m, n)
    staged = cg.Launch.serial
    scale_values(td, 2.0)
    assert cg.Launch.serial == staged               # nothing was staged
    assert not plan.valid
    y = k.spmv(td, tp, ti, tx, m, n)
    assert _loop().last_launch.plan is None
    _check(y, 8.0 * data, indptr, indices, x, m, n)
    # the same through a graph
    with appy.graph() as g:
        scale_values(td, 0.5)
    torch.cuda.synchronize()
    for _ in range(3):
        y = k.spmv(td, tp, ti, tx, m, n)
    plan = _loop().last_launch.plan
    assert plan is not None and plan.valid
    g.launch(torch.cuda.current_stream().cuda_stream)
    assert not plan.valid
    y = k.spmv(td, tp, ti, tx, m, n)
    assert _loop().last_launch.plan is None
    _check(y, 4.0 * data, indptr, indices, x, m, n)
    g.close()


def test_another_matrix_at_the_same_addresses(env):
    torch, k = env
    m, n = 45_000, 1 << 20
    a = _matrix(np.full(m, 10), n, seed=4)
    b = _matrix(np.full(m, 10), n, seed=5)          # same shapes, other columns and values
    td, tp, ti, tx = _gpu(torch, *a)
    for _ in range(3):
        y = k.spmv(td, tp, ti, tx, m, n)
    assert _planned(_loop().last_launch)
    # copied over the first matrix, tensor by tensor
    for dst, src in zip((td, tp, ti), b[:3]):
        dst.copy_(torch.from_numpy(src).cuda())
    y = k.spmv(td, tp, ti, tx, m, n)
    assert _loop().last_launch.plan is None
    _check(y, b[0], b[1], b[2], a[3], m, n)
    for _ in range(2):
        y = k.spmv(td, tp, ti, tx, m, n)
    assert _planned(_loop().last_launch)
    _check(y, b[0], b[1], b[2], a[3], m, n)
    # the tensors freed and new ones allocated (the allocator hands out the same blocks again): other
    # objects, so nothing of the old plan applies, whatever their addresses and version counters
    addresses = (td.data_ptr(), tp.data_ptr(), ti.data_ptr())
    del td, tp, ti
    gc.collect()
    c = _matrix(np.full(m, 10), n, seed=6)
    td, tp, ti = _gpu(torch, *c[:3])
    same = (td.data_ptr(), tp.data_ptr(), ti.data_ptr()) == addresses
    for it in range(3):
        y = k.spmv(td, tp, ti, tx, m, n)
        assert (_loop().last_launch.plan is not None) == (it >= 1)
        _check(y, c[0], c[1], c[2], a[3], m, n)
    assert same or True        # (whether the blocks were handed out again is the allocator's business)


def test_reuse_can_be_switched_off_and_forced(env):
    torch, _k = env
    m, n = 40_000, 1 << 20
    data, indptr, indices, x = _matrix(np.full(m, 16), n, seed=7)
    td, tp, ti, tx = _gpu(torch, data, indptr, indices, x)
    off = selfcheck.kernels(hip_reuse=False)
    for _ in range(4):
        y = off.spmv(td, tp, ti, tx, m, n)
        assert _loop(hip_reuse=False).last_launch.plan is None
    _check(y, data, indptr, indices, x, m, n)
    now = selfcheck.kernels(hip_reuse="now")
    y = now.spmv(td, tp, ti, tx, m, n)
    assert _planned(_loop(hip_reuse="now").last_launch)            # built by the first launch
    _check(y, data, indptr, indices, x, m, n)
    later = selfcheck.kernels(hip_reuse=4)                        # built by the fourth launch over the same tensors
    for it in range(5):
        y = later.spmv(td, tp, ti, tx, m, n)
        assert _planned(_loop(hip_reuse=4).last_launch) == (it >= 3)
    _check(y, data, indptr, indices, x, m, n)
    # NumPy callers keep the forms that keep nothing (their arrays are copied per call)
    k = selfcheck.kernels()
    for _ in range(3):
        y = k.spmv(data, indptr, indices, x, m, n)
        assert _loop().last_launch.plan is None


@appy.jit
def windows(data, start, end, indices, x, y, beta, m):
    #pragma parallel for
    for i in range(m):
        s = 0.0
        #pragma simd
        for j in range(start[i], end[i]):
            s += data[j] * x[indices[j]]
        y[i] = beta * y[i] + s


def test_arrays_the_inspector_refuses_keep_the_other_forms(env):
    """Row ranges that do not follow one another, and indices outside the operand: legal loops (or loops that
    fault with or without a plan); no plan is built, the result is that of the loop as written."""
    torch, _k = env
    m, n = 40_000, 1 << 20
    data, indptr, indices, x = _matrix(np.full(m, 16), n, seed=8)
    start, end = indptr[:-1].copy(), indptr[1:].copy()
    start[[1000, 1001]] = start[[1001, 1000]]       # two rows swapped
    end[[1000, 1001]] = end[[1001, 1000]]
    td, ts, te, ti, tx = _gpu(torch, data, start, end, indices, x)
    terms = data.astype(np.float64) * x.astype(np.float64)[indices]
    cs = np.concatenate([[0.0], np.cumsum(terms)])
    ca = np.concatenate([[0.0], np.cumsum(np.abs(terms))])
    ref = 0.5 + cs[end] - cs[start]
    budget = 0.5 + ca[end] - ca[start]
    for _ in range(4):
        y = torch.ones(m, device="cuda")
        windows(td, ts, te, ti, tx, y, 0.5, m)
        assert _loop("windows").last_launch.plan is None
        assert np.all(np.abs(y.cpu().numpy() - ref) <= TOL * budget + 1e-9 * ca[-1])
    # the same arrays in order: a plan, and the statement after the loop runs once per row
    ts, te = _gpu(torch, indptr[:-1].copy(), indptr[1:].copy())
    ref = 0.5 + cs[indptr[1:]] - cs[indptr[:-1]]
    budget = 0.5 + ca[indptr[1:]] - ca[indptr[:-1]]
    for it in range(3):
        y = torch.ones(m, device="cuda")
        windows(td, ts, te, ti, tx, y, 0.5, m)
        assert (_loop("windows").last_launch.plan is not None) == (it >= 1)
        assert np.all(np.abs(y.cpu().numpy() - ref) <= TOL * budget + 1e-9 * ca[-1])


def test_terms_with_a_scalar_factor_integer_sums_and_no_second_operand(env):
    torch, _k = env
    rng = np.random.default_rng(9)
    m, n = 40_000, 1 << 20
    ln = rng.integers(4, 24, m)
    data, indptr, indices, x = _matrix(ln, n, seed=10)
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
    def integer(w, indptr, indices, xi, y, m):
        #pragma parallel for
        for i in range(m):
            s = 0
            #pragma simd
            for j in range(indptr[i], indptr[i + 1]):
                s += w[j] * xi[indices[j]]
            y[i] = s

    @appy.jit
    def pattern(indptr, indices, x, y, m):
        #pragma parallel for
        for i in range(m):
            s = 0.0
            #pragma simd
            for j in range(indptr[i], indptr[i + 1]):
                s += x[indices[j]]
            y[i] = s

    td, tp, ti, tx, tw, txi = _gpu(torch, data, indptr, indices, x, w, xi)
    ref, budget = vo.spmv_csr(data, indptr, indices, x, (m, n))
    for alpha in (0.5, -3.0, 0.5):                  # scalars of the term are read at every launch, not kept in the plan
        for it in range(3):
            y = torch.empty(m, device="cuda")
            scaled(td, tp, ti, tx, y, alpha, m)
            ok, worst = vo.within_budget(y.cpu().numpy(), alpha * ref, abs(alpha) * budget, TOL)
            assert ok, worst
    assert _planned(_loop("scaled").last_launch)
    exact = np.zeros(m, dtype=np.int64)
    np.add.at(exact, np.repeat(np.arange(m), ln), w.astype(np.int64) * xi[indices])
    for it in range(3):
        yi = torch.zeros(m, dtype=torch.int32, device="cuda")
        integer(tw, tp, ti, txi, yi, m)
        assert np.array_equal(yi.cpu().numpy(), exact)          # integer sums: exact in any order
    assert _planned(_loop("integer").last_launch)
    ones = np.ones(nnz, dtype=np.float32)
    for it in range(3):
        y = torch.empty(m, device="cuda")
        pattern(tp, ti, tx, y, m)
        _check(y, ones, indptr, indices, x, m, n)
    assert _planned(_loop("pattern").last_launch)


def test_a_part_of_the_rows_and_rows_with_many_elements_in_one_tile(env):
    """A loop over rows [lo, hi) of the matrix; rows whose elements crowd into a narrow band of columns, so
    that one tile holds long runs of slots of the same row, and more than 1024 rows with runs."""
    torch, _k = env
    rng = np.random.default_rng(11)
    m, n = 40_000, 1 << 20
    ln = np.full(m, 2, dtype=np.int64)
    ln[::50] = 300                                              # 800 rows of 300 elements ...
    indptr = np.zeros(m + 1, dtype=np.int64)
    np.cumsum(ln, out=indptr[1:])
    cols = np.empty(int(indptr[-1]), dtype=np.int64)
    for i in range(m):                                          # ... all within 4096 columns of one range
        cols[indptr[i]:indptr[i + 1]] = np.sort(rng.choice(4096, size=ln[i], replace=False)) + 5000
    data = rng.standard_normal(len(cols), dtype=np.float32)
    x = rng.standard_normal(n, dtype=np.float32)
    indptr, cols = indptr.astype(np.int32), cols.astype(np.int32)

    @appy.jit
    def part(data, indptr, indices, x, y, lo, hi):
        #pragma parallel for
        for i in range(lo, hi):
            s = 0.0
            #pragma simd
            for j in range(indptr[i], indptr[i + 1]):
                s += data[j] * x[indices[j]]
            y[i] = s

    td, tp, ti, tx = _gpu(torch, data, indptr, cols, x)
    ref, budget = vo.spmv_csr(data, indptr, cols, x, (m, n))
    for lo, hi in ((0, m), (123, m - 77), (5000, 5000 + 33_000)):
        for it in range(3):
            y = torch.full((m,), 7.0, device="cuda")
            part(td, tp, ti, tx, y, lo, hi)
            yh = y.cpu().numpy()
            assert np.all(yh[:lo] == 7.0) and np.all(yh[hi:] == 7.0)
            assert np.all(np.abs(yh[lo:hi] - ref[lo:hi]) <= TOL * budget[lo:hi])
        assert _planned(_loop("part").last_launch)


@pytest.mark.parametrize("grid,split", [(8, 3), (16, 1), (64, 5)])
def test_few_workgroups_walk_many_cells_one_after_the_other(env, grid, split):
    """The kernel that runs a plan gives every workgroup a sequence of runs of tiles (a cell, or a part of one)
    and walks their tiles as one sequence: with few workgroups each walks many, among them cells without any
    element (all columns of a block of rows in one range) and a last block of rows that is not full.  The result
    must not depend on how the runs are dealt out."""
    torch, _k = env
    rng = np.random.default_rng(17)
    m, n = 3 * 32768 + 1234, 1 << 21
    ln = rng.integers(0, 40, m).astype(np.int64)
    ln[32768:65536] = 12
    indptr = np.zeros(m + 1, dtype=np.int64)
    np.cumsum(ln, out=indptr[1:])
    cols = rng.integers(0, n, int(indptr[-1]))
    lo, hi = int(indptr[32768]), int(indptr[65536])
    cols[lo:hi] = rng.integers(5 * (n // 8), 6 * (n // 8), hi - lo)          # the second block of rows: one range only
    data = rng.standard_normal(len(cols), dtype=np.float32)
    x = rng.standard_normal(n, dtype=np.float32)
    indptr, cols = indptr.astype(np.int32), cols.astype(np.int32)
    ref, budget = vo.spmv_csr(data, indptr, cols, x, (m, n))
    td, tp, ti, tx = _gpu(torch, data, indptr, cols, x)
    dealt = selfcheck.kernels(hip_reuse="now", hip_plan_grid=grid, hip_plan_split=split)
    usual = selfcheck.kernels(hip_reuse="now", hip_plan_split=split)
    ys = []
    for k in (dealt, usual):
        for it in range(2):
            y = k.spmv(td, tp, ti, tx, m, n)
            yh = y.cpu().numpy()
            assert np.all(np.abs(yh - ref) <= TOL * budget)
            ys.append(y)
        launch = _loop(hip_plan_split=split).last_launch              # (the loop that ran last)
        assert _planned(launch) and launch.plan.split == split and launch.plan.ncell == 32
        assert launch.grid[0] == (grid if k is dealt else min(32 * split, launch.hw.cus // 8 * 8))
    assert all(torch.equal(ys[0], y) for y in ys[1:])
    appy.release()


@pytest.mark.parametrize("seed", range(12))
def test_random_shapes_ranges_and_row_lengths(env, seed):
    """Matrices of random sizes and row-length laws, a random range of their rows, random numbers of workgroups:
    the launches over the kept order must give the oracle's product for the rows of the range and touch no other."""
    torch, _k = env
    rng = np.random.default_rng(1000 + seed)
    m = int(rng.integers(40_000, 150_000))
    n = int(rng.integers((1 << 20) + 1, 1 << 23))
    law = ["0..3", "16", "1..40", "zipf", "0,10,20", "banded"][seed % 6]
    if law == "banded":
        ln = rng.integers(1, 24, m)
    else:
        ln = _lengths(law, m, rng)
    indptr = np.zeros(m + 1, dtype=np.int64)
    np.cumsum(ln, out=indptr[1:])
    nnz = int(indptr[-1])
    if law == "banded":
        # columns near the diagonal: most cells of a block of rows hold nothing
        rows = np.repeat(np.arange(m), ln)
        cols = np.clip((rows * (n / max(m, 1))).astype(np.int64) + rng.integers(-3000, 3000, nnz), 0, n - 1)
    else:
        cols = rng.integers(0, n, nnz)
    data = rng.standard_normal(nnz).astype(np.float32)
    x = rng.standard_normal(n).astype(np.float32)
    indptr32, cols32 = indptr.astype(np.int32), cols.astype(np.int32)
    lo = int(rng.integers(0, m // 8))
    hi = int(rng.integers(m - m // 8, m + 1)) if seed % 2 else m
    if seed % 2 == 0:
        lo = 0

    opts = {"hip_reuse": "now"}
    if seed % 3 == 0:
        opts["hip_plan_grid"] = int(rng.choice([8, 24, 64]))

    @appy.jit(**opts)
    def part(data, indptr, indices, x, y, lo, hi):
        #pragma parallel for
        for i in range(lo, hi):
            s = 0.0
            #pragma simd
            for j in range(indptr[i], indptr[i + 1]):
                s += data[j] * x[indices[j]]
            y[i] = s

    td, tp, ti, tx = _gpu(torch, data, indptr32, cols32, x)
    ref, budget = vo.spmv_csr(data, indptr32, cols32, x, (m, n))
    planned = 0
    for it in range(2):
        y = torch.full((m,), 7.0, device="cuda")
        part(td, tp, ti, tx, y, lo, hi)
        yh = y.cpu().numpy()
        assert np.all(yh[:lo] == 7.0) and np.all(yh[hi:] == 7.0)
        assert np.all(np.abs(yh[lo:hi] - ref[lo:hi]) <= TOL * budget[lo:hi]), (law, m, n, lo, hi)
        planned += _planned(_loop("part").last_launch)
    # (small or very sparse inputs do not qualify for a plan: then the other forms have been checked)
    assert planned in (0, 2)
    print(f"random shapes: law {law} m {m} n {n} rows [{lo}, {hi}) nnz {nnz}: {'kept order' if planned else 'other forms'}")
    appy.release()


def test_plans_are_bounded_released_and_kept_out_of_the_way(env, monkeypatch):
    torch, k = env
    m, n = 40_000, 1 << 20
    mats = [_matrix(np.full(m, 8 + s), n, seed=20 + s) for s in range(3)]
    dev = [_gpu(torch, *mt) for mt in mats]
    loop = None
    for td, tp, ti, tx in dev:
        for _ in range(2):
            k.spmv(td, tp, ti, tx, m, n)
        loop = _loop()
        assert _planned(loop.last_launch)
    assert len(loop._plans) == cg.PLANS_PER_LOOP                    # the least recently used one has gone
    held = sum(pl.nbytes for pl in loop._plans)
    assert held > 0
    appy.release()
    assert loop._plans == [] and not cg._live_plans
    # a limit on what a loop may hold that no plan fits under: the forms that keep nothing, same results
    monkeypatch.setenv("APPY_HIP_SCRATCH_MAX_BYTES", str(1 << 20))
    td, tp, ti, tx = dev[0]
    for _ in range(3):
        y = k.spmv(td, tp, ti, tx, m, n)
        assert _loop().last_launch.plan is None
    _check(y, *mats[0][:3], mats[0][3], m, n)
