"""Parity at the full workload sizes through facts that need no oracle run:
closed forms, exact special cases, linearity and cross-kernel identities.
Inputs are built on the device (seeded), so the whole file runs in seconds.

Sizes: float32 N = 2^28 for the reductions, N = 2^24 for vec_add, 16384 x 16384
for GEMV, M = N = 2^22 for SpMV (uniform 16/row and Zipf(1.5) clipped to
[1, 4096]), M = N = 2^20 with 128 columns for SpMM."""
import numpy as np
import pytest

from appy_amd.backends.hip import selfcheck

pytestmark = pytest.mark.gpu
TOL = 1e-5


@pytest.fixture(scope="module")
def env(gpu):
    import torch

    torch.cuda.set_device(0)
    return torch, selfcheck.kernels()


def test_vec_add_full_size_bit_exact(env):
    torch, k = env
    n = 1 << 24
    g = torch.Generator(device="cuda").manual_seed(1)
    a = torch.empty(n, device="cuda").uniform_(-1, 1, generator=g)
    b = torch.empty(n, device="cuda").uniform_(-1, 1, generator=g)
    c = k.vec_add(a, b)
    assert torch.equal(c, a + b)                    # IEEE addition, element by element
    assert torch.equal(k.vec_add(b, a), c)          # commutative


def test_reductions_full_size_closed_forms(env):
    torch, k = env
    n = 1 << 28
    ones = torch.ones(n, device="cuda")
    assert k.vector_sum(ones) == float(n)                                   # exact: integers below 2^53
    mask = torch.zeros(n, dtype=torch.bool, device="cuda")
    mask[::2] = True
    assert k.masked_sum(ones, mask) == float(n // 2)
    assert k.masked_sum(ones, ~mask) == float(n // 2)
    del ones
    g = torch.Generator(device="cuda").manual_seed(2)
    A = torch.rand(n, device="cuda", generator=g)
    s = k.vector_sum(A)
    budget = float(A.sum(dtype=torch.float64))                              # all terms positive: sum(|terms|) = sum
    assert abs(s - budget) <= TOL * budget
    # complement identity and linearity, within the same budget
    m1, m0 = k.masked_sum(A, mask), k.masked_sum(A, ~mask)
    assert abs((m1 + m0) - s) <= 2 * TOL * budget
    A.mul_(2.0)                                                             # exact in binary floating point
    assert abs(k.vector_sum(A) - 2 * s) <= 2 * TOL * budget


def test_gemv_full_size_exact_cases(env):
    torch, k = env
    r = 16384
    g = torch.Generator(device="cuda").manual_seed(3)
    A = torch.randn((r, r), device="cuda", generator=g)
    for col in (0, 4097, r - 1):
        e = torch.zeros(r, device="cuda")
        e[col] = 1.0
        assert torch.equal(k.gemv(A, e), A[:, col])                         # products by 0 and 1 are exact
    x = torch.randn(r, device="cuda", generator=g)
    y = k.gemv(A, x)
    ref = A.double() @ x.double()
    budget = A.double().abs() @ x.double().abs()
    assert bool(((y.double() - ref).abs() <= TOL * budget).all())


def _csr(torch, lengths, n, seed):
    from oracle.device_workloads import device_csr

    return device_csr(torch, lengths, n, seed)


@pytest.mark.parametrize("kind", ["uniform", "powerlaw"])
def test_spmv_full_size_row_lengths_and_linearity(env, kind):
    torch, k = env
    m = 1 << 22
    if kind == "uniform":
        lengths = np.full(m, 16, dtype=np.int64)
    else:
        lengths = np.clip(np.random.default_rng(104).zipf(1.5, m), 1, 4096).astype(np.int64)
    data, indptr, indices = _csr(torch, lengths, m, seed=7)
    ones_x = torch.ones(m, device="cuda")
    # all values 1 and x = 1: y is the row length, exactly (integers <= 4096 in float32)
    y = k.spmv(torch.ones_like(data), indptr, indices, ones_x, m, m)
    assert torch.equal(y, torch.from_numpy(lengths).to("cuda").float())
    # x = column index (exact in float32 below 2^24): y is the sum of the row's column indices
    col_x = torch.arange(m, device="cuda", dtype=torch.float32)
    y = k.spmv(torch.ones_like(data), indptr, indices, col_x, m, m)
    seg = torch.zeros(m, dtype=torch.float64, device="cuda")
    rows = torch.repeat_interleave(torch.arange(m, device="cuda"), torch.from_numpy(lengths).to("cuda"))
    seg.index_add_(0, rows, indices.double())
    assert bool(((y.double() - seg).abs() <= TOL * seg).all())
    # random values: linear in x within the budget sum(|a||x|)
    x = torch.randn(m, device="cuda", generator=torch.Generator(device="cuda").manual_seed(8))
    y1 = k.spmv(data, indptr, indices, x, m, m)
    y2 = k.spmv(data, indptr, indices, 2 * x, m, m)
    budget = torch.zeros(m, dtype=torch.float64, device="cuda")
    budget.index_add_(0, rows, (data.double() * x[indices.long()].double()).abs())
    assert bool(((y2.double() - 2 * y1.double()).abs() <= 4 * TOL * budget).all())
    ref = torch.zeros(m, dtype=torch.float64, device="cuda")
    ref.index_add_(0, rows, data.double() * x[indices.long()].double())
    assert bool(((y1.double() - ref).abs() <= TOL * budget).all())


@pytest.mark.parametrize("kind", ["uniform", "powerlaw"])
def test_spmv_full_size_with_the_order_of_the_elements_kept(env, kind):
    """The same tensors launch after launch: the first launch reads the raw arrays, the second works out the
    order of the elements and runs it, the third only runs it.  All three against a float64 sum built with
    `index_add_`; exact cases (all ones) through the kept order as well; the same bits from launch to launch."""
    import appy_amd as appy
    from appy_amd.backends.hip import codegen as cg

    torch, k = env
    m = 1 << 22
    if kind == "uniform":
        lengths = np.full(m, 16, dtype=np.int64)
    else:
        lengths = np.clip(np.random.default_rng(104).zipf(1.5, m), 1, 4096).astype(np.int64)
    data, indptr, indices = _csr(torch, lengths, m, seed=11)
    x = torch.randn(m, device="cuda", generator=torch.Generator(device="cuda").manual_seed(12))
    rows = torch.repeat_interleave(torch.arange(m, device="cuda"), torch.from_numpy(lengths).to("cuda"))
    terms = data.double() * x[indices.long()].double()
    ref = torch.zeros(m, dtype=torch.float64, device="cuda").index_add_(0, rows, terms)
    budget = torch.zeros(m, dtype=torch.float64, device="cuda").index_add_(0, rows, terms.abs())
    del terms, rows

    def last_plan():
        loops = [v[0] for kk, v in cg.code_cache.items() if kk[-1] == "spmv" and getattr(v[0], "last_launch", None) is not None
                 and v[0].options.get("hip_reuse", True) is True]
        return max(loops, key=lambda lp: lp.last_launch.serial).last_launch.plan

    ys = []
    for launch in range(3):
        y = k.spmv(data, indptr, indices, x, m, m)
        assert (last_plan() is not None) == (launch >= 1)
        assert bool(((y.double() - ref).abs() <= TOL * budget).all())
        ys.append(y)
    assert torch.equal(ys[1], ys[2])
    plan = last_plan()
    assert plan.ncell == 8 * (m >> 15) and plan.split == 1 and plan.inspector_ms > 0
    # all values 1 and x = 1: the row lengths, exactly - through a plan (the tensors are seen twice)
    ones, ones_x = torch.ones_like(data), torch.ones(m, device="cuda")
    for launch in range(2):
        y = k.spmv(ones, indptr, indices, ones_x, m, m)
        assert torch.equal(y, torch.from_numpy(lengths).to("cuda").float())
    assert last_plan() is not None and last_plan() is not plan
    appy.release()


def test_spmv_full_size_banded_matrix_shares_its_cells(env):
    """A banded matrix of 2^22 rows (16 per row within 3000 columns of the diagonal): of the eight cells of a block of
    rows one holds everything, so two workgroups share every cell and the runs are dealt by size; the product against a
    float64 sum built with `index_add_`, the same bits from launch to launch."""
    import appy_amd as appy
    from appy_amd.backends.hip import codegen as cg

    torch, k = env
    m = n = 1 << 22
    g = torch.Generator(device="cuda").manual_seed(5)
    rows = torch.arange(m, device="cuda").repeat_interleave(16)
    cols = (rows + torch.randint(-3000, 3000, (rows.numel(),), device="cuda", generator=g)).clamp_(0, n - 1)
    cols, _ = cols.view(m, 16).sort(dim=1)
    indices = cols.reshape(-1).to(torch.int32)
    indptr = (torch.arange(m + 1, device="cuda") * 16).to(torch.int32)
    data = torch.randn(rows.numel(), device="cuda", generator=g)
    x = torch.randn(n, device="cuda", generator=g)
    terms = data.double() * x.double()[indices.long()]
    ref = torch.zeros(m, device="cuda", dtype=torch.float64).index_add_(0, rows, terms)
    budget = torch.zeros(m, device="cuda", dtype=torch.float64).index_add_(0, rows, terms.abs())
    del rows, cols, terms
    ys = []
    for launch in range(3):
        y = k.spmv(data, indptr, indices, x, m, n)
        assert bool(((y.double() - ref).abs() <= TOL * budget).all())
        ys.append(y)
    assert torch.equal(ys[1], ys[2])
    loops = [v[0] for kk, v in cg.code_cache.items() if kk[-1] == "spmv" and getattr(v[0], "last_launch", None) is not None
             and v[0].options.get("hip_reuse", True) is True]
    launch = max(loops, key=lambda lp: lp.last_launch.serial).last_launch
    plan = launch.plan
    assert plan is not None and plan.ncell == 8 * (m >> 15) and plan.split == 2 and launch.grid[0] == plan.grid
    appy.release()


def test_spmm_full_size_against_spmv_columns(env):
    torch, k = env
    m = 1 << 20
    lengths = np.minimum(np.random.default_rng(5).poisson(32, m), m).astype(np.int64)
    data, indptr, indices = _csr(torch, lengths, m, seed=9)
    B = torch.randn((m, 128), device="cuda", generator=torch.Generator(device="cuda").manual_seed(10))
    C = torch.full((m, 128), float("nan"), device="cuda")
    k.spmm(data, indptr, indices, B, C, m)
    for col in (0, 77, 127):
        y = k.spmv(data, indptr, indices, B[:, col].contiguous(), m, m)
        # same products, different summation order: both are within the budget of the exact value
        rows = torch.repeat_interleave(torch.arange(m, device="cuda"), torch.from_numpy(lengths).to("cuda"))
        budget = torch.zeros(m, dtype=torch.float64, device="cuda")
        budget.index_add_(0, rows, (data.double() * B[indices.long(), col].double()).abs())
        assert bool(((C[:, col].double() - y.double()).abs() <= 2 * TOL * budget).all())
    # rows without non-zeros are exactly zero
    empty = torch.from_numpy(lengths == 0).to("cuda")
    if bool(empty.any()):
        assert bool((C[empty] == 0).all())
