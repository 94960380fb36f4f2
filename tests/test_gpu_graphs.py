"""HIP-graph capture of launch sequences: every replay is compared with the
same steps launched one by one, with eager launches and synchronisations
between the replays."""
import time

import numpy as np
import pytest

import appy

pytestmark = pytest.mark.gpu


@appy.jit
def jacobi_step(A, B):
    #pragma parallel for simd
    for i in range(1, A.shape[0] - 1):
        B[i] = 0.33333 * (A[i - 1] + A[i] + A[i + 1])
    #pragma parallel for simd
    for i in range(1, A.shape[0] - 1):
        A[i] = 0.33333 * (B[i - 1] + B[i] + B[i + 1])


@appy.jit
def scale_rows(M, f):
    #pragma parallel for
    for i in range(M.shape[0]):
        #pragma simd
        for j in range(M.shape[1]):
            M[i, j] = M[i, j] * f


def test_replays_equal_eager_steps_on_gpu_tensors(gpu):
    import torch

    n, steps = 4001, 20
    rng = np.random.default_rng(0)
    a0, b0 = rng.random(n), rng.random(n)
    A = torch.from_numpy(a0).cuda()
    B = torch.from_numpy(b0).cuda()
    jacobi_step(A.clone(), B.clone())                 # compiled and loaded before the capture
    with appy.graph() as g:
        for _ in range(steps):
            jacobi_step(A, B)
    assert g.launches == 2 * steps
    assert np.array_equal(A.cpu().numpy(), a0)        # capturing runs nothing
    Ae, Be = torch.from_numpy(a0).cuda(), torch.from_numpy(b0).cuda()
    for replay in range(4):
        g.launch()
        g.synchronize()
        for _ in range(steps):                        # eager work of the same program between replays
            jacobi_step(Ae, Be)
        torch.cuda.synchronize()
        assert torch.equal(A, Ae) and torch.equal(B, Be), replay
    # ordered with PyTorch's stream when asked to
    s = torch.cuda.current_stream().cuda_stream
    A.mul_(2.0)
    g.launch(stream=s)
    Ae.mul_(2.0)
    for _ in range(steps):
        jacobi_step(Ae, Be)
    torch.cuda.synchronize()
    assert torch.equal(A, Ae)
    g.close()


def test_resident_numpy_arrays_can_be_captured_and_scalars_are_frozen(gpu):
    rng = np.random.default_rng(1)
    M = rng.random((300, 70))
    ref = M.copy()
    f = 1.5
    with appy.resident(M):
        scale_rows(M, f)                              # warm-up, eager: M *= 1.5
        with appy.graph() as g:
            scale_rows(M, f)
            scale_rows(M, 2.0)
        f = 100.0                                     # not seen by the graph
        for _ in range(3):
            g.launch()
        appy.sync_host(M)
        assert np.allclose(M, ref * 1.5 * (1.5 * 2.0) ** 3, rtol=1e-13)
        g.launch()
    assert np.allclose(M, ref * 1.5 * (1.5 * 2.0) ** 4, rtol=1e-13)   # downloaded on leaving the block


def test_what_cannot_be_captured_raises_and_leaves_a_working_runtime(gpu):
    import torch

    A = np.ones(1000)
    B = np.ones(1000)
    with pytest.raises(RuntimeError, match="cannot be captured.*host array"):
        with appy.graph():
            jacobi_step(A, B)

    @appy.jit
    def total(x):
        s = 0.0
        #pragma parallel for simd shared(s)
        for i in range(x.shape[0]):
            s += x[i]
        return s

    x = torch.ones(1000, device="cuda", dtype=torch.float64)
    assert total(x) == 1000.0
    with pytest.raises(RuntimeError, match="cannot be captured"):
        with appy.graph():
            total(x)
    with pytest.raises(RuntimeError, match="launched no kernel"):
        with appy.graph():
            pass
    with pytest.raises(RuntimeError, match="nested"):
        with appy.graph():
            with appy.graph():
                pass
    # the runtime still works eagerly afterwards
    jacobi_step(A, B)
    assert total(x) == 1000.0 and np.isclose(A[500], 0.33333 * 3 * 0.33333 * 3)


def test_replay_is_faster_than_launching_one_by_one(gpu):
    import torch

    n, steps = 4001, 200
    A = torch.rand(n, device="cuda", dtype=torch.float64)
    B = torch.rand(n, device="cuda", dtype=torch.float64)
    jacobi_step(A, B)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        jacobi_step(A, B)
    torch.cuda.synchronize()
    eager = time.perf_counter() - t0
    with appy.graph() as g:
        for _ in range(steps):
            jacobi_step(A, B)
    g.launch()
    g.synchronize()
    t0 = time.perf_counter()
    g.launch()
    g.synchronize()
    replay = time.perf_counter() - t0
    print(f"\n{2 * steps} launches: eager {eager * 1e3:.2f} ms, one graph replay {replay * 1e3:.2f} ms")
    assert replay < eager


@appy.jit
def column_sums(A, out):
    #pragma parallel for
    for j in range(A.shape[1]):
        s = 0.0
        for i in range(A.shape[0]):
            s += A[i, j]
        out[j] = s


def test_two_phase_launches_are_captured_with_both_kernels(gpu):
    """A tall matrix with few columns runs as two kernels with a scratch buffer between them;
    a captured launch replays both and keeps using the buffer it was recorded with."""
    import torch

    A = torch.rand(300_000, 24, device="cuda", dtype=torch.float64)
    out = torch.zeros(24, device="cuda", dtype=torch.float64)
    column_sums(A, out)                               # compiled and loaded before the capture
    assert torch.allclose(out, A.sum(dim=0))
    out.zero_()
    with appy.graph() as g:
        column_sums(A, out)
    assert not out.any()
    for replay in range(3):
        A.mul_(1.5)
        column_sums(A[:1000], torch.zeros_like(out))  # eager launches of the same loop in between
        g.launch()
        g.synchronize()
        assert torch.allclose(out, A.sum(dim=0)), replay


def test_loops_regenerated_on_every_call_give_their_scratch_memory_back(gpu):
    """`clear_cache=True` builds a new loop object per call; the scratch buffer of the one it
    replaces returns to the pool."""
    import ctypes

    import torch

    from appy_amd.backends.hip import runtime as rt

    fresh = appy.jit(_plain_column_sums, clear_cache=True)
    A = torch.rand(200_000, 8, device="cuda", dtype=torch.float64)
    out = torch.zeros(8, device="cuda", dtype=torch.float64)
    fresh(A, out)
    torch.cuda.synchronize()
    used, cached = ctypes.c_uint64(), ctypes.c_uint64()
    rt.check(rt.lib().appy_hip_pool_stats(ctypes.byref(used), ctypes.byref(cached)))
    held = used.value
    for _ in range(3):
        fresh(A, out)
        assert torch.allclose(out, A.sum(dim=0))
    torch.cuda.synchronize()
    rt.check(rt.lib().appy_hip_pool_stats(ctypes.byref(used), ctypes.byref(cached)))
    assert used.value == held


def _plain_column_sums(A, out):
    #pragma parallel for
    for j in range(A.shape[1]):
        s = 0.0
        for i in range(A.shape[0]):
            s += A[i, j]
        out[j] = s
