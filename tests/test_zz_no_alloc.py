"""``appy_hip_launch_static_scratch``: the launch entry point that allocates nothing.

The two kernels of a two-phase column reduction (partial sums of the parts of a strip in a scratch
buffer, then a finishing kernel) are launched through the C ABI twice: with a scratch buffer from the
library's allocator through ``appy_hip_launch`` (the existing entry point), and with the library's
static per-GPU scratch buffer through ``appy_hip_launch_static_scratch``.  The results must be equal
bit for bit, on two calls in a row, the second on a smaller input (the static buffer still holds the
first call's partial results).  Collected last (file name) so that a failure here hides no other test."""
import ctypes as C

import numpy as np
import pytest

import appy_amd as appy
from appy_amd.backends.hip import codegen as cg
from appy_amd.backends.hip import runtime as rt

pytestmark = pytest.mark.gpu


@appy.jit
def column_dot(A, y, x):
    #pragma parallel for
    for j in range(A.shape[1]):
        s = 0.0
        #pragma simd
        for i in range(A.shape[0]):
            s += A[i, j] * y[i]
        x[j] = s


def _staged(A, y, x):
    """The staged two-phase launch of `column_dot` on GPU tensors (nothing is launched here)."""
    column_dot(A[:64], y[:64], x)               # compiles the loop
    loop = [v[0] for kk, v in cg.code_cache.items() if kk[-1] == "column_dot"][-1]
    launch = loop.prepare({"A": A, "y": y, "x": x, "A_shape_0": A.shape[0], "A_shape_1": A.shape[1]})
    assert launch.spec.phase == 1 and launch.second is not None
    return launch


def _scratch_field(kernel):
    return next(f for f, p in zip(kernel._field_names, kernel.src.params) if p.role == "scratch")


def _pool_bytes():
    used, cached = C.c_uint64(), C.c_uint64()
    rt.check(rt.lib().appy_hip_pool_stats(C.byref(used), C.byref(cached)))
    return used.value + cached.value


def _run_both_ways(shape, seed):
    import torch

    rng = np.random.default_rng(seed)
    A = torch.from_numpy(rng.standard_normal(shape, dtype=np.float32)).cuda()
    y = torch.from_numpy(rng.standard_normal(shape[0], dtype=np.float32)).cuda()
    x_ref = torch.full((shape[1],), float("nan"), dtype=torch.float32, device="cuda")
    x_new = torch.full((shape[1],), float("nan"), dtype=torch.float32, device="cuda")

    # the existing entry point: scratch from the library's allocator (staged by the launcher)
    ref = _staged(A, y, x_ref)
    ref.launch_only()
    fin, fin_args, fin_grid, fin_block = ref.second

    # the new entry point: the same kernels and argument blocks, the scratch pointer left NULL by the
    # caller and filled in by the library with its static buffer
    new = _staged(A, y, x_new)
    nbytes = 8 * new.nsplit * shape[1] * max(1, len(new.loop.analysis.strip[id(new.loop.analysis.strip_split)]))
    assert 0 < nbytes <= rt.STATIC_SCRATCH_BYTES
    first_field, second_field = _scratch_field(new.kernel), _scratch_field(new.second[0])
    setattr(new.args, first_field, None)
    setattr(new.second[1], second_field, None)
    before = _pool_bytes()
    rt.launch_static_scratch(new.function(), new.grid, new.block, new.args, first_field, nbytes, new.stream)
    rt.launch_static_scratch(new.second[0].function(new.device), new.second[2], new.second[3], new.second[1],
                             second_field, nbytes, new.stream)
    assert _pool_bytes() == before          # nothing came from, or went back to, the allocator
    torch.cuda.synchronize()
    got, want = x_new.cpu().numpy(), x_ref.cpu().numpy()
    assert not np.isnan(want).any()
    assert np.array_equal(got, want), np.abs(got - want).max()
    # and the result itself is right
    exact = A.cpu().numpy().astype(np.float64).T @ y.cpu().numpy().astype(np.float64)
    budget = np.abs(A.cpu().numpy().astype(np.float64)).T @ np.abs(y.cpu().numpy().astype(np.float64))
    assert np.all(np.abs(got - exact) <= 1e-5 * budget)


def test_static_scratch_launches_equal_allocated_scratch_launches_twice_in_a_row(gpu):
    _run_both_ways((300_000, 64), seed=1)
    _run_both_ways((120_001, 40), seed=2)        # smaller: the buffer still holds the first call's partial sums


def test_requests_beyond_the_static_buffer_are_refused(gpu):
    import torch

    A = torch.zeros((200_000, 64), dtype=torch.float32, device="cuda")
    y = torch.zeros(200_000, dtype=torch.float32, device="cuda")
    x = torch.zeros(64, dtype=torch.float32, device="cuda")
    launch = _staged(A, y, x)
    field = _scratch_field(launch.kernel)
    with pytest.raises(rt.HipError, match="APPY_HIP_STATIC_SCRATCH_BYTES"):
        rt.launch_static_scratch(launch.function(), launch.grid, launch.block, launch.args, field,
                                 rt.STATIC_SCRATCH_BYTES + 1, launch.stream)
    off = getattr(type(launch.args), field).offset
    lib = rt.lib()
    g, b = launch.grid, launch.block
    # an offset that is not a pointer slot of the block
    assert lib.appy_hip_launch_static_scratch(launch.function(), g[0], 1, 1, b[0], 1, 1, 0, None, C.byref(launch.args),
                                              C.sizeof(launch.args), off + 4, 64) != 0
    assert lib.appy_hip_launch_static_scratch(launch.function(), g[0], 1, 1, b[0], 1, 1, 0, None, C.byref(launch.args),
                                              C.sizeof(launch.args), C.sizeof(launch.args), 64) != 0
    assert lib.appy_hip_launch_static_scratch(None, 1, 1, 1, 64, 1, 1, 0, None, C.byref(launch.args),
                                              C.sizeof(launch.args), off, 64) != 0
    # offsets near the top of the address range, which wrap around when the size of a pointer is added to them
    for wrap in (2 ** 64 - 8, 2 ** 64 - 16):
        assert lib.appy_hip_launch_static_scratch(launch.function(), g[0], 1, 1, b[0], 1, 1, 0, None, C.byref(launch.args),
                                                  C.sizeof(launch.args), C.c_size_t(wrap), 64) != 0
