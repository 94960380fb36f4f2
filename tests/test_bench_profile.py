"""bench.py reports HBM traffic per launch from the committed counter summary
(profiles/bench_kernels_pmc_fetch_write_size.txt), and only for the kernel shape that summary was measured
with.  These checks need no GPU: every bench workload has a line, the line names the shape the launch
heuristics pick today at the bench sizes (a kernel that changed shape needs new counter runs), and the figures
are plausible against the algorithmic bytes."""
import numpy as np
import pytest

import bench
from appy_amd.backends.hip import codegen as cg
from appy_amd.backends.hip import selfcheck


class Shape:
    """Stand-in for an array argument: the launch heuristics only look at shapes."""

    def __init__(self, *shape):
        self.shape, self.ndim = tuple(shape), len(shape)


N28, N24, N27, R, M4, M5 = 1 << 28, 1 << 24, 1 << 27, 16384, 1 << 22, 1 << 20
NNZ4, NNZ5 = 16 * M4, 32 * M5
# workload -> (function, parallel iterations, scalars the bounds use, array shapes)
CASES = {
    "vector_sum": ("vector_sum", N28, {"A_shape_0": N28}, {"A": Shape(N28), "s": Shape(1)}),
    "masked_sum": ("masked_sum", N28, {"A_shape_0": N28}, {"A": Shape(N28), "M": Shape(N28), "s": Shape(1)}),
    "copy": ("copy", N28, {"a_shape_0": N28}, {"a": Shape(N28), "c": Shape(N28)}),
    "vec_add": ("vec_add", N24, {"a_shape_0": N24}, {"a": Shape(N24), "b": Shape(N24), "c": Shape(N24)}),
    "vec_add_2p27": ("vec_add", N27, {"a_shape_0": N27}, {"a": Shape(N27), "b": Shape(N27), "c": Shape(N27)}),
    "gemv": ("gemv", R, {"A_shape_0": R, "A_shape_1": R}, {"A": Shape(R, R), "x": Shape(R), "y": Shape(R)}),
    "gemv_columns": ("gemv_columns", R, {"A_shape_0": R, "A_shape_1": R}, {"A": Shape(R, R), "x": Shape(R), "y": Shape(R)}),
    "gather": ("gather_dot", 1 << 26, {"v_shape_0": 1 << 26}, {"v": Shape(1 << 26), "idx": Shape(1 << 26), "x": Shape(M4), "s": Shape(1)}),
    "spmv_uniform": ("spmv", M4, {"M": M4}, {"A_data": Shape(NNZ4), "A_indptr": Shape(M4 + 1), "A_indices": Shape(NNZ4),
                                         "x": Shape(M4), "y": Shape(M4)}),
    "spmm": ("spmm", M5, {"M": M5, "y_shape_1": 128}, {"A_data": Shape(NNZ5), "A_indptr": Shape(M5 + 1), "A_indices": Shape(NNZ5),
                                                      "B": Shape(M5, 128), "y": Shape(M5, 128)}),
}
CASES["spmv_powerlaw16"] = CASES["spmv_uniform"]
NNZ4P = 409_544_241         # Zipf(1.5) clipped at 4096 over 2^22 rows, as the bench draws it: 97.6 elements per row
CASES["spmv_powerlaw"] = ("spmv", M4, {"M": M4}, {"A_data": Shape(NNZ4P), "A_indptr": Shape(M4 + 1), "A_indices": Shape(NNZ4P),
                                            "x": Shape(M4), "y": Shape(M4)})


def loop_of(fn):
    selfcheck.compile_all_patterns()
    hits = [loop for key, (loop, _src) in cg.code_cache.items() if key[-1] == fn and loop.options.get("dry_run")]
    assert hits, fn
    return hits[-1]


def test_every_default_workload_has_a_traffic_line(monkeypatch):
    import sys

    traffic = bench.load_profile_traffic()
    monkeypatch.setattr(sys, "argv", ["bench.py"])
    wanted = bench.parse_args().workloads.split(",")
    assert sorted(wanted) == sorted(CASES)
    # (the CSR SpMV workloads have a second line each: the launches that run a kept order of the elements)
    assert sorted(traffic) == sorted(wanted + [w + "_reused" for w in wanted if w.startswith("spmv_")])


@pytest.mark.parametrize("workload", sorted(CASES))
def test_profile_was_measured_with_the_shape_the_bench_launches(workload):
    traffic = bench.load_profile_traffic()
    fn, n_outer, env, arrays = CASES[workload]
    loop = loop_of(fn)
    env = dict(env, __appy_mid=n_outer // 2)
    arrays = {k: v for k, v in arrays.items() if k in loop.analysis.arrays}
    spec = loop.choose_spec(n_outer, env, arrays)
    if workload.startswith("spmv_"):
        # launches that read the raw arrays: the elements of rows up to 512 elements are grouped by stripe
        assert spec.rows == "mixed"
        stripes, _shift, _entries = loop.grouped_shape(n_outer, env, arrays)
        spec = cg.Spec("team", block=256, vec=1, width=64, parts=stripes, aux="cells", guard=1, block_rows=256)
        # launches that run a kept order of the elements
        shape = loop.plan_shape(n_outer, env, arrays)
        kept = cg.plan_kernel_spec(shape.tile, shape.entries, n_outer)
        tag, _nbytes = traffic[workload + "_reused"]
        assert tag == kept.tag(), f"{workload}: the counter summary was measured with {tag}, a kept order runs as {kept.tag()} now"
        assert bench.load_profile_requests()[workload + "_reused"][0] == kept.tag()
        assert bench.load_profile_requests()[workload][0] == spec.tag()
    tag, nbytes = traffic[workload]
    assert tag == spec.tag(), f"{workload}: the counter summary was measured with {tag}, the launch picks {spec.tag()} now"


def test_traffic_figures_are_plausible():
    """Measured traffic is at least what the algorithm must move (minus what a cache hands back between
    launches of the small vec_add) and the summary's own algorithmic bytes equal the formulas of bench.py."""
    traffic = bench.load_profile_traffic()
    alg = {}
    with open(bench.TRAFFIC_PROFILE) as fh:
        for ln in fh:
            parts = ln.split()
            if parts[:1] == ["traffic"]:
                alg[parts[1]] = int(dict(p.split("=", 1) for p in parts[2:] if "=" in p)["algorithmic_bytes"])
    assert alg["vector_sum"] == 4 * N28 + 8 and alg["masked_sum"] == 5 * N28 + 8 and alg["copy"] == 8 * N28
    assert alg["vec_add"] == 12 * N24 and alg["gemv"] == 4 * (R * R + 2 * R)
    assert alg["spmv_uniform"] == 8 * NNZ4 + 4 * (M4 + 1) + 8 * M4
    for name, (_tag, nbytes) in traffic.items():
        assert nbytes >= 0.99 * alg[name], name
    # a kept order of the elements: 8 bytes per element and 2 per slot streamed once, the operand from the L2s, eight sums per row
    for name in ("spmv_uniform", "spmv_powerlaw", "spmv_powerlaw16"):
        assert alg[name + "_reused"] == alg[name]
        assert 1.2 * alg[name] < traffic[name + "_reused"][1] < min(2.2 * alg[name], traffic[name][1]), name
    # streams: traffic equals the algorithmic bytes to a percent; gathers: several times more
    for name in ("vector_sum", "masked_sum", "copy", "gemv", "vec_add_2p27"):
        assert traffic[name][1] <= 1.01 * alg[name], name
    assert traffic["gather"][1] > 10 * alg["gather"] and traffic["spmv_powerlaw"][1] < 4 * alg["spmv_powerlaw"]
    # rows of 16 elements grouped by column stripe: the elements are written and read once more, the gathers hit in the L2s
    assert 3 * alg["spmv_uniform"] < traffic["spmv_uniform"][1] < 5 * alg["spmv_uniform"]
    assert np.isfinite(float(traffic["spmm"][1]))
