"""Golden generated kernels: the HIP C++ text the generator emits for the six
workload loops is compared with committed snapshots (tests/golden/kernels/), so
that a change of the generated code shows up as a reviewable diff.  The
reference keeps the same kind of test for its generated Triton modules
(old-tests/codegen/triton/dry_run/test_vec_add_np.py:8-57, goldens in golden/);
set UPDATE_GOLDEN=1 to rewrite the snapshots, as there."""
import os

import pytest

from appy_amd.backends.hip import codegen as cg
from appy_amd.backends.hip import selfcheck
from appy_amd.backends.hip.kernelgen import Spec

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "kernels")

# snapshot name -> (loop (function name), the launch shape the bench workloads use)
CASES = {
    "vec_add": ("vec_add", Spec("flat", block=256, vec=4, unroll=2)),
    "vec_add_streaming": ("vec_add", Spec("flat", block=1024, vec=4, unroll=1, stream_loads=True, stream_stores=True)),
    "copy": ("copy", Spec("flat", block=512, vec=4, unroll=1, stream_loads=True, stream_stores=True)),
    "vector_sum": ("vector_sum", Spec("flat", block=512, vec=4, unroll=2, stream_loads=True)),
    "masked_sum": ("masked_sum", Spec("flat", block=512, vec=4, unroll=4, stream_loads=True)),
    "gemv": ("gemv", Spec("team", block=256, vec=4, width=32, stream_loads=True)),
    "gemv_columns": ("gemv_columns", Spec("strip", block=1024, vec=1, unroll=8, stream_loads=True)),
    # CSR rows below the size from which rows are sorted by length: one team width for all rows
    "spmv": ("spmv", Spec("team", block=256, vec=4, width=4, stream_loads=True)),
    # the five kernels of a launch with rows sorted by length (config 4)
    "spmv_bins": ("spmv", Spec("team", block=1024, vec=1, width=1, aux="bins")),
    "spmv_rows_of_all_classes": ("spmv", Spec("team", block=256, vec=4, width=64, stream_loads=True, rows="mixed")),
    "spmv_plan": ("spmv", Spec("team", block=256, vec=1, width=8, rows="list", parts=8, aux="plan")),
    "spmv_parts": ("spmv", Spec("team", block=256, vec=4, width=16, stream_loads=True, phase=1, rows="list", parts=8)),
    "spmv_fold": ("spmv", Spec("team", block=256, vec=4, width=1, stream_loads=True, phase=2, rows="list", parts=8)),
    # the kernels of a launch that groups the elements of short rows by column stripe (config 4, uniform rows)
    "spmv_group": ("spmv", Spec("team", block=256, vec=1, width=64, parts=8, aux="group", block_rows=256)),
    "spmv_group_kept_rows": ("spmv", Spec("team", block=256, vec=1, width=64, parts=8, aux="group", block_rows=256, skip_long=True)),
    "spmv_cells": ("spmv", Spec("team", block=256, vec=1, width=64, parts=8, aux="cells", block_rows=256, guard=1)),
    "spmv_sums_of_cells": ("spmv", Spec("team", block=256, vec=4, width=1, phase=2, guard=1)),
    # the kept order of the elements (row plans): the kernel that writes the pairs the inspector sorts, the kernel that runs a plan
    "spmv_plan_pairs": ("spmv", Spec("team", block=256, vec=1, width=64, aux="rkeys", block_rows=256)),
    "spmv_plan_run": ("spmv", Spec("team", block=1024, vec=1, width=1024, unroll=6, parts=8, aux="xcells")),
    "spmm": ("spmm", Spec("team", block=256, vec=4, width=32, extent=128)),
}


def kernel_text(name):
    selfcheck.compile_all_patterns()
    fn, spec = CASES[name]
    loops = [loop for key, (loop, _) in cg.code_cache.items() if key[-1] == fn]
    assert loops, name
    text = loops[-1].kernel_for(spec).src.text
    return text[text.index("// kernel for"):]


@pytest.mark.parametrize("name", sorted(CASES))
def test_generated_kernel_matches_snapshot(name):
    text = kernel_text(name)
    path = os.path.join(HERE, name + ".hip")
    if os.environ.get("UPDATE_GOLDEN") == "1":
        os.makedirs(HERE, exist_ok=True)
        with open(path, "w") as f:
            f.write(text)
    with open(path) as f:
        assert f.read() == text, f"generated kernel for {name} changed; review and rerun with UPDATE_GOLDEN=1"
