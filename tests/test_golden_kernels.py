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

# loop (function name) -> the launch shape the bench workloads use
CASES = {
    "vec_add": Spec("flat", block=256, vec=4, unroll=2),
    "copy": Spec("flat", block=256, vec=4, unroll=1, stream_loads=True, stream_stores=True),
    "vector_sum": Spec("flat", block=256, vec=4, unroll=2, stream_loads=True),
    "masked_sum": Spec("flat", block=256, vec=4, unroll=2, stream_loads=True),
    "gemv": Spec("team", block=256, vec=4, width=32, stream_loads=True),
    "gemv_columns": Spec("strip", block=1024, vec=1, unroll=8, stream_loads=True),
    "spmv": Spec("team", block=256, vec=4, width=4, stream_loads=True),
    "spmm": Spec("team", block=256, vec=4, width=32, extent=128),
}


def kernel_text(name):
    selfcheck.compile_all_patterns()
    loops = [loop for key, (loop, _) in cg.code_cache.items() if key[-1] == name]
    assert loops, name
    text = loops[-1].kernel_for(CASES[name]).src.text
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
