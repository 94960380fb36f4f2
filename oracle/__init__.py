"""CPU oracle for the annotated-loop hot path.  TEST INFRASTRUCTURE ONLY.

Nothing under ``appy_amd/`` imports this package: it is used by ``tests/``,
by ``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of ``bench.py``
as the checker, never as the thing that is measured as the product or shipped.

The reference has no compiled component on this path; its CPU path is the
annotated function run by the Python interpreter with the pragmas read as
comments ("Comment this line to run the function in the Python interpreter",
reference tree: examples/02-vec_sum.py:5; the ``dry_run`` switch,
appy/dispatcher.py:46-53).  The oracle therefore has two layers:

``loops``      the reference's loop bodies, literally (examples/01..06), for
               small inputs;
``vectorised`` float64 NumPy/SciPy restatements of the same loops for full
               sizes, with the per-output error budget sum(|terms|).

Parity status per function (what pins it is in tests/test_oracle.py):

=================  ==========================================================
vec_add            pinned: IEEE-754 addition is its own definition; literal
                   loop; commutativity; a + 0 = a
vector_sum         pinned: literal loop, math.fsum, closed form sum(1..n)
masked_sum         pinned: literal loops (both source forms), all-true /
                   all-false masks, complement identity
gemv               pinned: literal loop, unit vectors select columns,
                   identity matrix, linearity
spmv_csr           pinned: literal loop, dense matmul of the same matrix,
                   SciPy's CSR product (the reference's own test oracle,
                   tests/integration/triton/tutorial/test_spmv.py:24-30),
                   empty rows, identity
spmm_csr           pinned: literal loop, column-wise equality with spmv_csr,
                   dense matmul
=================  ==========================================================

The reference holds no golden vectors for this path (its tests draw unseeded
random inputs); tests/golden/ holds small seeded inputs with the float64
results of this oracle so that runs on the GPU box need no reference files.
"""
from . import loops, vectorised, workloads  # noqa: F401
