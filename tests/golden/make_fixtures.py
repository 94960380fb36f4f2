"""Writes tests/golden/*.npz: small seeded inputs for each loop pattern with the
float64 results of the CPU oracle (oracle/vectorised.py) and the error budgets.

The reference holds no golden vectors for this path (its tests draw unseeded
random inputs and compare with NumPy at run time), and it cannot be imported
in the build container (missing third-party packages), so these vectors come
from the oracle, which tests/test_oracle.py pins independently.  Run from the
repository root:  python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import vectorised as vo  # noqa: E402
from oracle import workloads as wl  # noqa: E402


def main():
    a, b = wl.vec_add(1537, seed=11)
    np.savez_compressed(os.path.join(HERE, "vec_add.npz"), a=a, b=b, c=vo.vec_add(a, b))

    A, M = wl.reduce_inputs(5003, seed=12)
    s, sb = vo.vector_sum(A)
    m, mb = vo.masked_sum(A, M)
    np.savez_compressed(os.path.join(HERE, "reductions.npz"), A=A, M=M, vector_sum=s, vector_sum_budget=sb,
                        masked_sum=m, masked_sum_budget=mb)

    Am, x = wl.gemv(61, 259, seed=13)
    y, yb = vo.gemv(Am, x)
    np.savez_compressed(os.path.join(HERE, "gemv.npz"), A=Am, x=x, y=y, budget=yb)

    data, indptr, indices, xs = wl.spmv_powerlaw(257, 300, clip=96, seed=14)
    y, yb = vo.spmv_csr(data, indptr, indices, xs, (257, 300))
    np.savez_compressed(os.path.join(HERE, "spmv.npz"), data=data, indptr=indptr, indices=indices, x=xs, y=y, budget=yb)

    data, indptr, indices, B = wl.spmm(129, 140, 128, mean_row=12, seed=15)
    C, Cb = vo.spmm_csr(data, indptr, indices, B, (129, 140))
    np.savez_compressed(os.path.join(HERE, "spmm.npz"), data=data, indptr=indptr, indices=indices, B=B, C=C, budget=Cb)


if __name__ == "__main__":
    main()
