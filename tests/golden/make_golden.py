"""Writes the golden fixtures in this directory.

    python tests/golden/make_golden.py

The sparse operands come from this repository's own seeded generators; the
expected products are computed here with scipy.sparse in float64 (a stock
library, independent of the oracle and of the HIP path).  The reference
repository holds no golden vectors for SpMM (its check, compiled out by
default, compares against cuSPARSE at run time), so these fixtures are what the
oracle is pinned to.
"""
import importlib
import os
import sys

import numpy as np
import scipy.sparse as sp

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)


def product_f64(g, B):
    A = sp.csr_matrix((g.val.astype(np.float64), g.col, g.rowptr), shape=(g.rows, g.cols))
    return A @ B.astype(np.float64)


def main():
    graphs = importlib.import_module("hp-spmm-sddmm_amd.graphs")

    # configuration 0: 4096 x 4096, 16 nnz/row, K = 32, seed 0 (whole)
    g = graphs.make_graph("c0_uniform")
    B = graphs.make_dense("c0_uniform", g.cols, 32)
    np.savez_compressed(os.path.join(HERE, "c0_uniform_k32.npz"), rowptr=g.rowptr, col=g.col, val=g.val,
                        B=B, C64=product_f64(g, B))

    # configuration 1 at 1/20 size (1000 vertices), K = 64
    g = graphs.make_graph("c1_citation", 0.05)
    B = graphs.make_dense("c1_citation", g.cols, 64)
    np.savez_compressed(os.path.join(HERE, "c1_citation_small_k64.npz"), rowptr=g.rowptr, col=g.col,
                        val=g.val, B=B, C64=product_f64(g, B))

    # R-MAT scale 9: empty rows and hub rows, K = 128
    g = graphs.rmat(9, 16 << 9, 0.57, 0.19, 0.19, 4)
    B = graphs.dense_normal(g.cols, 128, 4128)
    np.savez_compressed(os.path.join(HERE, "rmat9_k128.npz"), rowptr=g.rowptr, col=g.col, val=g.val,
                        B=B, C64=product_f64(g, B))
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)))


if __name__ == "__main__":
    main()
