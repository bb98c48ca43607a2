"""Structure checks (bit-exact, CPU only) for the seeded generators and the golden fixtures."""
import hashlib
import os
import subprocess
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = os.path.join(ROOT, "tests", "golden")

SCALED = [("c0_uniform", 1.0), ("c1_citation", 1.0), ("c2_social", 0.02), ("c3_copurchase", 0.01),
          ("c4_rmat", 0.004)]


def check_csr_invariants(g):
    rp, col, val = g.rowptr, g.col, g.val
    assert rp.dtype == np.int32 and col.dtype == np.int32 and val.dtype == np.float32
    assert rp.shape == (g.rows + 1,) and rp[0] == 0 and rp[-1] == col.size == val.size
    deg = np.diff(rp)
    assert (deg >= 0).all()
    assert col.size == 0 or (col.min() >= 0 and col.max() < g.cols)
    # strictly increasing columns inside each row: no duplicates, sorted
    inner = np.ones(col.size, dtype=bool)
    inner[rp[:-1][deg > 0]] = False  # first entry of each row has no predecessor in the row
    assert (np.diff(col.astype(np.int64), prepend=-1)[inner] > 0).all()
    assert np.isfinite(val).all()


def pattern_is_symmetric(g):
    import scipy.sparse as sp
    A = sp.csr_matrix((np.ones(g.nnz, np.int8), g.col, g.rowptr), shape=(g.rows, g.cols))
    return (A != A.T).nnz == 0


@pytest.mark.parametrize("name,scale", SCALED)
def test_invariants(pkg, name, scale):
    g = pkg.graphs.make_graph(name, scale)
    check_csr_invariants(g)
    if name != "c0_uniform":
        assert g.rows == g.cols and pattern_is_symmetric(g)


def test_c0_shape(pkg):
    g = pkg.graphs.make_graph("c0_uniform")
    assert (g.rows, g.cols, g.nnz) == (4096, 4096, 65536)
    assert (np.diff(g.rowptr) == 16).all()
    assert g.val.min() >= -1 and g.val.max() < 1 and abs(float(g.val.mean())) < 0.02
    # uniformly placed columns: every column hit about 16 times
    hits = np.bincount(g.col, minlength=4096)
    assert hits.min() >= 1 and hits.max() < 50
    B = pkg.graphs.make_dense("c0_uniform", 4096, 32)
    assert abs(float(B.mean())) < 0.01 and abs(float(B.std()) - 1) < 0.01


def test_c1_citation_properties(pkg):
    g = pkg.graphs.make_graph("c1_citation")
    st = pkg.graphs.degree_stats(g.rowptr)
    assert g.rows == 20000 and 4.5 < st["mean_degree"] < 5.5 and 120 <= st["max_degree"] <= 230
    assert st["empty_row_fraction"] == 0.0
    deg = np.diff(g.rowptr)
    rows = np.repeat(np.arange(g.rows), deg)
    assert np.array_equal(np.unique(rows[rows == g.col]), np.arange(g.rows)), "self-loop on every vertex"
    np.testing.assert_array_equal(g.val, (1.0 / deg[rows]).astype(np.float32))
    np.testing.assert_allclose(np.add.reduceat(g.val.astype(np.float64), g.rowptr[:-1]), 1.0, atol=1e-5)


def test_scaled_families_have_their_character(pkg):
    graphs = pkg.graphs
    g = graphs.make_graph("c2_social", 0.05)
    st = graphs.degree_stats(g.rowptr)
    assert st["max_degree"] > 10 * st["mean_degree"] and st["cv"] > 1.2
    assert g.val.min() >= 0 and g.val.max() < 1
    g = graphs.make_graph("c4_rmat", 0.01)
    st = graphs.degree_stats(g.rowptr)
    assert st["empty_row_fraction"] > 0.15 and st["max_degree"] > 100 * st["mean_degree"]
    assert g.val.min() >= -1 and g.val.max() < 1
    g = graphs.make_graph("c3_copurchase", 0.01)
    st = graphs.degree_stats(g.rowptr)
    assert 35 < st["mean_degree"] < 65 and 0.5 < st["cv"] < 1.2


HELD_OUT_SCALE = 0.004  # about 4e5 nonzeros each


@pytest.mark.parametrize("name", ["h1_prefattach", "h2_rmat", "h3_grid", "h4_bipartite", "h5_blocks", "h6_uniform100",
                                  "h7_groups"])
def test_held_out_families(pkg, name):
    """The families the plan's choice is checked on: valid CSR, sorted rows without duplicates, the same
    matrix from the same name and scale, and the property each one is there for."""
    graphs = pkg.graphs
    assert name in graphs.HELD_OUT
    g = graphs.make_graph(name, HELD_OUT_SCALE)
    check_csr_invariants(g)
    assert _digest(g) == _digest(graphs.make_graph(name, HELD_OUT_SCALE))
    assert 3.0e5 <= g.nnz <= 4.5e5
    deg = np.diff(g.rowptr)
    if name == "h1_prefattach":      # 24 edges per new vertex, both directions stored; a few hubs
        assert g.rows == g.cols and pattern_is_symmetric(g)
        assert deg.min() >= 20 and 40 < deg.mean() < 50 and deg.max() > 20 * deg.mean()
    elif name == "h2_rmat":           # 2^n vertices, skewed rows, some without any entry
        assert g.rows == g.cols and g.rows & (g.rows - 1) == 0 and pattern_is_symmetric(g)
        assert deg.max() > 20 * deg.mean() and (deg == 0).any()
    elif name == "h3_grid":           # 9-point mesh + 2 long-range entries per row: near-constant short rows
        side = int(round(g.rows ** 0.5))
        assert side * side == g.rows == g.cols and pattern_is_symmetric(g)
        assert 12.5 < deg.mean() < 13.5 and deg.max() <= 25
        r = np.repeat(np.arange(g.rows), deg)
        near = np.abs(g.col.astype(np.int64) - r) <= side + 1
        assert 0.6 < near.mean() < 0.75   # the mesh neighbours lie within one mesh row of the diagonal
    elif name == "h4_bipartite":      # users x items, 8 : 1, popular items
        assert g.rows > 8 * g.cols * 0.95 and g.rows < 8 * g.cols * 1.1
        hits = np.sort(np.bincount(g.col, minlength=g.cols))[::-1]
        assert hits[: g.cols // 100].sum() > 0.05 * g.nnz      # the top 1 % of the items take > 5 % of the entries
        assert deg.max() > 4 * deg.mean()
    elif name == "h5_blocks":         # most entries inside diagonal blocks of mixed sizes
        assert g.rows == g.cols and pattern_is_symmetric(g)
        r = np.repeat(np.arange(g.rows), deg)
        assert (np.abs(g.col.astype(np.int64) - r) < 4096).mean() > 0.85
    elif name == "h7_groups":         # users x items 1 : 2 out of a community graph: the rows kept are the first half
        assert g.cols == 2 * g.rows and 55 < deg.mean() < 75
        import scipy.sparse as sp
        A = sp.csr_matrix((np.ones(g.nnz, np.float32), g.col, g.rowptr), shape=(g.rows, g.cols))
        square = A[:, : g.rows]       # the kept rows against their own vertices: still a symmetric pattern
        assert (square != square.T).nnz == 0
        common = (A[:64] @ A.T).toarray()           # items shared between 64 users and all users
        np.fill_diagonal(common[:, :64], 0)
        assert (common.max(axis=1) >= 5).mean() > 0.8   # most users share several items with some other user
    else:                             # exactly 100 entries in every row, anywhere
        assert (deg == 100).all()
        assert np.bincount(g.col, minlength=g.cols).max() < 200


def test_values_symmetric(pkg):
    import scipy.sparse as sp
    g = pkg.graphs.make_graph("c4_rmat", 0.002)
    A = sp.csr_matrix((g.val, g.col, g.rowptr), shape=(g.rows, g.cols))
    assert abs(A - A.T).max() == 0


def _digest(g):
    h = hashlib.sha256()
    for a in (g.rowptr, g.col, g.val):
        h.update(np.ascontiguousarray(a).tobytes())
    return h.hexdigest()


def test_reproducible_and_thread_count_independent(pkg):
    g1 = pkg.graphs.make_graph("c3_copurchase", 0.004)
    g2 = pkg.graphs.make_graph("c3_copurchase", 0.004)
    assert _digest(g1) == _digest(g2)
    code = ("import importlib,sys,hashlib,numpy as np; sys.path.insert(0, %r); "
            "gr=importlib.import_module('hp-spmm-sddmm_amd.graphs'); g=gr.make_graph('c3_copurchase',0.004); "
            "h=hashlib.sha256(); [h.update(np.ascontiguousarray(a).tobytes()) for a in (g.rowptr,g.col,g.val)]; "
            "B=gr.make_dense('c3_copurchase', 100, 64); h.update(B.tobytes()); print(h.hexdigest())" % ROOT)
    outs = []
    for threads in ("1", "3"):
        env = dict(os.environ, OMP_NUM_THREADS=threads)
        outs.append(subprocess.check_output([sys.executable, "-c", code], env=env).decode().strip())
    assert outs[0] == outs[1]


@pytest.mark.parametrize("fixture,maker", [
    ("c0_uniform_k32.npz", lambda gr: (gr.make_graph("c0_uniform"), 32, "c0_uniform")),
    ("c1_citation_small_k64.npz", lambda gr: (gr.make_graph("c1_citation", 0.05), 64, "c1_citation")),
])
def test_generators_reproduce_golden_inputs(pkg, fixture, maker):
    """The committed fixtures pin the generators: same seed, same bits."""
    z = np.load(os.path.join(GOLDEN, fixture))
    g, k, name = maker(pkg.graphs)
    assert np.array_equal(g.rowptr, z["rowptr"]) and np.array_equal(g.col, z["col"])
    assert np.array_equal(g.val, z["val"])
    assert np.array_equal(pkg.graphs.make_dense(name, g.cols, k), z["B"])


def test_dense_generators(pkg):
    B = pkg.graphs.dense_normal(5000, 64, 9)
    assert B.shape == (5000, 64) and B.dtype == np.float32
    assert abs(float(B.mean())) < 0.01 and abs(float(B.std()) - 1.0) < 0.01
    # odd element count: last element still written
    odd = pkg.graphs.dense_normal(3, 1, 9)
    assert np.isfinite(odd).all()
    U = pkg.graphs.dense_uniform(5000, 32, 9)  # the reference's rand(-1, 1) operand
    assert U.min() >= -1 and U.max() < 1 and abs(float(U.mean())) < 0.01


def test_bad_arguments(pkg):
    with pytest.raises(ValueError):
        pkg.graphs.uniform_rows(4, 4, 5, 0)  # more nonzeros per row than columns
    with pytest.raises(ValueError):
        pkg.graphs.rmat(0, 10, 0.5, 0.2, 0.2, 0)
