"""Seeded synthetic inputs for the SpMM benchmark configurations.

Thin ctypes binding of csrc/graphgen.cpp plus the table of benchmark
configurations.  The reference has no generators (its inputs are downloaded
.smtx files, dataset/download.sh, and an unseeded dense operand,
test/test_all.cpp:53); these replace them with reproducible ones.
"""
import ctypes
import os
from dataclasses import dataclass

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libhpspmm_graphgen.so")
_lib = None

_i64 = ctypes.c_int64
_u64 = ctypes.c_uint64
_dbl = ctypes.c_double
_p = ctypes.c_void_p

VAL_SYM_UNIFORM_PM1 = 0
VAL_SYM_UNIFORM_01 = 1
VAL_ROW_NORMALISED = 2
VAL_ONES = 3


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise RuntimeError(
                f"{_LIB_PATH} is missing: run `python -c 'import __graft_entry__ as g; g.build()'` "
                "(or hp-spmm-sddmm_amd/build.py) first")
        L = ctypes.CDLL(_LIB_PATH)
        L.hpspmm_gen_last_error.restype = ctypes.c_char_p
        for name in ("rows", "cols", "nnz"):
            f = getattr(L, f"hpspmm_graph_{name}")
            f.argtypes, f.restype = [_p], _i64
        for name in ("rowptr", "col", "val"):
            f = getattr(L, f"hpspmm_graph_{name}")
            f.argtypes, f.restype = [_p], _p
        L.hpspmm_graph_free.argtypes = [_p]
        L.hpspmm_gen_uniform_rows.argtypes, L.hpspmm_gen_uniform_rows.restype = [_i64, _i64, _i64, _u64], _p
        L.hpspmm_gen_citation.argtypes, L.hpspmm_gen_citation.restype = [_i64, _dbl, _i64, _i64, _u64], _p
        L.hpspmm_gen_powerlaw.argtypes = [_i64, _dbl, _dbl, _i64, ctypes.c_int, _u64]
        L.hpspmm_gen_powerlaw.restype = _p
        L.hpspmm_gen_community.argtypes = [_i64, _dbl, _dbl, _i64, _dbl, _i64, _u64]
        L.hpspmm_gen_community.restype = _p
        L.hpspmm_gen_rmat.argtypes, L.hpspmm_gen_rmat.restype = [ctypes.c_int, _i64, _dbl, _dbl, _dbl, _u64], _p
        L.hpspmm_gen_named.argtypes, L.hpspmm_gen_named.restype = [ctypes.c_char_p, _dbl], _p
        L.hpspmm_gen_dense_normal.argtypes = [_u64, _i64, _p]
        L.hpspmm_gen_dense_uniform.argtypes = [_u64, _i64, ctypes.c_float, ctypes.c_float, _p]
        _lib = L
    return _lib


@dataclass
class CSR:
    """Host CSR: int32 rowptr[rows+1], int32 col[nnz], float32 val[nnz]."""
    rows: int
    cols: int
    rowptr: np.ndarray
    col: np.ndarray
    val: np.ndarray

    @property
    def nnz(self):
        return int(self.col.shape[0])


def _take(handle):
    L = lib()
    if not handle:
        raise ValueError(L.hpspmm_gen_last_error().decode())
    try:
        rows, cols, nnz = (L.hpspmm_graph_rows(handle), L.hpspmm_graph_cols(handle),
                           L.hpspmm_graph_nnz(handle))

        def arr(ptr, n, dt):
            out = np.empty(n, dtype=dt)
            if n:
                ctypes.memmove(out.ctypes.data, ptr, n * out.itemsize)
            return out

        return CSR(rows, cols,
                   arr(L.hpspmm_graph_rowptr(handle), rows + 1, np.int32),
                   arr(L.hpspmm_graph_col(handle), nnz, np.int32),
                   arr(L.hpspmm_graph_val(handle), nnz, np.float32))
    finally:
        L.hpspmm_graph_free(handle)


def uniform_rows(rows, cols, nnz_per_row, seed):
    return _take(lib().hpspmm_gen_uniform_rows(rows, cols, nnz_per_row, seed))


def citation(n, alpha, wmax, n_edges, seed):
    return _take(lib().hpspmm_gen_citation(n, alpha, wmax, n_edges, seed))


def powerlaw(n, gamma, i0, n_edges, seed, value_mode=VAL_SYM_UNIFORM_01):
    return _take(lib().hpspmm_gen_powerlaw(n, gamma, i0, n_edges, value_mode, seed))


def community(n, mu, sigma, n_comm, p_intra, n_edges, seed):
    return _take(lib().hpspmm_gen_community(n, mu, sigma, n_comm, p_intra, n_edges, seed))


def rmat(scale, n_edges, a, b, c, seed):
    return _take(lib().hpspmm_gen_rmat(scale, n_edges, a, b, c, seed))


def dense_normal(rows, k, seed):
    """rows x k float32 N(0,1), row-major."""
    out = np.empty((rows, k), dtype=np.float32)
    lib().hpspmm_gen_dense_normal(seed, rows * k, out.ctypes.data_as(_p))
    return out


def dense_uniform(rows, k, seed, lo=-1.0, hi=1.0):
    """rows x k float32 U(lo,hi): the distribution of the reference's rand() operand."""
    out = np.empty((rows, k), dtype=np.float32)
    lib().hpspmm_gen_dense_uniform(seed, rows * k, lo, hi, out.ctypes.data_as(_p))
    return out


# --------------------------------------------------------------------------
# Benchmark configurations.  `scale` < 1 shrinks vertex and edge counts
# together (tests use that); scale = 1 is the benchmark size.
# --------------------------------------------------------------------------

CONFIG_K = {
    "c0_uniform": (32,),
    "c1_citation": (32, 64, 128),
    "c2_social": (32, 64, 128),
    "c3_copurchase": (64,),
    "c4_rmat": (128,),
}
CONFIG_SEED = {"c0_uniform": 0, "c1_citation": 1, "c2_social": 2, "c3_copurchase": 3, "c4_rmat": 4,
               "h1_prefattach": 11, "h2_rmat": 12, "h3_grid": 13, "h4_bipartite": 14, "h5_blocks": 15,
               "h6_uniform100": 16, "h7_groups": 17}
# Families none of the library's thresholds was chosen on (scale 1 = about 10^8 nonzeros): they check
# that the plan's choice of strategy holds up on matrices unlike the benchmark's four.
HELD_OUT = ("h1_prefattach", "h2_rmat", "h3_grid", "h4_bipartite", "h5_blocks", "h6_uniform100", "h7_groups")


def make_graph(name, scale=1.0):
    """Build the sparse operand of a named benchmark configuration (parameters live in
    hpspmm_gen_named, csrc/graphgen.cpp, shared with the C++ host layer)."""
    if name not in CONFIG_SEED:
        raise KeyError(name)
    return _take(lib().hpspmm_gen_named(name.encode(), float(scale)))


def make_dense(name, rows, k):
    """The dense operand B (rows x k, N(0,1)) of a named configuration."""
    return dense_normal(rows, k, CONFIG_SEED[name] + 1000 * k)


def degree_stats(rowptr):
    """rows, nnz, mean / max degree, empty-row fraction and row-length CV
    (population sigma / mean, the statistic of spmm/mm/spmm_common.cpp:311-321)."""
    deg = np.diff(rowptr.astype(np.int64))
    mean = float(deg.mean()) if deg.size else 0.0
    return {
        "rows": int(deg.size),
        "nnz": int(deg.sum()),
        "mean_degree": mean,
        "max_degree": int(deg.max()) if deg.size else 0,
        "empty_row_fraction": float((deg == 0).mean()) if deg.size else 0.0,
        "cv": float(deg.std() / mean) if mean > 0 else 0.0,
    }
