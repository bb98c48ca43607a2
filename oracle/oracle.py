"""ctypes binding of the CPU oracle (oracle/spmm_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
the cpu_baseline leg of bench.py, always as the checker and never as the thing
that is measured or shipped.  The product package must not import this module.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle_spmm.so")
_lib = None

_i64 = ctypes.c_int64
_p = ctypes.c_void_p


def build(force=False):
    """Compile the oracle with gcc (host code only)."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _HERE], stdout=subprocess.DEVNULL)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        L.oracle_num_threads.restype = ctypes.c_int
        L.oracle_csr_spmm_f32.argtypes = [_i64, _i64, _p, _p, _p, _p, _p]
        L.oracle_csr_spmm_f32_rows.argtypes = [_i64, _i64, _i64, _p, _p, _p, _p, _p]
        L.oracle_csr_spmm_f64.argtypes = [_i64, _i64, _p, _p, _p, _p, _p, _p]
        L.oracle_csr_spmm_f64_rows.argtypes = [_i64, _i64, _i64, _p, _p, _p, _p, _p, _p]
        L.oracle_coo_spmm_acc_f32.argtypes = [_i64, _i64, _p, _p, _p, _p, _p]
        L.oracle_csr_to_dense.argtypes = [_i64, _i64, _p, _p, _p, _p]
        L.oracle_max_abs_err.argtypes = [_i64, _p, _p, ctypes.c_float]
        L.oracle_max_abs_err.restype = ctypes.c_float
        L.oracle_max_norm_err.argtypes = [_i64, _p, _p, _p, _p]
        L.oracle_max_norm_err.restype = ctypes.c_double
        L.oracle_row_length_cv.argtypes = [_i64, _p]
        L.oracle_row_length_cv.restype = ctypes.c_double
        _lib = L
    return _lib


def _c(a, dtype):
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def num_threads():
    return int(lib().oracle_num_threads())


def _check_csr(rowptr, col, val, B):
    M = rowptr.shape[0] - 1
    nnz = int(rowptr[-1]) if M >= 0 else 0
    assert rowptr[0] == 0 and col.shape[0] == nnz and val.shape[0] == nnz
    assert B.ndim == 2
    if nnz:
        assert 0 <= int(col.min()) and int(col.max()) < B.shape[0]
    return M, nnz


def csr_spmm_f32(rowptr, col, val, B):
    """C = A @ B in FP32, sequential per-row accumulation in stored order."""
    rowptr, col = _c(rowptr, np.int32), _c(col, np.int32)
    val, B = _c(val, np.float32), _c(B, np.float32)
    M, _ = _check_csr(rowptr, col, val, B)
    K = B.shape[1]
    C = np.empty((M, K), dtype=np.float32)
    lib().oracle_csr_spmm_f32(M, K, _ptr(rowptr), _ptr(col), _ptr(val), _ptr(B), _ptr(C))
    return C


def csr_spmm_f32_rows(rowptr, col, val, B, row_begin, row_end, out=None):
    """Rows [row_begin, row_end) of C = A @ B; returns the (row_end-row_begin, K) slab."""
    rowptr, col = _c(rowptr, np.int32), _c(col, np.int32)
    val, B = _c(val, np.float32), _c(B, np.float32)
    K = B.shape[1]
    n = row_end - row_begin
    slab = out if out is not None else np.empty((n, K), dtype=np.float32)
    # the C entry indexes C by absolute row: offset the base pointer back
    base = slab.ctypes.data - row_begin * K * 4
    lib().oracle_csr_spmm_f32_rows(row_begin, row_end, K, _ptr(rowptr), _ptr(col), _ptr(val),
                                   _ptr(B), ctypes.c_void_p(base))
    return slab


def csr_spmm_f64(rowptr, col, val, B, want_abs=True):
    """(C64, S64): float64 accumulation and S = |A| @ |B| (the error denominator)."""
    rowptr, col = _c(rowptr, np.int32), _c(col, np.int32)
    val, B = _c(val, np.float32), _c(B, np.float32)
    M, _ = _check_csr(rowptr, col, val, B)
    K = B.shape[1]
    C = np.empty((M, K), dtype=np.float64)
    S = np.empty((M, K), dtype=np.float64) if want_abs else None
    lib().oracle_csr_spmm_f64(M, K, _ptr(rowptr), _ptr(col), _ptr(val), _ptr(B), _ptr(C),
                              _ptr(S) if want_abs else None)
    return C, S


def csr_spmm_f64_rows(rowptr, col, val, B, row_begin, row_end):
    rowptr, col = _c(rowptr, np.int32), _c(col, np.int32)
    val, B = _c(val, np.float32), _c(B, np.float32)
    K = B.shape[1]
    n = row_end - row_begin
    C = np.empty((n, K), dtype=np.float64)
    S = np.empty((n, K), dtype=np.float64)
    off = row_begin * K * 8
    lib().oracle_csr_spmm_f64_rows(row_begin, row_end, K, _ptr(rowptr), _ptr(col), _ptr(val),
                                   _ptr(B), ctypes.c_void_p(C.ctypes.data - off),
                                   ctypes.c_void_p(S.ctypes.data - off))
    return C, S


def coo_spmm_acc_f32(row, col, val, B, C):
    """C += A @ B for COO A, entries in stored order; C is modified in place."""
    row, col = _c(row, np.int32), _c(col, np.int32)
    val, B = _c(val, np.float32), _c(B, np.float32)
    assert C.dtype == np.float32 and C.flags.c_contiguous and C.shape[1] == B.shape[1]
    nnz = row.shape[0]
    assert col.shape[0] == nnz and val.shape[0] == nnz
    if nnz:
        assert 0 <= int(row.min()) and int(row.max()) < C.shape[0]
        assert 0 <= int(col.min()) and int(col.max()) < B.shape[0]
    lib().oracle_coo_spmm_acc_f32(nnz, B.shape[1], _ptr(row), _ptr(col), _ptr(val), _ptr(B), _ptr(C))
    return C


def csr_to_dense(rowptr, col, val, N):
    rowptr, col, val = _c(rowptr, np.int32), _c(col, np.int32), _c(val, np.float32)
    M = rowptr.shape[0] - 1
    D = np.empty((M, N), dtype=np.float32)
    lib().oracle_csr_to_dense(M, N, _ptr(rowptr), _ptr(col), _ptr(val), _ptr(D))
    return D


def max_abs_err(x, y, div=1.0):
    x, y = _c(x, np.float32).ravel(), _c(y, np.float32).ravel()
    assert x.shape == y.shape
    return float(lib().oracle_max_abs_err(x.shape[0], _ptr(x), _ptr(y), ctypes.c_float(div)))


def max_norm_err(got, C64, S64):
    """max |got - C64| / S64 (exact-zero required where S64 == 0); returns (err, argmax)."""
    got = _c(got, np.float32).ravel()
    C64, S64 = _c(C64, np.float64).ravel(), _c(S64, np.float64).ravel()
    assert got.shape == C64.shape == S64.shape
    pos = ctypes.c_int64(-1)
    e = lib().oracle_max_norm_err(got.shape[0], _ptr(got), _ptr(C64), _ptr(S64), ctypes.byref(pos))
    return float(e), int(pos.value)


def row_length_cv(rowptr):
    rowptr = _c(rowptr, np.int32)
    return float(lib().oracle_row_length_cv(rowptr.shape[0] - 1, _ptr(rowptr)))
