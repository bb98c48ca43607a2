"""Pins the CPU oracle (oracle/spmm_oracle.c) without any GPU.

The reference has no golden vectors, known-answer tests or CPU SpMM, so the
oracle is pinned by: scipy float64 products committed under tests/golden,
dense brute force on small inputs, closed forms, an independent rounding-exact
restatement of the FP32 accumulation, and the semantics the reference's own
helper routines define (CSR->dense scatter, max-abs-error compare, row-length CV).
"""
import os

import numpy as np
import pytest
import scipy.sparse as sp

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
FIXTURES = ["c0_uniform_k32.npz", "c1_citation_small_k64.npz", "rmat9_k128.npz"]


def _load(name):
    z = np.load(os.path.join(GOLDEN, name))
    return z["rowptr"], z["col"], z["val"], z["B"], z["C64"]


def _rand_csr(rng, m, n, density, empty_frac=0.2):
    A = sp.random(m, n, density=density, format="csr", dtype=np.float32,
                  random_state=np.random.RandomState(int(rng.integers(1 << 30))))
    A.sort_indices()
    keep = rng.random(m) >= empty_frac
    A = sp.diags(keep.astype(np.float32)) @ A
    A = A.tocsr()
    A.eliminate_zeros()
    A.sort_indices()
    return A.indptr.astype(np.int32), A.indices.astype(np.int32), A.data.astype(np.float32)


@pytest.mark.parametrize("name", FIXTURES)
def test_golden_products(oracle, name):
    rowptr, col, val, B, want = _load(name)
    C64, S64 = oracle.csr_spmm_f64(rowptr, col, val, B)
    # float64 oracle against scipy's float64 product: rounding noise only
    scale = np.abs(want).max()
    assert np.abs(C64 - want).max() <= 1e-13 * scale * max(1, int(np.diff(rowptr).max()))
    # its abs-sum against numpy |A| @ |B|
    A = sp.csr_matrix((np.abs(val).astype(np.float64), col, rowptr), shape=(rowptr.size - 1, B.shape[0]))
    S_want = A @ np.abs(B).astype(np.float64)
    np.testing.assert_allclose(S64, S_want, rtol=1e-12, atol=0)
    # FP32 oracle: inside the forward error bound of a length-d recursive sum, n*u*S
    C32 = oracle.csr_spmm_f32(rowptr, col, val, B)
    deg = np.diff(rowptr).astype(np.float64)[:, None]
    bound = (deg + 1) * 2.0 ** -24 * S_want
    assert np.all(np.abs(C32.astype(np.float64) - want) <= bound + 1e-300)
    # and by the benchmark's metric
    err, _ = oracle.max_norm_err(C32, want, S_want)
    assert err <= 1e-5


def test_brute_force_dense(oracle):
    rng = np.random.default_rng(1)
    for m, n, k in [(1, 1, 1), (5, 7, 3), (40, 30, 32), (33, 65, 17)]:
        rowptr, col, val = _rand_csr(rng, m, n, 0.3)
        B = rng.standard_normal((n, k)).astype(np.float32)
        dense = np.zeros((m, n), dtype=np.float64)
        for i in range(m):
            for j in range(rowptr[i], rowptr[i + 1]):
                dense[i, col[j]] += float(val[j])
        want = np.zeros((m, k))
        for i in range(m):
            for c in range(n):
                for q in range(k):
                    want[i, q] += dense[i, c] * float(B[c, q])
        C64, _ = oracle.csr_spmm_f64(rowptr, col, val, B)
        np.testing.assert_allclose(C64, want, rtol=1e-12, atol=1e-14)
        np.testing.assert_allclose(oracle.csr_spmm_f32(rowptr, col, val, B), want, rtol=0, atol=1e-4)


def test_fp32_accumulation_is_sequential_unfused(oracle):
    """Stored-order recursive sum, product rounded to FP32 before the add
    (the arithmetic of spmm_kernel.cu:338-346) - checked bit for bit against a
    numpy restatement that rounds explicitly at every step."""
    rng = np.random.default_rng(2)
    rowptr, col, val = _rand_csr(rng, 25, 40, 0.4)
    B = rng.standard_normal((40, 8)).astype(np.float32)
    got = oracle.csr_spmm_f32(rowptr, col, val, B)
    want = np.zeros((25, 8), dtype=np.float32)
    for i in range(25):
        acc = np.zeros(8, dtype=np.float32)
        for j in range(rowptr[i], rowptr[i + 1]):
            prod = (val[j] * B[col[j]]).astype(np.float32)  # one rounding
            acc = (acc + prod).astype(np.float32)           # second rounding
        want[i] = acc
    assert np.array_equal(got, want)
    # a fused multiply-add, or a reversed order, gives different bits on this input
    fused = np.zeros((25, 8), dtype=np.float32)
    rev = np.zeros((25, 8), dtype=np.float32)
    for i in range(25):
        acc = np.zeros(8, dtype=np.float64)
        accr = np.zeros(8, dtype=np.float32)
        for j in range(rowptr[i], rowptr[i + 1]):
            acc = (np.float64(val[j]) * B[col[j]].astype(np.float64) + acc).astype(np.float32).astype(np.float64)
        for j in range(rowptr[i + 1] - 1, rowptr[i] - 1, -1):
            accr = (accr + (val[j] * B[col[j]]).astype(np.float32)).astype(np.float32)
        fused[i] = acc
        rev[i] = accr
    assert not np.array_equal(got, fused) and not np.array_equal(got, rev)


def test_closed_forms(oracle):
    rng = np.random.default_rng(3)
    n, k = 300, 32
    B = rng.standard_normal((n, k)).astype(np.float32)
    ar = np.arange(n + 1, dtype=np.int32)
    # identity
    C = oracle.csr_spmm_f32(ar, np.arange(n, dtype=np.int32), np.ones(n, np.float32), B)
    assert np.array_equal(C, B)
    # permutation = row gather
    perm = rng.permutation(n).astype(np.int32)
    assert np.array_equal(oracle.csr_spmm_f32(ar, perm, np.ones(n, np.float32), B), B[perm])
    # scaling: diag(d) B
    d = rng.uniform(-2, 2, n).astype(np.float32)
    assert np.array_equal(oracle.csr_spmm_f32(ar, np.arange(n, dtype=np.int32), d, B), d[:, None] * B)
    # all values 1 (the reference's own regime): C[i] = sum of the selected B rows
    rowptr, col, _ = _rand_csr(rng, 50, n, 0.1)
    C64, S = oracle.csr_spmm_f64(rowptr, col, np.ones(col.size, np.float32), B)
    for i in range(50):
        np.testing.assert_allclose(C64[i], B[col[rowptr[i]:rowptr[i + 1]]].astype(np.float64).sum(0), atol=1e-12)
    # row-normalised A times ones = ones on non-empty rows, zeros on empty ones
    deg = np.diff(rowptr)
    val = np.repeat(1.0 / np.maximum(deg, 1), deg).astype(np.float32)
    C = oracle.csr_spmm_f32(rowptr, col, val, np.ones((n, 4), np.float32))
    np.testing.assert_allclose(C[deg > 0], 1.0, atol=1e-6)
    assert not C[deg == 0].any()
    # one hub row over every column
    hub_ptr = np.array([0, 0, n, n], dtype=np.int32)
    C64, _ = oracle.csr_spmm_f64(hub_ptr, np.arange(n, dtype=np.int32), np.ones(n, np.float32), B)
    np.testing.assert_allclose(C64[1], B.astype(np.float64).sum(0), atol=1e-12)
    assert not C64[0].any() and not C64[2].any()
    # transposed operand would fail: A (2x3) with distinct entries against a hand result
    rp = np.array([0, 2, 3], np.int32)
    ci = np.array([0, 2, 1], np.int32)
    va = np.array([2.0, 3.0, 5.0], np.float32)
    Bs = np.array([[1, 10], [2, 20], [4, 40]], np.float32)
    assert np.array_equal(oracle.csr_spmm_f32(rp, ci, va, Bs), np.array([[14, 140], [10, 100]], np.float32))


def test_row_slab_entry_points(oracle):
    rowptr, col, val, B, want = _load("rmat9_k128.npz")
    full = oracle.csr_spmm_f32(rowptr, col, val, B)
    slab = oracle.csr_spmm_f32_rows(rowptr, col, val, B, 100, 300)
    assert np.array_equal(slab, full[100:300])
    C64, S64 = oracle.csr_spmm_f64_rows(rowptr, col, val, B, 100, 300)
    np.testing.assert_allclose(C64, want[100:300], rtol=1e-12, atol=1e-12)


def test_coo_accumulate(oracle):
    rng = np.random.default_rng(4)
    rowptr, col, val = _rand_csr(rng, 60, 50, 0.2)
    B = rng.standard_normal((50, 16)).astype(np.float32)
    deg = np.diff(rowptr)
    row = np.repeat(np.arange(60, dtype=np.int32), deg)
    C0 = rng.standard_normal((60, 16)).astype(np.float32)
    # CSR order, zero start: identical bits to the CSR oracle
    C = np.zeros((60, 16), np.float32)
    oracle.coo_spmm_acc_f32(row, col, val, B, C)
    assert np.array_equal(C, oracle.csr_spmm_f32(rowptr, col, val, B))
    # accumulates into what is there
    C = C0.copy()
    oracle.coo_spmm_acc_f32(row, col, val, B, C)
    want, S = oracle.csr_spmm_f64(rowptr, col, val, B)
    np.testing.assert_allclose(C, C0 + want, atol=1e-5)
    # zero-valued padding entries (row 0, col 0) change nothing; entry order is free up to rounding
    p = rng.permutation(col.size)
    prow = np.concatenate([row[p], np.zeros(7, np.int32)])
    pcol = np.concatenate([col[p], np.zeros(7, np.int32)])
    pval = np.concatenate([val[p], np.zeros(7, np.float32)])
    C = np.zeros((60, 16), np.float32)
    oracle.coo_spmm_acc_f32(prow, pcol, pval, B, C)
    np.testing.assert_allclose(C, want, atol=1e-5)


def test_csr_to_dense(oracle):
    rng = np.random.default_rng(5)
    rowptr, col, val = _rand_csr(rng, 30, 20, 0.3)
    A = sp.csr_matrix((val, col, rowptr), shape=(30, 20))
    assert np.array_equal(oracle.csr_to_dense(rowptr, col, val, 20), A.toarray())
    # duplicates: the later entry wins (scatter by assignment)
    rp = np.array([0, 3], np.int32)
    D = oracle.csr_to_dense(rp, np.array([1, 1, 0], np.int32), np.array([5, 7, 2], np.float32), 3)
    assert np.array_equal(D, np.array([[2, 7, 0]], np.float32))


def test_compare_and_cv(oracle):
    rng = np.random.default_rng(6)
    x = rng.standard_normal(1000).astype(np.float32)
    y = x + rng.uniform(-0.05, 0.05, 1000).astype(np.float32)
    assert oracle.max_abs_err(x, y) == pytest.approx(float(np.abs(x - y).max()), rel=1e-6)
    # the accumulate-200-then-divide form
    assert oracle.max_abs_err(200 * x, x, div=200.0) <= 1e-6
    assert oracle.max_abs_err(x, x) == 0.0
    bad = x.copy()
    bad[17] = np.nan
    assert np.isnan(oracle.max_abs_err(bad, x))
    rowptr = np.array([0, 3, 3, 10, 11], np.int32)
    deg = np.diff(rowptr)
    assert oracle.row_length_cv(rowptr) == pytest.approx(deg.std() / deg.mean(), rel=1e-12)


def test_normalised_error_metric(oracle):
    C64 = np.array([1.0, -2.0, 0.0, 4.0])
    S = np.array([2.0, 2.0, 0.0, 8.0])
    got = np.array([1.0, -2.0, 0.0, 4.0], np.float32)
    assert oracle.max_norm_err(got, C64, S) == (0.0, -1)
    got[3] = 4.0008
    e, pos = oracle.max_norm_err(got, C64, S)
    assert pos == 3 and e == pytest.approx(1e-4, rel=1e-2)
    got[2] = 1e-30  # nonzero where the denominator is zero
    e, pos = oracle.max_norm_err(got, C64, S)
    assert np.isinf(e) and pos == 2
    got[2] = np.nan
    assert np.isinf(oracle.max_norm_err(got, C64, S)[0])
