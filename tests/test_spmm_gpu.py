"""GPU parity tests: the HIP path, called through the C ABI, against the CPU oracle.

Tolerance (stated by the task's acceptance bar): for every output element
    |C_gpu - C_f64| <= 1e-4 * sum_j |a_ij| |b_jk|
with the float64 result and the denominator from the oracle; where the
denominator is 0 (empty rows) the GPU value must be exactly 0.  CSR structure
and output shape are compared exactly.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

TOL = 1e-4


def _to_dev(gpu, *arrays):
    import torch
    return [torch.from_numpy(np.ascontiguousarray(a)).to(gpu) for a in arrays]


def _run(pkg, gpu, g, B, flags=0, poison=True, options=None):
    import torch
    capi = pkg.capi
    k = B.shape[1]
    rp, ci, v, Bd = _to_dev(gpu, g.rowptr, g.col, g.val, B)
    C = torch.full((g.rows, k), float("nan") if poison else 0.0, device=gpu, dtype=torch.float32)
    plan = capi.Plan(g.rows, g.cols, rp, ci, k, flags, options=options)
    info = plan.info
    capi.csr_spmm(plan, rp, ci, v, Bd, C)
    torch.cuda.synchronize()
    # structure must be untouched by the call
    assert torch.equal(rp.cpu(), torch.from_numpy(g.rowptr))
    assert torch.equal(ci.cpu(), torch.from_numpy(g.col))
    plan.destroy()
    return C.cpu().numpy(), info


def _check(oracle, g, B, C, what=""):
    assert C.shape == (g.rows, B.shape[1]) and C.dtype == np.float32
    C64, S64 = oracle.csr_spmm_f64(g.rowptr, g.col, g.val, B)
    err, pos = oracle.max_norm_err(C, C64, S64)
    assert err <= TOL, f"{what}: normalised error {err:.3e} at flat index {pos}"
    deg = np.diff(g.rowptr)
    assert not C[deg == 0].any(), f"{what}: empty rows must be exact zeros"
    return err


def _strategies(capi):
    return [("auto", capi.PLAN_DEFAULT), ("rows", capi.PLAN_FORCE_ROWS),
            ("rows_csr", capi.PLAN_FORCE_ROWS | capi.PLAN_NO_ROW_TILES),
            ("seg", capi.PLAN_FORCE_SEGMENTS),
            ("seg8_nohub", capi.PLAN_FORCE_SEGMENTS | capi.plan_segment_shift(3) | capi.PLAN_NO_HUB_CACHE),
            ("seg64_noremap", capi.PLAN_FORCE_SEGMENTS | capi.plan_segment_shift(6) | capi.PLAN_NO_XCD_REMAP),
            ("seg_hub", capi.PLAN_FORCE_SEGMENTS | capi.PLAN_HUB_CACHE | capi.plan_hub_log2(8)),
            ("seg16_hub_all", capi.PLAN_FORCE_SEGMENTS | capi.plan_segment_shift(4) | capi.PLAN_HUB_CACHE
             | capi.plan_hub_log2(24)),
            ("routed", capi.PLAN_FORCE_ROUTED),
            ("routed_sort_values", capi.PLAN_FORCE_ROUTED | capi.PLAN_ROUTED_SORT_VALUES),
            ("routed_tiny", capi.PLAN_FORCE_ROUTED | capi.plan_hub_log2(3) | capi.plan_segment_shift(3)
             | capi.plan_routed_row_log2(1)),
            ("routed_s16", capi.PLAN_FORCE_ROUTED | capi.plan_hub_log2(10) | capi.plan_segment_shift(4)
             | capi.plan_routed_row_log2(3)),
            ("cluster", capi.PLAN_CLUSTER),
            ("cluster_seg", capi.PLAN_CLUSTER | capi.PLAN_FORCE_SEGMENTS | capi.PLAN_NO_HUB_CACHE),
            ("routed_3phases", capi.PLAN_FORCE_ROUTED | capi.plan_routed_phases(3) | capi.plan_routed_row_log2(4)),
            ("routed_7phases_tiny", capi.PLAN_FORCE_ROUTED | capi.plan_routed_phases(7) | capi.plan_hub_log2(5)
             | capi.plan_segment_shift(3) | capi.plan_routed_row_log2(1)),
            ("sweep", capi.PLAN_FORCE_SWEEP),
            # routed in column-tile phases (only where K is a multiple of the tile width and wider; otherwise
            # these are plain routed plans)
            ("routed_tiles32", capi.flags_with_options(capi.PLAN_FORCE_ROUTED, routed_tile_width=32)),
            ("routed_tiles64_tiny", capi.flags_with_options(
                capi.PLAN_FORCE_ROUTED | capi.plan_hub_log2(5) | capi.plan_segment_shift(3) | capi.plan_routed_row_log2(1),
                routed_tile_width=64)),
            ("routed_tiles32_no_lds", capi.flags_with_options(
                capi.PLAN_FORCE_ROUTED | capi.plan_hub_log2(7) | capi.plan_routed_row_log2(3),
                routed_tile_width=32, routed_lds_rows=-1)),
            ("routed_tiles32_lds16", capi.flags_with_options(
                capi.PLAN_FORCE_ROUTED | capi.plan_hub_log2(12) | capi.plan_routed_row_log2(5),
                routed_tile_width=32, routed_lds_rows=16)),
            ("routed_tiles32_s16", capi.flags_with_options(
                capi.PLAN_FORCE_ROUTED | capi.plan_hub_log2(10) | capi.plan_segment_shift(4) | capi.plan_routed_row_log2(3),
                routed_tile_width=32))]


@pytest.mark.parametrize("k", [32, 64, 128])
def test_config0_uniform(pkg, oracle, gpu, k):
    g = pkg.graphs.make_graph("c0_uniform")
    B = pkg.graphs.make_dense("c0_uniform", g.cols, k)
    for name, flags in _strategies(pkg.capi):
        C, _ = _run(pkg, gpu, g, B, flags)
        _check(oracle, g, B, C, f"c0 k={k} {name}")


@pytest.mark.parametrize("k", [32, 64, 128])
def test_config1_citation(pkg, oracle, gpu, k):
    g = pkg.graphs.make_graph("c1_citation")
    B = pkg.graphs.make_dense("c1_citation", g.cols, k)
    for name, flags in _strategies(pkg.capi):
        C, info = _run(pkg, gpu, g, B, flags)
        _check(oracle, g, B, C, f"c1 k={k} {name}")
    # row-normalised A times a constant matrix gives that constant back
    ones = np.ones((g.cols, k), dtype=np.float32)
    C, _ = _run(pkg, gpu, g, ones)
    np.testing.assert_allclose(C, 1.0, rtol=0, atol=2e-6)


@pytest.mark.parametrize("name,scale", [("c2_social", 0.02), ("c3_copurchase", 0.01), ("c4_rmat", 0.004)])
@pytest.mark.parametrize("k", [32, 64, 128])
def test_scaled_configs(pkg, oracle, gpu, name, scale, k):
    g = pkg.graphs.make_graph(name, scale)
    B = pkg.graphs.make_dense(name, g.cols, k)
    for sname, flags in _strategies(pkg.capi):
        C, _ = _run(pkg, gpu, g, B, flags)
        _check(oracle, g, B, C, f"{name} k={k} {sname}")


def test_deterministic_and_strategies_agree(pkg, oracle, gpu):
    g = pkg.graphs.make_graph("c4_rmat", 0.004)
    B = pkg.graphs.make_dense("c4_rmat", g.cols, 64)
    ref, _ = _run(pkg, gpu, g, B, pkg.capi.PLAN_FORCE_SEGMENTS)
    again, _ = _run(pkg, gpu, g, B, pkg.capi.PLAN_FORCE_SEGMENTS)
    assert np.array_equal(ref, again), "segments strategy must be bit-reproducible"
    # hashed slices with the compact buffer of hot rows (the column-range slices keep none)
    fl = (pkg.capi.PLAN_FORCE_ROUTED | pkg.capi.PLAN_ROUTED_SORT_VALUES | pkg.capi.plan_hub_log2(9)
          | pkg.capi.plan_routed_row_log2(2))
    r1, info = _run(pkg, gpu, g, B, fl)
    r2, _ = _run(pkg, gpu, g, B, fl)
    assert info["strategy"] == pkg.capi.STRATEGY_ROUTED and info["hub_rows"] > 0
    assert np.array_equal(r1, r2), "routed strategy must be bit-reproducible"
    # column-range slices where the plan finds them usable: values in place, no compact buffer, two launches
    fl = pkg.capi.PLAN_FORCE_ROUTED | pkg.capi.plan_routed_row_log2(2)
    q1, info = _run(pkg, gpu, g, B, fl)
    q2, _ = _run(pkg, gpu, g, B, fl)
    assert info["strategy"] == pkg.capi.STRATEGY_ROUTED
    assert (info["launches_per_spmm"], info["hub_rows"] > 0) in ((2, False), (3, True))
    assert np.array_equal(q1, q2), "routed strategy must be bit-reproducible"
    rows, _ = _run(pkg, gpu, g, B, pkg.capi.PLAN_FORCE_ROWS)
    # the whole-row kernel accumulates in stored order with FMA; rows that fit one
    # segment are accumulated identically by the segments kernel
    deg = np.diff(g.rowptr)
    short = deg <= 1
    assert np.array_equal(rows[short], ref[short])


def test_closed_forms(pkg, oracle, gpu):
    import scipy.sparse as sp
    graphs = pkg.graphs
    n, k = 777, 64
    rng = np.random.default_rng(5)
    B = rng.standard_normal((n, k)).astype(np.float32)
    # identity: C == B bit for bit
    eye = graphs.CSR(n, n, np.arange(n + 1, dtype=np.int32), np.arange(n, dtype=np.int32),
                     np.ones(n, dtype=np.float32))
    for _, flags in _strategies(pkg.capi):
        C, _ = _run(pkg, gpu, eye, B, flags)
        assert np.array_equal(C, B)
    # permutation: row gather, bit for bit
    perm = rng.permutation(n).astype(np.int32)
    pm = graphs.CSR(n, n, np.arange(n + 1, dtype=np.int32), perm, np.ones(n, dtype=np.float32))
    for _, flags in _strategies(pkg.capi):
        C, _ = _run(pkg, gpu, pm, B, flags)
        assert np.array_equal(C, B[perm])
    # one hub row over all columns plus empty rows around it, all values 1: column sums
    rowptr = np.zeros(n + 1, dtype=np.int32)
    rowptr[401:] = n
    hub = graphs.CSR(n, n, rowptr, np.arange(n, dtype=np.int32), np.ones(n, dtype=np.float32))
    for _, flags in _strategies(pkg.capi):
        C, _ = _run(pkg, gpu, hub, B, flags)
        np.testing.assert_allclose(C[400], B.astype(np.float64).sum(0), rtol=0, atol=1e-4 * np.abs(B).sum(0).max())
        assert not C[:400].any() and not C[401:].any()
    # random rectangular matrix (rows != cols) against scipy in float64
    A = sp.random(300, 1000, density=0.03, format="csr", dtype=np.float32, random_state=3)
    A.sort_indices()
    g = graphs.CSR(300, 1000, A.indptr.astype(np.int32), A.indices.astype(np.int32), A.data)
    B2 = rng.standard_normal((1000, 32)).astype(np.float32)
    want = A.astype(np.float64) @ B2.astype(np.float64)
    S = abs(A).astype(np.float64) @ np.abs(B2).astype(np.float64)
    for _, flags in _strategies(pkg.capi):
        C, _ = _run(pkg, gpu, g, B2, flags)
        assert np.all(np.abs(C - want) <= TOL * S + 0.0)


def test_linearity_and_column_tiles(pkg, oracle, gpu):
    g = pkg.graphs.make_graph("c3_copurchase", 0.004)
    B1 = pkg.graphs.dense_normal(g.cols, 128, 11)
    B2 = pkg.graphs.dense_normal(g.cols, 128, 12)
    C1, _ = _run(pkg, gpu, g, B1)
    C2, _ = _run(pkg, gpu, g, B2)
    C12, _ = _run(pkg, gpu, g, B1 + B2)
    _, S1 = oracle.csr_spmm_f64(g.rowptr, g.col, g.val, B1)
    _, S2 = oracle.csr_spmm_f64(g.rowptr, g.col, g.val, B2)
    assert np.all(np.abs(C12.astype(np.float64) - C1 - C2) <= 3 * TOL * (S1 + S2) + 1e-30)
    # K=128 restricted to its first 32 columns == K=32 run on B[:, :32]
    C32, _ = _run(pkg, gpu, g, np.ascontiguousarray(B1[:, :32]), pkg.capi.PLAN_FORCE_SEGMENTS | pkg.capi.plan_segment_shift(6))
    C128, _ = _run(pkg, gpu, g, B1, pkg.capi.PLAN_FORCE_SEGMENTS | pkg.capi.plan_segment_shift(6))
    assert np.array_equal(C32, C128[:, :32])


@pytest.mark.parametrize("k", [1, 2, 3, 5, 7, 30, 41, 47, 50, 127, 129, 130, 173, 259])
def test_k_not_a_multiple_of_four(pkg, oracle, gpu, k):
    """Row lengths that are not a multiple of 4 (rows of B and C start at any multiple of 4 bytes; the
    number of classes of a node classifier is such a K): whole rows over row tiles (16-byte gathers
    at 4-byte alignment; K < 4 from a padded copy of B) and over the CSR arrays, forced segments (three lengths) and the
    plan-less entry point with the run-time-K sub-wave kernels, the lane that owns the last columns
    of a row reading and writing only those that exist.  C poisoned with NaN beforehand and laid out
    with guard rows, which must stay untouched."""
    import torch
    capi = pkg.capi
    g = pkg.graphs.make_graph("c4_rmat", 0.004)
    B = pkg.graphs.dense_normal(g.cols, k, 77)
    C, info = _run(pkg, gpu, g, B)
    # (below 4 columns through a copy of B with rows of 4 floats: one more launch)
    assert info["strategy"] == capi.STRATEGY_ROWS and info["launches_per_spmm"] == (2 if k < 4 else 1), info
    assert info["row_tiles"] > 0, info
    _check(oracle, g, B, C, f"rows k={k}")
    C, info = _run(pkg, gpu, g, B, capi.PLAN_NO_ROW_TILES)
    assert info["strategy"] == capi.STRATEGY_ROWS and info["row_tiles"] == 0, info
    _check(oracle, g, B, C, f"rows over the CSR arrays k={k}")
    for shift in (0, 3, 7):
        C, info = _run(pkg, gpu, g, B, capi.PLAN_FORCE_SEGMENTS | capi.plan_segment_shift(shift))
        assert info["strategy"] == capi.STRATEGY_SEGMENTS and info["launches_per_spmm"] == 2, info
        _check(oracle, g, B, C, f"segments k={k} shift={shift}")
        again, _ = _run(pkg, gpu, g, B, capi.PLAN_FORCE_SEGMENTS | capi.plan_segment_shift(shift))
        assert np.array_equal(C, again), "bit-reproducible"
    # B and C inside larger allocations: nothing may be read past the last row of B (NaN there would
    # show) nor written past the last row of C
    rp, ci, v = _to_dev(gpu, g.rowptr, g.col, g.val)
    pad = 64
    Bbig = torch.full((g.cols * k + pad,), float("nan"), device=gpu)
    Bbig[:g.cols * k] = torch.from_numpy(B).to(gpu).reshape(-1)
    Cbig = torch.full((g.rows * k + pad,), 12345.0, device=gpu)
    Bd, Cd = Bbig[:g.cols * k].view(g.cols, k), Cbig[:g.rows * k].view(g.rows, k)
    for flags in (capi.PLAN_DEFAULT, capi.PLAN_NO_ROW_TILES, capi.PLAN_FORCE_SEGMENTS):
        Cd.fill_(float("nan"))
        plan = capi.Plan(g.rows, g.cols, rp, ci, k, flags)
        capi.csr_spmm(plan, rp, ci, v, Bd, Cd)
        torch.cuda.synchronize()
        plan.destroy()
        _check(oracle, g, B, Cd.cpu().numpy(), f"guarded k={k} flags={flags}")
        assert bool((Cbig[g.rows * k:] == 12345.0).all()), f"k={k}: wrote past the last row of C"
    Cn = torch.full((g.rows, k), float("nan"), device=gpu)
    capi.csr_spmm_noplan(g.rows, g.cols, rp, ci, v, Bd, Cn)
    _check(oracle, g, B, Cn.cpu().numpy(), f"noplan k={k}")


@pytest.mark.parametrize("k", [4, 8, 12, 16, 20, 24, 48, 96, 100, 160, 200, 256, 384])
def test_multiple_of_four_k(pkg, oracle, gpu, k):
    """Every multiple of 4 besides the tuned sizes (the reference has a kernel of its own for K < 32,
    spmm_kernel.cu:372-387, 406-410): whole rows on a small matrix - over row tiles in 32-column tiles,
    the last one narrower, or over the CSR arrays with hub rows on a wavefront each -, the run-time-K
    segments kernels when forced, and the plan-less entry point; C poisoned with NaN beforehand, empty
    rows exact zeros."""
    import torch
    capi = pkg.capi
    g = pkg.graphs.make_graph("c4_rmat", 0.004)  # hub rows of thousands of nonzeros, 40 % empty rows
    B = pkg.graphs.dense_normal(g.cols, k, 78)
    C, info = _run(pkg, gpu, g, B)
    assert info["strategy"] == capi.STRATEGY_ROWS and info["launches_per_spmm"] == 1 and info["row_tiles"] > 0, info
    _check(oracle, g, B, C, f"rows k={k}")
    C, info = _run(pkg, gpu, g, B, capi.PLAN_NO_ROW_TILES)
    assert info["strategy"] == capi.STRATEGY_ROWS and info["row_tiles"] == 0, info
    _check(oracle, g, B, C, f"rows over the CSR arrays k={k}")
    for shift in (0, 3, 7):
        C, info = _run(pkg, gpu, g, B, capi.PLAN_FORCE_SEGMENTS | capi.plan_segment_shift(shift))
        assert info["strategy"] == capi.STRATEGY_SEGMENTS and info["launches_per_spmm"] == 2, info
        assert shift == 0 or info["segment_length"] == 1 << shift
        _check(oracle, g, B, C, f"segments k={k} shift={shift}")
        again, _ = _run(pkg, gpu, g, B, capi.PLAN_FORCE_SEGMENTS | capi.plan_segment_shift(shift))
        assert np.array_equal(C, again), "bit-reproducible"
    rp, ci, v, Bd = _to_dev(gpu, g.rowptr, g.col, g.val, B)
    Cn = torch.full((g.rows, k), float("nan"), device=gpu)
    capi.csr_spmm_noplan(g.rows, g.cols, rp, ci, v, Bd, Cn)
    _check(oracle, g, B, Cn.cpu().numpy(), f"noplan k={k}")


@pytest.mark.parametrize("k", [16, 41, 96])
def test_multiple_of_four_k_large_graph(pkg, oracle, gpu, k):
    """Beyond 2^21 nonzeros the plan picks whole rows over row tiles for these K by itself - or, from
    K = 16 on a matrix of 2^22 nonzeros and more, one of the tuned layouts in column tiles."""
    capi = pkg.capi
    g = pkg.graphs.make_graph("c2_social", 0.05)
    assert g.nnz > 1 << 21
    B = pkg.graphs.dense_normal(g.cols, k, 79)
    C, info = _run(pkg, gpu, g, B)
    tiled = (capi.STRATEGY_SWEEP, capi.STRATEGY_ROUTED, capi.STRATEGY_ORDERED)
    assert (info["strategy"] == capi.STRATEGY_ROWS and info["row_tiles"] > 0) or \
        (k >= 16 and info["strategy"] in tiled), info
    _check(oracle, g, B, C, f"auto k={k}")


def test_edge_shapes(pkg, oracle, gpu):
    import torch
    capi, graphs = pkg.capi, pkg.graphs
    # all rows empty
    g = graphs.CSR(100, 50, np.zeros(101, dtype=np.int32), np.zeros(0, dtype=np.int32), np.zeros(0, dtype=np.float32))
    B = graphs.dense_normal(50, 32, 1)
    for _, flags in _strategies(capi):
        C, _ = _run(pkg, gpu, g, B, flags)
        assert C.shape == (100, 32) and not C.any()
    # the same through the C ABI with NULL for everything a matrix without nonzeros never reads (col, val,
    # B), at row lengths of every kind: tuned, a multiple of 4, not one, below 4 (B through a padded copy)
    import ctypes
    L = capi.lib()
    rp = torch.zeros(101, dtype=torch.int32, device=gpu)
    for k in (32, 100, 41, 5, 3, 1):
        handle = ctypes.c_void_p()
        capi.check(L.hpspmm_plan_create(100, 50, 0, rp.data_ptr(), None, k, capi.PLAN_DEFAULT, None, ctypes.byref(handle)))
        C = torch.full((100, k), float("nan"), device=gpu)
        capi.check(L.hpspmm_csr_spmm(handle, rp.data_ptr(), None, None, None, C.data_ptr(), None))
        torch.cuda.synchronize()
        assert not C.cpu().numpy().any(), f"empty matrix, k={k}"
        L.hpspmm_plan_destroy(handle)
    # a single row, a single nonzero
    g = graphs.CSR(1, 3, np.array([0, 1], dtype=np.int32), np.array([2], dtype=np.int32), np.array([2.5], dtype=np.float32))
    B = graphs.dense_normal(3, 128, 2)
    for _, flags in _strategies(capi):
        C, _ = _run(pkg, gpu, g, B, flags)
        assert np.array_equal(C[0], np.float32(2.5) * B[2])
    # zero rows: nothing to do, no error
    rp = torch.zeros(1, dtype=torch.int32, device=gpu)
    ci = torch.zeros(0, dtype=torch.int32, device=gpu)
    plan = capi.Plan(0, 5, rp, ci, 32)
    capi.csr_spmm(plan, rp, ci, torch.zeros(0, device=gpu), torch.zeros(5, 32, device=gpu), torch.zeros(0, 32, device=gpu))
    plan.destroy()
    # segment boundaries exactly on row boundaries, and rows spanning many segments
    n = 64
    deg = np.array([8] * 16 + [0] * 8 + [64] * 4 + [1] * 8 + [200] + [0] * 27, dtype=np.int32)
    assert deg.size == n
    rowptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int32)
    rng = np.random.default_rng(0)
    col = np.concatenate([np.sort(rng.choice(300, d, replace=False)) for d in deg]).astype(np.int32)
    val = rng.uniform(-1, 1, col.size).astype(np.float32)
    g = graphs.CSR(n, 300, rowptr, col, val)
    for k in (32, 64, 128):
        B = graphs.dense_normal(300, k, 9)
        for shift in (3, 4, 5, 6):
            C, _ = _run(pkg, gpu, g, B, capi.PLAN_FORCE_SEGMENTS | capi.plan_segment_shift(shift))
            _check(oracle, g, B, C, f"boundaries k={k} shift={shift}")


def test_noplan_entry(pkg, oracle, gpu):
    import torch
    g = pkg.graphs.make_graph("c1_citation", 0.2)
    for k in (32, 64, 128, 10):
        B = pkg.graphs.dense_normal(g.cols, k, 3)
        rp, ci, v, Bd = _to_dev(gpu, g.rowptr, g.col, g.val, B)
        C = torch.full((g.rows, k), float("nan"), device=gpu)
        pkg.capi.csr_spmm_noplan(g.rows, g.cols, rp, ci, v, Bd, C)
        torch.cuda.synchronize()
        _check(oracle, g, B, C.cpu().numpy(), f"noplan k={k}")


def test_fill(pkg, gpu):
    import torch
    x = torch.empty(100003, device=gpu)
    pkg.capi.fill_f32(x, 0.0)
    assert not x.any().item()
    pkg.capi.fill_f32(x, -2.5)
    assert torch.all(x == -2.5).item()


def _check_accumulated(got, C0, C64, S64, calls, what):
    """C0 + calls * (A B) within calls * TOL * (sum |a||b| + |C0|); a failure names the worst element."""
    err = np.abs(got.astype(np.float64) - (C0 + calls * C64))
    bound = calls * TOL * (S64 + np.abs(C0))
    bad = ~(err <= bound)  # (also catches NaN)
    if bad.any():
        i, j = np.unravel_index(np.argmax(np.where(bad, err - bound, -np.inf)), err.shape)
        raise AssertionError(f"{what}: {int(bad.sum())} elements out of tolerance in {len(np.unique(np.nonzero(bad)[0]))} "
                             f"rows; worst at ({i}, {j}): got {got[i, j]!r}, expected {C0[i, j] + calls * C64[i, j]!r}, "
                             f"C0 {C0[i, j]!r}, bound {bound[i, j]:.3e}")


@pytest.mark.parametrize("k", [32, 64, 128, 24, 16, 96, 200, 7, 41, 173])
def test_coo_accumulate(pkg, oracle, gpu, k):
    """The LBSpMM contract: C += A B, padded zero entries, rows in permuted order."""
    import torch
    g = pkg.graphs.make_graph("c4_rmat", 0.002)
    B = pkg.graphs.dense_normal(g.cols, k, 21)
    deg = np.diff(g.rowptr)
    row = np.repeat(np.arange(g.rows, dtype=np.int32), deg)
    # rows emitted in a permuted order, ids unchanged; then zero padding to a multiple of 32
    order = np.random.default_rng(1).permutation(g.rows)
    idx = np.concatenate([np.arange(g.rowptr[r], g.rowptr[r + 1]) for r in order]) if g.nnz else np.zeros(0, int)
    pad = (-g.nnz) % 32
    prow = np.concatenate([row[idx], np.zeros(pad, np.int32)])
    pcol = np.concatenate([g.col[idx], np.zeros(pad, np.int32)])
    pval = np.concatenate([g.val[idx], np.zeros(pad, np.float32)])
    C0 = pkg.graphs.dense_normal(g.rows, k, 22)
    r_, c_, v_, Bd, C = _to_dev(gpu, prow, pcol, pval, B, C0)
    pkg.capi.coo_spmm_accumulate(g.rows, g.cols, r_, c_, v_, Bd, C)
    torch.cuda.synchronize()
    C64, S64 = oracle.csr_spmm_f64(g.rowptr, g.col, g.val, B)
    got = C.cpu().numpy()
    _check_accumulated(got, C0, C64, S64, 1, f"k={k}, first call")
    # twice more: accumulates (the reference runs it 200 times and divides)
    pkg.capi.coo_spmm_accumulate(g.rows, g.cols, r_, c_, v_, Bd, C)
    pkg.capi.coo_spmm_accumulate(g.rows, g.cols, r_, c_, v_, Bd, C)
    torch.cuda.synchronize()
    got = C.cpu().numpy()
    _check_accumulated(got, C0, C64, S64, 3, f"k={k}, three calls")


def test_error_codes(pkg, gpu):
    import torch
    capi = pkg.capi
    rp = torch.tensor([0, 2, 1, 3], dtype=torch.int32, device=gpu)  # decreases
    ci = torch.tensor([0, 1, 2], dtype=torch.int32, device=gpu)
    with pytest.raises(capi.HpSpmmError) as ei:
        capi.Plan(3, 3, rp, ci, 32)
    assert ei.value.code == capi.ERR_BAD_CSR
    rp = torch.tensor([0, 1, 2, 3], dtype=torch.int32, device=gpu)
    ci = torch.tensor([0, 1, 3], dtype=torch.int32, device=gpu)  # col == cols
    with pytest.raises(capi.HpSpmmError) as ei:
        capi.Plan(3, 3, rp, ci, 32)
    assert ei.value.code == capi.ERR_BAD_CSR
    ci = torch.tensor([0, 1, 2], dtype=torch.int32, device=gpu)
    rp_bad = torch.tensor([0, 1, 2, 4], dtype=torch.int32, device=gpu)  # rowptr[rows] != nnz
    with pytest.raises(capi.HpSpmmError) as ei:
        capi.Plan(3, 3, rp_bad, ci, 32)
    assert ei.value.code == capi.ERR_BAD_CSR
    with pytest.raises(capi.HpSpmmError) as ei:
        capi.Plan(3, 3, rp, ci, 0)
    assert ei.value.code == capi.ERR_INVALID_ARG
    # a good plan still works after the failures
    plan = capi.Plan(3, 3, rp, ci, 32)
    assert plan.info["rows"] == 3
    plan.destroy()


def test_other_csr_arrays_are_refused(pkg, oracle, gpu):
    """A plan holds the structure it was built from; rowptr / col at other addresses are most likely
    another matrix and are refused, whatever strategy the plan chose - unless the plan was created
    with HPSPMM_PLAN_ALLOW_MOVED_CSR, in which case copies of the same structure give the same product."""
    import torch
    capi = pkg.capi
    g = pkg.graphs.make_graph("c4_rmat", 0.004)
    k = 64
    B = pkg.graphs.make_dense("c4_rmat", g.cols, k)
    rp, ci, v, Bd = _to_dev(gpu, g.rowptr, g.col, g.val, B)
    rp2, ci2 = rp.clone(), ci.clone()
    for name, flags in _strategies(capi):
        plan = capi.Plan(g.rows, g.cols, rp, ci, k, flags)
        C = torch.full((g.rows, k), float("nan"), device=gpu)
        for bad_rp, bad_ci in ((rp2, ci), (rp, ci2), (rp2, ci2)):
            with pytest.raises(capi.HpSpmmError) as ei:
                capi.csr_spmm(plan, bad_rp, bad_ci, v, Bd, C)
            assert ei.value.code == capi.ERR_INVALID_ARG, name
            assert "not the arrays this plan was built from" in str(ei.value)
        torch.cuda.synchronize()
        assert torch.isnan(C).all().item(), f"{name}: a refused call must not launch anything"
        capi.csr_spmm(plan, rp, ci, v, Bd, C)  # the plan itself is still good
        _check(oracle, g, B, C.cpu().numpy(), f"after refusals, {name}")
        plan.destroy()
        plan = capi.Plan(g.rows, g.cols, rp, ci, k, flags | capi.PLAN_ALLOW_MOVED_CSR)
        C.fill_(float("nan"))
        capi.csr_spmm(plan, rp2, ci2, v, Bd, C)
        _check(oracle, g, B, C.cpu().numpy(), f"moved arrays allowed, {name}")
        plan.destroy()


def test_large_hot_set(pkg, oracle, gpu):
    """A hot set of 2^18 columns, four times the plan's own choice (the selected columns are ranked by
    a radix sort of several tiles).  Forced routed strategy with that hot set and 4 phases on an
    R-MAT of 524k columns; checked on row ranges that include the heaviest rows."""
    capi = pkg.capi
    g = pkg.graphs.make_graph("c4_rmat", 0.125)
    assert g.cols > 1 << 18
    k = 32
    B = pkg.graphs.make_dense("c4_rmat", g.cols, k)
    flags = capi.PLAN_FORCE_ROUTED | capi.plan_hub_log2(18) | capi.plan_routed_phases(4) | capi.PLAN_ROUTED_SORT_VALUES
    C, info = _run(pkg, gpu, g, B, flags)
    assert info["strategy"] == capi.STRATEGY_ROUTED and info["hub_rows"] > 1 << 17, info
    again, info2 = _run(pkg, gpu, g, B, flags)
    assert info == info2 and np.array_equal(C, again)
    top = int(np.argmax(np.diff(g.rowptr)))
    for lo, hi in ((0, 2000), (max(0, top - 10), min(g.rows, top + 10)), (g.rows - 2000, g.rows)):
        C64, S64 = oracle.csr_spmm_f64_rows(g.rowptr, g.col, g.val, B, lo, hi)
        err, pos = oracle.max_norm_err(C[lo:hi], C64, S64)
        assert err <= TOL, (lo, hi, err, pos)


def test_two_plans_of_one_matrix_give_the_same_bits(pkg, oracle, gpu):
    """Plan construction is deterministic, the clustering included: a second plan of the same matrix
    orders the rows alike, so C agrees bit for bit between plans, not only between calls."""
    capi = pkg.capi
    for name, scale, k, flags in (("c3_copurchase", 0.05, 64, capi.PLAN_DEFAULT),
                                  ("c3_copurchase", 0.02, 32, capi.PLAN_CLUSTER | capi.PLAN_FORCE_SEGMENTS),
                                  ("c4_rmat", 0.008, 128, capi.PLAN_CLUSTER),
                                  ("c2_social", 0.1, 128, capi.PLAN_DEFAULT)):
        g = pkg.graphs.make_graph(name, scale)
        B = pkg.graphs.make_dense(name, g.cols, k)
        C1, i1 = _run(pkg, gpu, g, B, flags)
        C2, i2 = _run(pkg, gpu, g, B, flags)
        assert i1 == i2, (name, i1, i2)
        assert np.array_equal(C1, C2), f"{name}: two plans, different bits"
        if name == "c3_copurchase":
            assert i1["strategy"] == capi.STRATEGY_ORDERED and i1["lds_served_nnz"] >= 0.3 * g.nnz, i1


def test_xcd_placement_is_verified_at_plan_time(pkg, oracle, gpu):
    """The routed strategy relies on workgroup b running on XCD b % 8.  The plan measures that once
    per device; on the whole MI355X it holds and the social graph gets the routed strategy.  With the
    probe overridden to 'does not hold' the plan keeps to a strategy without XCD placement and the
    product is the same to rounding."""
    capi = pkg.capi
    g = pkg.graphs.make_graph("c2_social", 0.1)
    k = 128
    B = pkg.graphs.make_dense("c2_social", g.cols, k)
    C, info = _run(pkg, gpu, g, B, capi.PLAN_NO_SWEEP)  # (the sweep strategy, which this graph gets by default, places nothing)
    assert info["strategy"] == capi.STRATEGY_ROUTED, info
    _check(oracle, g, B, C, "probe result")
    C0, info0 = _run(pkg, gpu, g, B, capi.PLAN_NO_SWEEP, options={"xcd_dealing": 2})
    assert info0["strategy"] in (capi.STRATEGY_SEGMENTS, capi.STRATEGY_ROWS), info0
    _check(oracle, g, B, C0, "placement not available")


def _sample_check(oracle, g, B, C_dev, ranges, what):
    """Oracle check on contiguous row ranges of a large result held on the GPU."""
    for lo, hi in ranges:
        got = C_dev[lo:hi].cpu().numpy()
        C64, S64 = oracle.csr_spmm_f64_rows(g.rowptr, g.col, g.val, B, lo, hi)
        err, pos = oracle.max_norm_err(got, C64, S64)
        assert err <= TOL, f"{what}: rows [{lo},{hi}) normalised error {err:.3e} at {pos}"
        deg = np.diff(g.rowptr[lo:hi + 1])
        assert not got[deg == 0].any()


@pytest.mark.parametrize("name,k", [("c2_social", 128), ("c2_social", 64), ("c4_rmat", 128), ("c3_copurchase", 64),
                                    ("c2_social", 32)])
def test_full_size_configs(pkg, oracle, gpu, name, k):
    """The benchmark configurations at full size, default plan (the strategy the benchmark times):
    the oracle on every row, agreement between strategies, NaN-poisoned C fully overwritten."""
    import torch
    capi = pkg.capi
    g = pkg.graphs.make_graph(name)
    B = pkg.graphs.make_dense(name, g.cols, k)
    rp, ci, v, Bd = _to_dev(gpu, g.rowptr, g.col, g.val, B)
    out = {}
    for tag, flags in (("auto", capi.PLAN_DEFAULT),
                       ("plain", capi.PLAN_FORCE_SEGMENTS | capi.PLAN_NO_HUB_CACHE | capi.PLAN_NO_ROUTED)):
        C = torch.full((g.rows, k), float("nan"), device=gpu)
        plan = capi.Plan(g.rows, g.cols, rp, ci, k, flags)
        info = plan.info
        capi.csr_spmm(plan, rp, ci, v, Bd, C)
        torch.cuda.synchronize()
        plan.destroy()
        assert not torch.isnan(C).any().item(), f"{name} K={k} {tag}: C not fully written"
        out[tag] = (C, info)
    expect = {("c2_social", 128): capi.STRATEGY_SWEEP, ("c2_social", 64): capi.STRATEGY_SWEEP,
              ("c4_rmat", 128): capi.STRATEGY_ROUTED, ("c3_copurchase", 64): capi.STRATEGY_ORDERED,
              ("c2_social", 32): capi.STRATEGY_SWEEP}[(name, k)]
    assert out["auto"][1]["strategy"] == expect
    # the two strategies sum in different orders: they agree to rounding, scaled by |A| |B|
    plan = capi.Plan(g.rows, g.cols, rp, ci, k, capi.PLAN_FORCE_SEGMENTS | capi.PLAN_NO_HUB_CACHE | capi.PLAN_NO_ROUTED)
    S = torch.empty((g.rows, k), device=gpu)
    capi.csr_spmm(plan, rp, ci, v.abs(), Bd.abs(), S)
    torch.cuda.synchronize()
    plan.destroy()
    diff = (out["auto"][0] - out["plain"][0]).abs()
    assert torch.all(diff <= TOL * S).item(), f"{name} K={k}: strategies disagree by {float((diff / S.clamp_min(1e-30)).max()):.3e}"
    del S, diff
    # oracle over ALL rows, in slabs (the float64 result and its denominator of a slab at a time)
    slab = max(1, (1 << 25) // k)
    ranges = [(lo, min(lo + slab, g.rows)) for lo in range(0, g.rows, slab)]
    _sample_check(oracle, g, B, out["auto"][0], ranges, f"{name} K={k}")


def _random_csr(rng, rows, cols, mean_deg, skew, empty_frac, sorted_unique=True):
    """Random CSR with a heavy-tailed degree sequence; optionally unsorted columns with duplicates."""
    deg = np.minimum((rng.pareto(skew, rows) + 0.2) * mean_deg, cols * (1 if sorted_unique else 3)).astype(np.int64)
    deg[rng.random(rows) < empty_frac] = 0
    rowptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int32)
    parts = []
    for d in deg:
        if sorted_unique:
            parts.append(np.sort(rng.choice(cols, size=int(d), replace=False)))
        else:
            parts.append(rng.integers(0, cols, size=int(d)))
    col = (np.concatenate(parts) if parts else np.zeros(0)).astype(np.int32)
    val = rng.uniform(-1, 1, col.size).astype(np.float32)
    return rowptr, col, val


@pytest.mark.parametrize("seed", range(12))
def test_random_matrices_all_strategies(pkg, oracle, gpu, seed):
    """Randomised shapes, degree skews, empty rows; every strategy against scipy float64
    (independent of the oracle) at the benchmark tolerance."""
    import scipy.sparse as sp
    rng = np.random.default_rng(1000 + seed)
    rows = int(rng.integers(1, 3000))
    cols = int(rng.integers(1, 3000))
    k = int(rng.choice([32, 64, 128]))
    rowptr, col, val = _random_csr(rng, rows, cols, mean_deg=float(rng.uniform(0.5, 40)),
                                   skew=float(rng.uniform(0.8, 3.0)), empty_frac=float(rng.uniform(0, 0.6)),
                                   sorted_unique=(seed % 3 != 2))
    g = pkg.graphs.CSR(rows, cols, rowptr, col, val)
    B = rng.standard_normal((cols, k)).astype(np.float32)
    # copies: scipy canonicalises (sorts, merges duplicates) in place on the arrays it is given
    A = sp.csr_matrix((val.astype(np.float64), col.copy(), rowptr.copy()), shape=(rows, cols))
    Aabs = sp.csr_matrix((np.abs(val).astype(np.float64), col.copy(), rowptr.copy()), shape=(rows, cols))
    want = A @ B.astype(np.float64)
    S = Aabs @ np.abs(B).astype(np.float64)
    for name, flags in _strategies(pkg.capi):
        C, _ = _run(pkg, gpu, g, B, flags)
        bad = np.abs(C - want) > TOL * S
        assert not bad.any(), f"seed {seed} rows={rows} cols={cols} k={k} {name}: {int(bad.sum())} elements off"
        assert not C[np.diff(rowptr) == 0].any()


@pytest.mark.parametrize("seed", range(10))
def test_random_matrices_column_tiles(pkg, oracle, gpu, seed):
    """The same at row lengths outside the tuned set: from 16 columns up the forced sweep, routed and
    ordered plans run in column tiles; whole rows run over row tiles - B as it lies, then through the
    padded copy -, the others through the run-time-K kernels."""
    import scipy.sparse as sp
    rng = np.random.default_rng(2000 + seed)
    rows = int(rng.integers(1, 3000))
    cols = int(rng.integers(1, 3000))
    k = int(rng.choice([16, 17, 20, 30, 40, 41, 47, 96, 100, 127, 160, 173, 200, 256, 259, 384] if seed % 2 == 0 else
                       [1, 2, 3, 5, 6, 7, 9, 13, 33, 34, 35, 37, 66, 97, 131]))
    rowptr, col, val = _random_csr(rng, rows, cols, mean_deg=float(rng.uniform(0.5, 40)),
                                   skew=float(rng.uniform(0.8, 3.0)), empty_frac=float(rng.uniform(0, 0.6)),
                                   sorted_unique=(seed % 3 != 2))
    g = pkg.graphs.CSR(rows, cols, rowptr, col, val)
    B = rng.standard_normal((cols, k)).astype(np.float32)
    A = sp.csr_matrix((val.astype(np.float64), col.copy(), rowptr.copy()), shape=(rows, cols))
    Aabs = sp.csr_matrix((np.abs(val).astype(np.float64), col.copy(), rowptr.copy()), shape=(rows, cols))
    want = A @ B.astype(np.float64)
    S = Aabs @ np.abs(B).astype(np.float64)
    tiled = 0
    for name, flags in _strategies(pkg.capi):
        C, info = _run(pkg, gpu, g, B, flags)
        tiled += info["strategy"] in (pkg.capi.STRATEGY_SWEEP, pkg.capi.STRATEGY_ROUTED, pkg.capi.STRATEGY_ORDERED)
        bad = np.abs(C - want) > TOL * S
        assert not bad.any(), f"seed {seed} rows={rows} cols={cols} k={k} {name}: {int(bad.sum())} elements off"
        assert not C[np.diff(rowptr) == 0].any()
    assert tiled >= 4 or col.size == 0 or k < 16, f"seed {seed}: only {tiled} plans ran in column tiles"
    C, info = _run(pkg, gpu, g, B, pkg.capi.PLAN_FORCE_ROWS, options={"row_tiles_pad": 2})
    assert info["row_tiles"] > 0 or col.size == 0 or rows > 40 * col.size, info
    assert info["launches_per_spmm"] == (2 if info["row_tiles"] > 0 and k % 32 != 0 else 1), info
    bad = np.abs(C - want) > TOL * S
    assert not bad.any(), f"seed {seed} rows={rows} cols={cols} k={k} rows over the padded copy: {int(bad.sum())} elements off"
    assert not C[np.diff(rowptr) == 0].any()


def test_non_finite_values_stay_in_their_rows(pkg, oracle, gpu):
    """An inf / NaN in B reaches exactly the rows that reference that row of B (no 0 * inf leaks
    from padding or predication)."""
    g = pkg.graphs.make_graph("c1_citation", 0.1)
    for k in (32, 64, 128):
        B = pkg.graphs.dense_normal(g.cols, k, 5)
        B[7, 3] = np.inf
        B[11, 0] = np.nan
        rows = np.repeat(np.arange(g.rows), np.diff(g.rowptr))
        touched = np.zeros(g.rows, dtype=bool)
        touched[rows[(g.col == 7) | (g.col == 11)]] = True
        for name, flags in _strategies(pkg.capi):
            C, _ = _run(pkg, gpu, g, B, flags)
            finite_rows = np.isfinite(C).all(axis=1)
            assert finite_rows[~touched].all(), f"k={k} {name}: non-finite value leaked into an unrelated row"
            assert (~finite_rows[touched]).all(), f"k={k} {name}: a referencing row lost the non-finite value"


def test_unaligned_arrays_and_new_values_per_call(pkg, oracle, gpu):
    """Caller arrays that are only 4-byte aligned (views one element into a buffer), and a plan reused
    with different values: the plan holds structure only, so the second call must see the new values."""
    import torch
    capi = pkg.capi
    g = pkg.graphs.make_graph("c4_rmat", 0.004)
    for k in (32, 128):
        B = pkg.graphs.make_dense("c4_rmat", g.cols, k)
        Bd, = _to_dev(gpu, B)
        pad = lambda a: torch.from_numpy(np.concatenate([np.zeros(1, a.dtype), a])).to(gpu)[1:]
        rp, ci, v = pad(g.rowptr), pad(g.col), pad(g.val)
        assert v.data_ptr() % 16 == 4
        val2 = (g.val * np.float32(-0.5) + np.float32(0.25)).astype(np.float32)
        v2 = pad(val2)
        g2 = pkg.graphs.CSR(g.rows, g.cols, g.rowptr, g.col, val2)
        for name, flags in _strategies(capi):
            plan = capi.Plan(g.rows, g.cols, rp, ci, k, flags)
            C = torch.full((g.rows, k), float("nan"), device=gpu)
            capi.csr_spmm(plan, rp, ci, v, Bd, C)
            _check(oracle, g, B, C.cpu().numpy(), f"unaligned k={k} {name}")
            capi.csr_spmm(plan, rp, ci, v2, Bd, C)
            _check(oracle, g2, B, C.cpu().numpy(), f"unaligned, new values k={k} {name}")
            # B and C one float into their buffers as well: the 16-byte accesses of the kernels are then
            # misaligned, which the hardware serves (more slowly); the result must not change
            Bu = torch.cat([torch.zeros(1, device=gpu), Bd.reshape(-1)])[1:].view(g.cols, k)
            Cu = torch.full((g.rows * k + 1,), float("nan"), device=gpu)[1:].view(g.rows, k)
            assert Bu.data_ptr() % 16 == 4 and Cu.data_ptr() % 16 == 4
            capi.csr_spmm(plan, rp, ci, v2, Bu, Cu)
            assert torch.equal(Cu, C), f"B and C at 4-byte alignment k={k} {name}"
            plan.destroy()


def test_bound_values(pkg, oracle, gpu):
    """hpspmm_plan_bind_values: same bits as the unbound call, another pointer drops the binding,
    binding again picks up values changed in place."""
    import torch
    capi = pkg.capi
    g = pkg.graphs.make_graph("c4_rmat", 0.004)
    k = 64
    B = pkg.graphs.make_dense("c4_rmat", g.cols, k)
    val2 = (g.val * np.float32(0.75) - np.float32(0.125)).astype(np.float32)
    g2 = pkg.graphs.CSR(g.rows, g.cols, g.rowptr, g.col, val2)
    rp, ci, v, vb, Bd = _to_dev(gpu, g.rowptr, g.col, g.val, val2, B)
    for name, flags in _strategies(capi):
        plan = capi.Plan(g.rows, g.cols, rp, ci, k, flags)
        run = lambda vals: (lambda C: (capi.csr_spmm(plan, rp, ci, vals, Bd, C), C.cpu().numpy())[1])(
            torch.full((g.rows, k), float("nan"), device=gpu))
        unbound = run(v)
        plan.bind_values(v)
        assert np.array_equal(run(v), unbound), f"{name}: bound result differs from the unbound one"
        assert np.array_equal(run(v), unbound), f"{name}: second bound call differs"
        other = run(vb)                      # another array: used as given, binding dropped
        _check(oracle, g2, B, other, f"bound, other pointer {name}")
        assert np.array_equal(run(v), unbound), f"{name}: first array after the binding was dropped"
        plan.bind_values(v)
        v.copy_(vb)                          # changed in place ...
        plan.bind_values(v)                  # ... and bound again
        assert np.array_equal(run(v), other), f"{name}: binding again must pick up the new values"
        plan.bind_values(None)
        assert np.array_equal(run(v), other), f"{name}: unbound call after unbinding"
        v.copy_(torch.from_numpy(g.val).to(gpu))
        plan.destroy()


def test_hip_graph_capture_and_replay(pkg, oracle, gpu):
    """One SpMM is kernel launches only (no allocation, no memset, no host synchronisation), so it can
    be captured in a HIP graph; every replay must see the current contents of val and B."""
    import torch
    capi = pkg.capi
    g = pkg.graphs.make_graph("c4_rmat", 0.004)
    # every strategy at a tuned row length, then the tiled forms of the three layouts that have one, at a row
    # length that is not a multiple of 4 (3 tiles of 64 columns behind a padded copy of B)
    tiled = [(n, f) for n, f in _strategies(capi) if n in ("sweep", "routed", "routed_sort_values", "cluster_seg")]
    operands = {}
    # and row tiles at row lengths of their own: B as it lies (aligned, at 4-byte alignment), B through the padded copy
    other = [("row_tiles_k100", capi.PLAN_DEFAULT, 100), ("row_tiles_k41", capi.PLAN_DEFAULT, 41),
             ("row_tiles_k3", capi.PLAN_DEFAULT, 3)]
    for name, flags, k in [(n, f, 64) for n, f in _strategies(capi)] + [(n + "_tiled", f, 173) for n, f in tiled] + other:
        if k not in operands:
            operands[k] = _to_dev(gpu, g.rowptr, g.col, g.val, pkg.graphs.make_dense("c4_rmat", g.cols, k))
        rp, ci, v, Bd = operands[k]
        plan = capi.Plan(g.rows, g.cols, rp, ci, k, flags)
        if name.endswith("_tiled"):
            assert plan.info["column_tiles"] == 3, (name, plan.info)
        if name.startswith("row_tiles"):
            assert plan.info["row_tiles"] > 0 and plan.info["launches_per_spmm"] == (2 if k == 3 else 1), (name, plan.info)
        C = torch.full((g.rows, k), float("nan"), device=gpu)
        eager = torch.empty_like(C)
        capi.csr_spmm(plan, rp, ci, v, Bd, eager)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                capi.csr_spmm(plan, rp, ci, v, Bd, C, side)
        torch.cuda.current_stream().wait_stream(side)
        for scale in (1.0, -0.5, 2.0):
            v.copy_(torch.from_numpy(g.val).to(gpu) * scale)
            capi.csr_spmm(plan, rp, ci, v, Bd, eager)      # the program's own eager work between replays
            torch.cuda.synchronize()
            C.fill_(float("nan"))
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(C, eager), f"{name}: replay with values x{scale} differs from the eager call"
        v.copy_(torch.from_numpy(g.val).to(gpu))
        del graph
        plan.destroy()


def test_auto_strategy_leaves_short_rows_unrouted(pkg, oracle, gpu):
    """Popular columns but no long rows: routing would move nothing, so the plan must stay with
    segments or whole rows; forced routing of the same matrix still gives the right result."""
    import torch
    capi = pkg.capi
    rng = np.random.default_rng(77)
    rows, cols, per_row, k = 450_000, 500_000, 40, 64             # 18 M nonzeros: beyond the rows strategy
    pop = rng.zipf(1.6, size=rows * per_row) % cols               # heavy-tailed column popularity
    col = np.sort(pop.reshape(rows, per_row), axis=1).astype(np.int32).ravel()
    rowptr = (np.arange(rows + 1, dtype=np.int64) * per_row).astype(np.int32)
    val = rng.uniform(-1, 1, col.size).astype(np.float32)
    g = pkg.graphs.CSR(rows, cols, rowptr, col, val)
    B = rng.standard_normal((cols, k)).astype(np.float32)
    C, info = _run(pkg, gpu, g, B, capi.PLAN_DEFAULT)
    assert info["strategy"] in (capi.STRATEGY_SEGMENTS, capi.STRATEGY_ROWS)
    lo, hi = 50_000, 54_000
    C64, S64 = oracle.csr_spmm_f64_rows(g.rowptr, g.col, g.val, B, lo, hi)
    err, _ = oracle.max_norm_err(C[lo:hi], C64, S64)
    assert err <= TOL
    # a quarter of it is within the rows strategy's range (row tiles), and without the tiles it is not
    sub = pkg.graphs.CSR(rows // 4, cols, rowptr[:rows // 4 + 1], col[:rows // 4 * per_row],
                         val[:rows // 4 * per_row])
    Cs, info_s = _run(pkg, gpu, sub, B, capi.PLAN_DEFAULT)
    assert info_s["strategy"] == capi.STRATEGY_ROWS
    err, _ = oracle.max_norm_err(Cs[:4000], *oracle.csr_spmm_f64_rows(sub.rowptr, sub.col, sub.val, B, 0, 4000))
    assert err <= TOL
    _, info_s = _run(pkg, gpu, sub, B, capi.PLAN_NO_ROW_TILES)
    assert info_s["strategy"] == capi.STRATEGY_SEGMENTS
    Cr, info_r = _run(pkg, gpu, g, B, capi.PLAN_FORCE_ROUTED)
    assert info_r["strategy"] == capi.STRATEGY_ROUTED
    err, _ = oracle.max_norm_err(Cr[lo:hi], C64, S64)
    assert err <= TOL
    # segments and routed add every row's products in the same (stored) order here: no row is routed
    Cs, info_s = _run(pkg, gpu, g, B, capi.PLAN_FORCE_SEGMENTS)
    assert info_s["strategy"] == capi.STRATEGY_SEGMENTS
    assert np.array_equal(Cs, Cr)


@pytest.mark.parametrize("k", [32, 64, 128])
def test_caller_supplied_row_order(pkg, oracle, gpu, k):
    """hpspmm_plan_create_ordered: any permutation of the rows gives the product at the original row
    numbers; identity, reversed, random and rows sorted by length; rectangular A included."""
    import torch
    capi = pkg.capi
    rng = np.random.default_rng(11)
    g = pkg.graphs.make_graph("c4_rmat", 0.004)
    rowptr, col, val = _random_csr(rng, 1500, 700, mean_deg=12.0, skew=2.0, empty_frac=0.3, sorted_unique=True)
    rect = pkg.graphs.CSR(1500, 700, rowptr, col, val)
    for graph in (g, rect):
        B = rng.standard_normal((graph.cols, k)).astype(np.float32)
        rp, ci, v, Bd = _to_dev(gpu, graph.rowptr, graph.col, graph.val, B)
        deg = np.diff(graph.rowptr)
        orders = {"identity": np.arange(graph.rows), "reversed": np.arange(graph.rows)[::-1],
                  "random": rng.permutation(graph.rows), "by length": np.argsort(-deg, kind="stable")}
        for name, order in orders.items():
            od, = _to_dev(gpu, order.astype(np.int32))
            plan = capi.Plan(graph.rows, graph.cols, rp, ci, k, 0, row_order=od)
            assert plan.info["strategy"] == capi.STRATEGY_ORDERED
            C = torch.full((graph.rows, k), float("nan"), device=gpu)
            capi.csr_spmm(plan, rp, ci, v, Bd, C)
            again = torch.full_like(C, float("nan"))
            capi.csr_spmm(plan, rp, ci, v, Bd, again)
            plan.destroy()
            assert torch.equal(C, again), f"{name}: not reproducible"
            _check(oracle, graph, B, C.cpu().numpy(), f"ordered {name} k={k}")
        bad = torch.zeros(graph.rows, dtype=torch.int32, device=gpu)          # not a permutation
        with pytest.raises(capi.HpSpmmError) as ei:
            capi.Plan(graph.rows, graph.cols, rp, ci, k, 0, row_order=bad)
        assert ei.value.code == capi.ERR_INVALID_ARG


def test_clustering_finds_planted_communities(pkg, oracle, gpu):
    """Label propagation in the plan: on the co-purchase-style graph (vertex ids carry no information, 46 %
    of the nonzeros stay inside communities of ~37) most of those nonzeros must end up reading B from LDS;
    a square matrix that is not symmetric, and one without any structure, still give the right product."""
    import torch
    capi = pkg.capi
    flags = capi.PLAN_CLUSTER | capi.PLAN_FORCE_SEGMENTS | capi.PLAN_NO_HUB_CACHE
    g = pkg.graphs.make_graph("c3_copurchase", 0.02)
    B = pkg.graphs.make_dense("c3_copurchase", g.cols, 64)
    C, info = _run(pkg, gpu, g, B, flags)
    assert info["strategy"] == capi.STRATEGY_ORDERED
    assert info["lds_served_nnz"] >= 0.3 * g.nnz, info
    _check(oracle, g, B, C, "clustered co-purchase graph")
    rng = np.random.default_rng(5)
    rowptr, col, val = _random_csr(rng, 3000, 3000, mean_deg=20.0, skew=1.5, empty_frac=0.1, sorted_unique=True)
    sq = pkg.graphs.CSR(3000, 3000, rowptr, col, val)
    Bs = rng.standard_normal((3000, 32)).astype(np.float32)
    C, info = _run(pkg, gpu, sq, Bs, flags)
    assert info["strategy"] == capi.STRATEGY_ORDERED
    _check(oracle, sq, Bs, C, "clustered unsymmetric square matrix")


def test_clustering_of_rectangular_matrices_and_with_a_diagonal(pkg, oracle, gpu):
    """The community structure must also be found when the matrix is not a plain graph: half the rows of
    the co-purchase-style graph (users x items, taken as the bipartite graph of rows and columns) and the
    same graph with a unit diagonal added (A + I, the form graph networks feed); a users x items matrix
    without communities is not reordered, and the search for them ends early."""
    import scipy.sparse as sp
    capi, graphs = pkg.capi, pkg.graphs
    g = graphs.make_graph("c3_copurchase", 0.1)          # 245k vertices, 12 M nonzeros
    A = sp.csr_matrix((g.val, g.col, g.rowptr), shape=(g.rows, g.cols))
    k = 64
    B = graphs.make_dense("c3_copurchase", g.cols, k)

    def csr_of(M):
        M = M.tocsr()
        M.sort_indices()
        return graphs.CSR(M.shape[0], M.shape[1], M.indptr.astype(np.int32), M.indices.astype(np.int32),
                          M.data.astype(np.float32))

    half = csr_of(A[: g.rows // 2])
    C, info = _run(pkg, gpu, half, B, capi.PLAN_DEFAULT)
    assert info["strategy"] == capi.STRATEGY_ORDERED, info
    assert info["lds_served_nnz"] >= 0.25 * half.nnz, info
    _check(oracle, half, B, C, "half the rows of the co-purchase graph")
    C2, _ = _run(pkg, gpu, half, B, capi.PLAN_DEFAULT)
    assert np.array_equal(C.view(np.uint32), C2.view(np.uint32))  # two plans: same order, same bits

    with_diag = csr_of(A + sp.identity(g.rows, dtype=np.float32, format="csr"))
    C, info = _run(pkg, gpu, with_diag, B, capi.PLAN_DEFAULT)
    assert info["strategy"] == capi.STRATEGY_ORDERED, info
    assert info["lds_served_nnz"] >= 0.3 * with_diag.nnz, info
    _check(oracle, with_diag, B, C, "co-purchase graph with a unit diagonal")

    plain = graphs.make_graph("h4_bipartite", 0.12)      # users x items, popular items, no communities
    Bp = graphs.make_dense("h4_bipartite", plain.cols, k)
    C, info = _run(pkg, gpu, plain, Bp, capi.PLAN_DEFAULT)
    assert info["strategy"] != capi.STRATEGY_ORDERED, info
    _check(oracle, plain, Bp, C, "users x items")


def test_extreme_shapes(pkg, oracle, gpu):
    """One dense row among singletons, a permutation matrix, a single column, a single row: the shapes
    that stress the carry chains, the row lists and the hot-column logic of every strategy."""
    capi = pkg.capi
    rng = np.random.default_rng(9)
    n = 300_000
    cases = {
        "dense row": (n, n, np.concatenate([[0, n], n + np.arange(1, n, dtype=np.int64)]).astype(np.int32),
                      np.concatenate([np.arange(n, dtype=np.int32), rng.integers(0, n, n - 1).astype(np.int32)]), 64),
        "permutation": (n, n, np.arange(n + 1, dtype=np.int32), rng.permutation(n).astype(np.int32), 32),
        "one column": (n, 1, (np.arange(n + 1, dtype=np.int64) * 4).astype(np.int32), np.zeros(4 * n, np.int32), 128),
        "one row": (1, n, np.array([0, n], np.int32), np.arange(n, dtype=np.int32), 32),
    }
    strategies = [("auto", capi.PLAN_DEFAULT), ("rows", capi.PLAN_FORCE_ROWS),
                  ("rows_csr", capi.PLAN_FORCE_ROWS | capi.PLAN_NO_ROW_TILES),
                  ("seg", capi.PLAN_FORCE_SEGMENTS), ("seg32", capi.PLAN_FORCE_SEGMENTS
                  | capi.plan_segment_shift(5)), ("routed", capi.PLAN_FORCE_ROUTED),
                  ("cluster", capi.PLAN_CLUSTER | capi.PLAN_FORCE_SEGMENTS | capi.PLAN_NO_HUB_CACHE)]
    for what, (rows, cols, rowptr, col, k) in cases.items():
        val = rng.uniform(-1, 1, col.size).astype(np.float32)
        g = pkg.graphs.CSR(rows, cols, rowptr, col, val)
        B = rng.standard_normal((cols, k)).astype(np.float32)
        hi = min(rows, 64)
        C64, S64 = oracle.csr_spmm_f64_rows(g.rowptr, g.col, g.val, B, 0, hi)
        for name, flags in strategies:
            C, _ = _run(pkg, gpu, g, B, flags)
            assert not np.isnan(C).any(), f"{what} {name}: C not fully written"
            err, _ = oracle.max_norm_err(C[:hi], C64, S64)
            assert err <= TOL, f"{what} {name}: normalised error {err:.3e}"


def test_row_tiles_layout_and_fallback(pkg, oracle, gpu):
    """The rows strategy builds row tiles (every size class of row present: 1, 2, 4, 8 slots, several
    tiles) unless padding would dominate (mostly empty rows): then it walks the CSR arrays.  Both agree
    with the oracle; the tile layout shows in the plan's workspace."""
    capi = pkg.capi
    rng = np.random.default_rng(21)
    # one row of every length 0..200, shuffled, twice over
    lens = rng.permutation(np.concatenate([np.arange(201), np.arange(201)])).astype(np.int64)
    rows, cols = lens.size, 5000
    rowptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    col = rng.integers(0, cols, int(lens.sum())).astype(np.int32)
    val = rng.uniform(-1, 1, col.size).astype(np.float32)
    g = pkg.graphs.CSR(rows, cols, rowptr, col, val)
    for k in (32, 64, 128):
        B = rng.standard_normal((cols, k)).astype(np.float32)
        C, info = _run(pkg, gpu, g, B, capi.PLAN_DEFAULT)
        assert info["strategy"] == capi.STRATEGY_ROWS
        assert info["row_tiles"] * 64 >= col.size and info["workspace_bytes"] >= 4 * col.size
        _check(oracle, g, B, C, f"all row lengths k={k} tiles")
        C2, info2 = _run(pkg, gpu, g, B, capi.PLAN_NO_ROW_TILES)
        assert info2["strategy"] == capi.STRATEGY_ROWS and info2["row_tiles"] == 0
        _check(oracle, g, B, C2, f"all row lengths k={k} csr")
        # the groups of tiles dealt to the XCDs four at a time instead of one: the same tiles, the same bits
        Cr, info_r = _run(pkg, gpu, g, B, capi.PLAN_DEFAULT, options={"row_tiles_chunk_log2": 2})
        assert info_r["row_tiles"] == info["row_tiles"] and np.array_equal(C, Cr)
    # rows beyond 512 nonzeros get a workgroup each (8 wavefronts; 16 when a row exceeds 8192),
    # next to rows of 65..512 that one wavefront works through
    for longest in (5000, 9000):
        lens = rng.permutation(np.concatenate([np.arange(0, 520, 7), [513, 600, 1025, longest],
                                               np.full(300, 3)])).astype(np.int64)
        rows = lens.size
        rowptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        col = rng.integers(0, cols, int(lens.sum())).astype(np.int32)
        val = rng.uniform(-1, 1, col.size).astype(np.float32)
        g = pkg.graphs.CSR(rows, cols, rowptr, col, val)
        for k in (32, 128):
            B = rng.standard_normal((cols, k)).astype(np.float32)
            C, info = _run(pkg, gpu, g, B, capi.PLAN_DEFAULT)
            assert info["strategy"] == capi.STRATEGY_ROWS and info["row_tiles"] * 64 >= col.size
            _check(oracle, g, B, C, f"long rows up to {longest} k={k}")
            again, _ = _run(pkg, gpu, g, B, capi.PLAN_DEFAULT)
            assert np.array_equal(C, again), "workgroup-per-row reduction must be bit-reproducible"
            Cr, _ = _run(pkg, gpu, g, B, capi.PLAN_DEFAULT, options={"row_tiles_chunk_log2": 1})
            assert np.array_equal(C, Cr), "dealing the tiles in chunks must not change the result"
    # 400k rows, 2k nonzeros: 50k tiles of padding for 2k entries - not built
    rows = 400_000
    lens = np.zeros(rows, np.int64)
    lens[rng.choice(rows, 1000, replace=False)] = 2
    rowptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    col = rng.integers(0, 777, 2000).astype(np.int32)
    val = rng.uniform(-1, 1, 2000).astype(np.float32)
    g = pkg.graphs.CSR(rows, 777, rowptr, col, val)
    B = rng.standard_normal((777, 32)).astype(np.float32)
    C, info = _run(pkg, gpu, g, B, capi.PLAN_DEFAULT)
    assert info["strategy"] == capi.STRATEGY_ROWS and info["row_tiles"] == 0
    _check(oracle, g, B, C, "mostly empty rows")


@pytest.mark.parametrize("name,scale", [("h3_grid", 0.03), ("c4_rmat", 0.1), ("c1_citation", 4.0)])
def test_row_tile_chunks_per_xcd(pkg, oracle, gpu, name, scale):
    """hpspmm_plan_options.row_tiles_chunk_log2: 2^n consecutive groups of row tiles go to an XCD at a
    time (the groups of the long rows still one by one); from 2^21 nonzeros that is the default, with n
    picked by the size.  Thousands of tiles, every class of row, the long rows of an R-MAT graph on
    workgroups of their own, chunks of 2 to 512 groups: the oracle bar and the bits of the dealing
    one by one."""
    capi = pkg.capi
    g = pkg.graphs.make_graph(name, scale)
    for k in (32, 64, 128):
        B = pkg.graphs.make_dense(name, g.cols, k)
        C, info = _run(pkg, gpu, g, B, capi.PLAN_FORCE_ROWS, options={"row_tiles_chunk_log2": -1})
        assert info["strategy"] == capi.STRATEGY_ROWS and info["row_tiles"] > 1000
        _check(oracle, g, B, C, f"{name} k={k} one by one")
        for n in (0, 1, 5, 9):
            Cr, info_r = _run(pkg, gpu, g, B, capi.PLAN_FORCE_ROWS, options={"row_tiles_chunk_log2": n})
            assert info_r["row_tiles"] == info["row_tiles"]
            assert np.array_equal(C, Cr), f"{name} k={k} chunks of 2^{n}"


@pytest.mark.parametrize("k", [1, 2, 3, 4, 5, 7, 20, 31, 33, 36, 41, 63, 65, 100, 130, 172, 259])
def test_row_tiles_at_any_row_length(pkg, oracle, gpu, k):
    """Row tiles at a row length outside the tuned set: 32-column tiles, the last one narrower; B as it
    lies (K a multiple of 4: aligned gathers; else 16-byte gathers at 4-byte alignment, the lane of a
    row's last columns reading the row's last four floats) or through the plan's copy with rows padded
    to a multiple of 32 floats (one more launch).  Every size class of row, rows that get a whole
    workgroup, empty rows; B and C inside larger allocations whose surroundings hold NaN (B) and a
    marker (C): nothing beyond them may be read into the result or written.  Both forms give the same
    bits (the same gathers in the same order), and two runs of one form do."""
    import torch
    capi = pkg.capi
    rng = np.random.default_rng(100 + k)
    cols = 3000
    lens = rng.permutation(np.concatenate([np.arange(0, 140), np.arange(0, 520, 11), [513, 700, 1500, 9000],
                                           np.zeros(40, np.int64)])).astype(np.int64)
    rows = lens.size
    rowptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    col = rng.integers(0, cols, int(lens.sum())).astype(np.int32)
    col[-3:] = cols - 1  # the last row of B is gathered: a read past its end would reach the NaN behind it
    val = rng.uniform(-1, 1, col.size).astype(np.float32)
    g = pkg.graphs.CSR(rows, cols, rowptr, col, val)
    B = rng.standard_normal((cols, k)).astype(np.float32)
    rp, ci, v = _to_dev(gpu, g.rowptr, g.col, g.val)
    guard = 64
    Bbig = torch.full((guard + cols * k + guard,), float("nan"), device=gpu)
    Bbig[guard:guard + cols * k] = torch.from_numpy(B).to(gpu).reshape(-1)
    Cbig = torch.full((guard + rows * k + guard,), 12345.0, device=gpu)
    Bd, Cd = Bbig[guard:guard + cols * k].view(cols, k), Cbig[guard:guard + rows * k].view(rows, k)
    results = {}
    for form, pad in (("as it lies", 1), ("padded copy", 2)):
        plan = capi.Plan(rows, cols, rp, ci, k, capi.PLAN_DEFAULT, options={"row_tiles_pad": pad})
        info = plan.info
        padded = k < 4 or (pad == 2 and k % 32 != 0)  # (a row of fewer than 4 floats is always read from a copy)
        assert info["strategy"] == capi.STRATEGY_ROWS and info["row_tiles"] * 64 >= col.size, info
        assert info["launches_per_spmm"] == (2 if padded else 1) and info["k"] == k, info
        for attempt in range(2):
            Cd.fill_(float("nan"))
            capi.csr_spmm(plan, rp, ci, v, Bd, Cd)
            torch.cuda.synchronize()
            C = Cd.cpu().numpy().copy()
            _check(oracle, g, B, C, f"k={k} {form}")
            assert bool((Cbig[:guard] == 12345.0).all()) and bool((Cbig[guard + rows * k:] == 12345.0).all()), \
                f"k={k} {form}: wrote outside C"
            assert np.array_equal(results.setdefault(form, C), C), "bit-reproducible"
        plan.destroy()
    assert np.array_equal(results["as it lies"], results["padded copy"])
    # no row beyond 512 nonzeros: one wavefront per row tile, in workgroups of one (small grid) or four
    for scale in (0.25, 4.0):
        g = pkg.graphs.make_graph("c1_citation", scale)
        B = pkg.graphs.dense_normal(g.cols, k, 5)
        C, info = _run(pkg, gpu, g, B, capi.PLAN_FORCE_ROWS)
        assert info["strategy"] == capi.STRATEGY_ROWS and info["row_tiles"] > 0, info
        _check(oracle, g, B, C, f"k={k} citation graph x {scale}")


def test_auto_choice_at_mid_size(pkg, oracle, gpu):
    """Between the small and the large graphs: a community graph of 6 M nonzeros gets the ordered
    strategy by itself (label propagation finds its clusters), an R-MAT of the same size - hot columns,
    no communities - does not and stays with whole rows; both agree with the oracle."""
    capi = pkg.capi
    for name, scale, k, want in (("c3_copurchase", 0.05, 64, capi.STRATEGY_ORDERED),
                                 ("c4_rmat", 0.0625, 32, capi.STRATEGY_ROWS)):
        g = pkg.graphs.make_graph(name, scale)
        B = pkg.graphs.make_dense(name, g.cols, k)
        C, info = _run(pkg, gpu, g, B, capi.PLAN_DEFAULT)
        assert info["strategy"] == want, (name, info)
        if want == capi.STRATEGY_ROWS:
            assert info["row_tiles"] > 0
        else:
            assert info["lds_served_nnz"] >= 0.15 * g.nnz
        lo, hi = g.rows // 3, g.rows // 3 + 3000
        C64, S64 = oracle.csr_spmm_f64_rows(g.rowptr, g.col, g.val, B, lo, hi)
        err, _ = oracle.max_norm_err(C[lo:hi], C64, S64)
        assert err <= TOL, f"{name}: normalised error {err:.3e}"
        heavy = np.argsort(-np.diff(g.rowptr))[:4]
        for r in heavy:
            C64, S64 = oracle.csr_spmm_f64_rows(g.rowptr, g.col, g.val, B, int(r), int(r) + 1)
            err, _ = oracle.max_norm_err(C[r:r + 1], C64, S64)
            assert err <= TOL, f"{name}: heaviest rows: normalised error {err:.3e}"


def test_sweep_strategy(pkg, oracle, gpu):
    """The sweep strategy (row accumulators in LDS, all wavefronts walking B window by window): chosen
    by itself for a graph of long rows whose B is beyond the L2s, two launches, bit-reproducible across
    calls and across plans, same bits with bound values; PLAN_NO_SWEEP gives the routed strategy back."""
    import torch
    capi = pkg.capi
    g = pkg.graphs.make_graph("c2_social", 0.1)
    for k in (32, 64, 128):
        B = pkg.graphs.make_dense("c2_social", g.cols, k)
        C1, info = _run(pkg, gpu, g, B, capi.PLAN_FORCE_SWEEP)
        assert info["strategy"] == capi.STRATEGY_SWEEP and info["launches_per_spmm"] == 2, info
        _check(oracle, g, B, C1, f"sweep k={k}")
        C2, info2 = _run(pkg, gpu, g, B, capi.PLAN_FORCE_SWEEP)
        assert info2 == info and np.array_equal(C1, C2), "two sweep plans, different bits"
        rp, ci, v, Bd = _to_dev(gpu, g.rowptr, g.col, g.val, B)
        plan = capi.Plan(g.rows, g.cols, rp, ci, k, capi.PLAN_FORCE_SWEEP)
        C = torch.full((g.rows, k), float("nan"), device=gpu)
        plan.bind_values(v)
        capi.csr_spmm(plan, rp, ci, v, Bd, C)
        torch.cuda.synchronize()
        assert np.array_equal(C.cpu().numpy(), C1), "bound values, different bits"
        plan.destroy()
    # automatic choice: 12 MB of B and 9.6 M nonzeros in rows of 400 qualify, 3 MB of B (K = 32) do not
    B = pkg.graphs.make_dense("c2_social", g.cols, 128)
    _, info = _run(pkg, gpu, g, B, capi.PLAN_DEFAULT)
    assert info["strategy"] == capi.STRATEGY_SWEEP, info
    _, info = _run(pkg, gpu, g, B, capi.PLAN_NO_SWEEP)
    assert info["strategy"] == capi.STRATEGY_ROUTED, info
    B = pkg.graphs.make_dense("c2_social", g.cols, 32)
    _, info = _run(pkg, gpu, g, B, capi.PLAN_DEFAULT)
    assert info["strategy"] != capi.STRATEGY_SWEEP, info


def test_sweep_layout_corners(pkg, oracle, gpu):
    """Forced sweep plans whose layout is all corners: windows of a few columns, pieces of 64 nonzeros
    (most rows split, several bands), a lead of one window; a matrix with empty rows and a row of
    every column; columns out of order within the rows, duplicates included (the layout is then built
    from a sorted copy, and the values are still read where the caller has them)."""
    capi = pkg.capi
    rng = np.random.default_rng(11)
    cases = []
    g = pkg.graphs.make_graph("c2_social", 0.05)
    cases.append(("social", g))
    # empty rows, one-nonzero rows, one dense row, a last column that only the dense row uses
    rows, cols = 3000, 5000
    deg = rng.integers(0, 60, rows)
    deg[rng.random(rows) < 0.3] = 0
    deg[7] = cols
    deg[11] = 1
    rowptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int32)
    col = np.concatenate([np.sort(rng.choice(cols - 1 if d < cols else cols, int(d), replace=False)) for d in deg]).astype(np.int32)
    val = rng.uniform(-1, 1, col.size).astype(np.float32)
    cases.append(("ragged", pkg.graphs.CSR(rows, cols, rowptr, col, val)))
    for opts in ({}, {"sweep_window_log2": 12, "sweep_limit": 64, "sweep_lead": 1},
                 {"sweep_window_log2": 30, "sweep_limit": 1, "sweep_spin": -1}):
        for name, g in cases:
            if opts.get("sweep_limit") == 1 and name == "social":
                continue  # one piece per nonzero: only for the small matrix
            for k in (32, 64, 128):
                B = pkg.graphs.dense_normal(g.cols, k, 5)
                C, info = _run(pkg, gpu, g, B, capi.PLAN_FORCE_SWEEP, options=opts)
                assert info["strategy"] == capi.STRATEGY_SWEEP, (name, opts, info)
                _check(oracle, g, B, C, f"sweep corners {name} k={k} {opts}")
    # columns out of order within the rows (with duplicates): the sweep layout from a sorted copy
    rowptr, col, val = _random_csr(rng, 500, 700, 20, 1.5, 0.1, sorted_unique=False)
    g = pkg.graphs.CSR(500, 700, rowptr, col, val)
    for k in (32, 64, 128):
        B = pkg.graphs.dense_normal(700, k, 6)
        for opts in ({}, {"sweep_window_log2": 12, "sweep_limit": 16, "sweep_lead": 1}):
            C, info = _run(pkg, gpu, g, B, capi.PLAN_FORCE_SWEEP, options=opts)
            assert info["strategy"] == capi.STRATEGY_SWEEP, info
            _check(oracle, g, B, C, f"sweep forced on unsorted columns k={k} {opts}")
    # the social graph with every row's entries shuffled: the same layout as from the sorted rows, so the
    # same sums in the same order - bit for bit the product of the sorted matrix - and the default plan
    # still picks the sweep
    g = pkg.graphs.make_graph("c2_social", 0.1)
    perm = np.arange(g.nnz)
    for r in range(g.rows):
        lo, hi = g.rowptr[r], g.rowptr[r + 1]
        perm[lo:hi] = lo + rng.permutation(hi - lo)
    shuffled = pkg.graphs.CSR(g.rows, g.cols, g.rowptr, g.col[perm], g.val[perm])
    B = pkg.graphs.dense_normal(g.cols, 128, 7)
    C_sorted, info_sorted = _run(pkg, gpu, g, B, capi.PLAN_DEFAULT)
    C_shuffled, info_shuffled = _run(pkg, gpu, shuffled, B, capi.PLAN_DEFAULT)
    assert info_sorted["strategy"] == info_shuffled["strategy"] == capi.STRATEGY_SWEEP
    _check(oracle, shuffled, B, C_shuffled, "social graph with shuffled rows")
    assert np.array_equal(C_sorted, C_shuffled)


def test_sweep_is_not_chosen_for_a_banded_matrix(pkg, oracle, gpu):
    """Long rows over a large B, but every row inside a narrow band of columns: the walk over B would
    leave each wavefront busy in a few windows of its own, so the plan keeps to another strategy (and
    the forced sweep still gives the right product)."""
    capi = pkg.capi
    rng = np.random.default_rng(5)
    rows = cols = 40000
    per_row, half_band = 128, 600
    centre = np.arange(rows)
    lo = np.clip(centre - half_band, 0, cols - 2 * half_band)
    col = np.sort(lo[:, None] + np.argsort(rng.random((rows, 2 * half_band)), axis=1)[:, :per_row], axis=1)
    rowptr = (np.arange(rows + 1) * per_row).astype(np.int32)
    g = pkg.graphs.CSR(rows, cols, rowptr, col.reshape(-1).astype(np.int32),
                       rng.uniform(-1, 1, rows * per_row).astype(np.float32))
    B = pkg.graphs.dense_normal(cols, 64, 8)
    C, info = _run(pkg, gpu, g, B, capi.PLAN_DEFAULT)
    assert info["strategy"] != capi.STRATEGY_SWEEP, info
    _check(oracle, g, B, C, "banded, default plan")
    C, info = _run(pkg, gpu, g, B, capi.PLAN_FORCE_SWEEP)
    assert info["strategy"] == capi.STRATEGY_SWEEP, info
    _check(oracle, g, B, C, "banded, forced sweep")


@pytest.mark.parametrize("k,tile,ntiles", [(16, 32, 1), (30, 32, 1), (40, 64, 1), (41, 64, 1), (96, 128, 1),
                                           (127, 128, 1), (160, 64, 3), (173, 64, 3), (192, 64, 3), (200, 128, 2),
                                           (256, 128, 2), (259, 64, 5), (384, 128, 3)])
def test_column_tiles(pkg, oracle, gpu, k, tile, ntiles):
    """A row length from 16 up that is not a tuned one goes through the tuned layouts (sweep, routed,
    ordered) one column tile after the other, the last tile narrower than the layout when the width
    does not divide the row length (its surplus lanes idle); a row length that is not a multiple of 4
    is read through a copy of B with padded rows, one launch more, and written to C in place (B and C
    sit inside larger allocations here, NaN behind B, a sentinel behind C): the plan reports that strategy,
    the full row length and one set of launches per tile; the product meets the oracle's bar; a full
    tile t of C has the bits of the product with columns [t * tile, (t + 1) * tile) of B alone (same
    layout, same order of additions); bound values give the same bits.  Without a tuned layout the
    plan is the one for any row length."""
    import torch
    capi = pkg.capi
    cases = [("c2_social", 0.02, "sweep", capi.PLAN_FORCE_SWEEP, capi.STRATEGY_SWEEP),
             ("c4_rmat", 0.004, "routed", capi.PLAN_FORCE_ROUTED | capi.plan_routed_row_log2(2), capi.STRATEGY_ROUTED),
             ("c4_rmat", 0.004, "routed_hub", capi.PLAN_FORCE_ROUTED | capi.PLAN_ROUTED_SORT_VALUES | capi.plan_hub_log2(9)
              | capi.plan_routed_row_log2(2) | capi.plan_routed_phases(3), capi.STRATEGY_ROUTED),
             ("c3_copurchase", 0.01, "cluster", capi.PLAN_CLUSTER | capi.PLAN_FORCE_SEGMENTS | capi.PLAN_NO_HUB_CACHE,
              capi.STRATEGY_ORDERED)]
    for name, scale, label, flags, strategy in cases:
        g = pkg.graphs.make_graph(name, scale)
        B = pkg.graphs.make_dense(name, g.cols, k)
        C, info = _run(pkg, gpu, g, B, flags)
        what = f"{name} k={k} {label}"
        assert info["strategy"] == strategy and info["k"] == k and info["column_tiles"] == ntiles, (what, info)
        _check(oracle, g, B, C, what)
        for t in sorted(t for t in {0, k // tile - 1} if t >= 0 and (t + 1) * tile <= k):  # full tiles only
            Bt = np.ascontiguousarray(B[:, t * tile:(t + 1) * tile])
            Ct, info_t = _run(pkg, gpu, g, Bt, flags)
            assert info_t["strategy"] == strategy
            assert info_t["launches_per_spmm"] * ntiles == info["launches_per_spmm"] - (1 if k % 4 else 0)
            assert np.array_equal(C[:, t * tile:(t + 1) * tile], Ct), f"{what}: tile {t} differs from the product of that tile alone"
        rp, ci, v = _to_dev(gpu, g.rowptr, g.col, g.val)
        pad = 64
        Bbig = torch.full((g.cols * k + pad,), float("nan"), device=gpu)
        Bbig[:g.cols * k] = torch.from_numpy(B).to(gpu).reshape(-1)
        Cbig = torch.full((g.rows * k + pad,), 12345.0, device=gpu)
        Bd, Cb = Bbig[:g.cols * k].view(g.cols, k), Cbig[:g.rows * k].view(g.rows, k)
        Cb.fill_(float("nan"))
        plan = capi.Plan(g.rows, g.cols, rp, ci, k, flags)
        plan.bind_values(v)
        capi.csr_spmm(plan, rp, ci, v, Bd, Cb)
        torch.cuda.synchronize()
        assert np.array_equal(Cb.cpu().numpy(), C), f"{what}: bound values, different bits"
        assert bool((Cbig[g.rows * k:] == 12345.0).all()), f"{what}: wrote past the last row of C"
        plan.destroy()
    # a caller's row order
    g = pkg.graphs.make_graph("c3_copurchase", 0.01)
    B = pkg.graphs.make_dense("c3_copurchase", g.cols, k)
    rp, ci, v, Bd = _to_dev(gpu, g.rowptr, g.col, g.val, B)
    order = np.random.default_rng(5).permutation(g.rows).astype(np.int32)
    od, = _to_dev(gpu, order)
    plan = capi.Plan(g.rows, g.cols, rp, ci, k, 0, row_order=od)
    assert plan.info["strategy"] == capi.STRATEGY_ORDERED and plan.info["k"] == k
    Co = torch.full((g.rows, k), float("nan"), device=gpu)
    capi.csr_spmm(plan, rp, ci, v, Bd, Co)
    torch.cuda.synchronize()
    _check(oracle, g, B, Co.cpu().numpy(), f"row order k={k}")
    plan.destroy()
    # small and unforced: no tiles, the plan for any multiple of 4
    _, info = _run(pkg, gpu, g, B, capi.PLAN_DEFAULT)
    assert info["strategy"] in (capi.STRATEGY_ROWS, capi.STRATEGY_SEGMENTS) and info["k"] == k and info["column_tiles"] == 1, info
