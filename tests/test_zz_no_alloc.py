"""hpspmm_csr_spmm_static: the entry point that allocates nothing (its workspace is an array inside
the library's device image) against hpspmm_csr_spmm with a plan, through the C ABI.

Bar: the same as every SpMM parity test here - |C - C_f64| <= 1e-4 * sum_j |a_ij| |b_jk| against
the CPU oracle, exact zeros on empty rows - and, since both entry points run the same kernels,
bit-identical output when the plan is forced to the segment length the static entry point picks.
Two calls in a row share the static workspace; the second is smaller, so stale contents of the
first would show.
"""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

TOL = 1e-4


def _static_shift(nnz, k):
    """Segment length (log2) hpspmm_csr_spmm_static uses: the plan's rule, then raised until the
    carry slots fit 2^22 floats."""
    p = 64 // (k // 4)
    shift = 5
    while shift < 9 and (nnz >> (shift + 1)) // p >= 256 * 4 * 16:
        shift += 1
    while 2 * -(-nnz // (1 << shift)) * k > (1 << 22):
        shift += 1
    return shift


def _both(pkg, oracle, gpu, g, B, what):
    import torch
    capi = pkg.capi
    k = B.shape[1]
    dev = [torch.from_numpy(np.ascontiguousarray(a)).to(gpu) for a in (g.rowptr, g.col, g.val, B)]
    rp, ci, v, Bd = dev
    C_static = torch.empty((g.rows, k), device=gpu)
    # a first launch from the library loads its device image (code and the static workspace) onto the
    # GPU; what the entry point itself allocates is measured after that
    capi.fill_f32(C_static, float("nan"))
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    capi.csr_spmm_static(g.rows, g.cols, rp, ci, v, Bd, C_static)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before, "the static entry point must not allocate device memory"
    shift = _static_shift(g.nnz, k)
    flags = capi.PLAN_FORCE_SEGMENTS | capi.PLAN_NO_HUB_CACHE | capi.PLAN_NO_ROUTED | capi.PLAN_NO_CLUSTER
    if shift <= 15:
        flags |= capi.plan_segment_shift(shift)
    plan = capi.Plan(g.rows, g.cols, rp, ci, k, flags)
    C_plan = torch.full((g.rows, k), float("nan"), device=gpu)
    capi.csr_spmm(plan, rp, ci, v, Bd, C_plan)
    torch.cuda.synchronize()
    seg = plan.info["segment_length"]
    plan.destroy()
    a, b = C_static.cpu().numpy(), C_plan.cpu().numpy()
    C64, S64 = oracle.csr_spmm_f64(g.rowptr, g.col, g.val, B)
    for name, got in (("static", a), ("plan", b)):
        err, pos = oracle.max_norm_err(got, C64, S64)
        assert err <= TOL, f"{what} {name}: normalised error {err:.3e} at {pos}"
        assert not got[np.diff(g.rowptr) == 0].any(), f"{what} {name}: empty rows must be exact zeros"
    if seg == 1 << shift:
        assert np.array_equal(a, b), f"{what}: same kernels, same segment length: bits must agree"
    return a


@pytest.mark.parametrize("k", [128, 32, 64])
def test_static_entry_matches_planned_entry(pkg, oracle, gpu, k):
    graphs = pkg.graphs
    big = graphs.make_graph("c4_rmat", 0.032)      # ~3.7 M nonzeros, hub rows split over many segments, empty rows
    assert (1 << 21) < big.nnz <= (1 << 22)
    small = graphs.make_graph("c2_social", 0.01)   # second call: smaller, other shape, long rows
    assert small.nnz < big.nnz
    first = _both(pkg, oracle, gpu, big, graphs.make_dense("c4_rmat", big.cols, k), f"first call k={k}")
    _both(pkg, oracle, gpu, small, graphs.make_dense("c2_social", small.cols, k), f"second call k={k}")
    # and the first input again: the workspace now holds the second call's leftovers
    again = _both(pkg, oracle, gpu, big, graphs.make_dense("c4_rmat", big.cols, k), f"third call k={k}")
    assert np.array_equal(first, again)


def test_static_entry_limits_and_edges(pkg, oracle, gpu):
    import torch
    capi = pkg.capi
    L = capi.lib()
    fake = ctypes.c_void_p(4096)  # never dereferenced: the size checks come first
    too_many = (1 << 22) + 1
    assert L.hpspmm_csr_spmm_static(8, 8, too_many, fake, fake, fake, fake, 32, fake, None) == capi.ERR_INVALID_ARG
    assert b"static workspace" in L.hpspmm_last_error()
    assert L.hpspmm_csr_spmm_static(8, 8, 4, fake, fake, fake, fake, 48, fake, None) == capi.ERR_INVALID_ARG
    assert L.hpspmm_csr_spmm_static(8, 8, 4, None, fake, fake, fake, 32, fake, None) == capi.ERR_INVALID_ARG
    # no nonzeros at all: every row of a poisoned C becomes zero
    rp = torch.zeros(6, dtype=torch.int32, device=gpu)
    ci = torch.zeros(0, dtype=torch.int32, device=gpu)
    v = torch.zeros(0, dtype=torch.float32, device=gpu)
    B = torch.ones((7, 64), device=gpu)
    C = torch.full((5, 64), float("nan"), device=gpu)
    capi.csr_spmm_static(5, 7, rp, ci, v, B, C)
    torch.cuda.synchronize()
    assert not C.cpu().numpy().any()
    # exactly at the limit: 2^22 nonzeros, one dense-ish row among short ones
    rng = np.random.default_rng(3)
    rows, cols, k = 4096, 4096, 32
    deg = np.full(rows, (1 << 22) // rows, dtype=np.int64)
    rowptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int32)
    col = np.concatenate([np.sort(rng.choice(cols, size=int(d), replace=False)) for d in deg]).astype(np.int32)
    val = rng.uniform(-1, 1, col.size).astype(np.float32)
    g = pkg.graphs.CSR(rows, cols, rowptr, col, val)
    assert g.nnz == 1 << 22
    _both(pkg, oracle, gpu, g, rng.standard_normal((cols, k)).astype(np.float32), "at the limit")


def test_static_entry_under_graph_capture(pkg, oracle, gpu):
    """After hpspmm_static_workspace_init the entry point is launches only, so it can be captured: the
    replays (with the program's own eager calls between them) give the bits of the eager call."""
    import torch
    capi = pkg.capi
    capi.static_workspace_init()
    capi.static_workspace_init()  # later calls return at once
    g = pkg.graphs.make_graph("c4_rmat", 0.004)
    k = 64
    B = pkg.graphs.make_dense("c4_rmat", g.cols, k)
    rp, ci, v, Bd = [torch.from_numpy(np.ascontiguousarray(a)).to(gpu) for a in (g.rowptr, g.col, g.val, B)]
    C = torch.full((g.rows, k), float("nan"), device=gpu)
    eager = torch.empty_like(C)
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            capi.csr_spmm_static(g.rows, g.cols, rp, ci, v, Bd, C, side)
    torch.cuda.current_stream().wait_stream(side)
    for scale in (1.0, -0.5, 2.0):
        v.copy_(torch.from_numpy(g.val).to(gpu) * scale)
        capi.csr_spmm_static(g.rows, g.cols, rp, ci, v, Bd, eager)
        torch.cuda.synchronize()
        C.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(C, eager), f"replay with values x{scale} differs from the eager call"
    C64, S64 = oracle.csr_spmm_f64(g.rowptr, g.col, (g.val * 2.0).astype(np.float32), B)
    err, pos = oracle.max_norm_err(C.cpu().numpy(), C64, S64)
    assert err <= TOL, f"normalised error {err:.3e} at {pos}"
