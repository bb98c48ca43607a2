"""Generator families that none of the plan's thresholds was chosen on (preferential attachment,
an R-MAT with a flatter quadrant law, a 9-point mesh with random long-range entries, a rectangular
users x items matrix with Zipf popularity, blocks of mixed sizes along the diagonal, uniformly
placed nonzeros, users x items with communities): the default plan's product against the float64 oracle on slabs of rows, and the
default plan's time against every strategy forced on the same matrix.

Sizes here: about 1.5 M and 12 M nonzeros (the 100 M size of every family is part of the committed
table made by `bench.py --strategy-table`, which times the same comparison)."""
import importlib
import importlib.util
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOL = 1e-5           # |C - C64| <= TOL * (|A| |B|): ten times tighter than the bar of the other parity tests (1e-4)
# The default plan against the fastest forced strategy: within 10 % (the committed table has it within
# 7.5 % on every line of 12 M nonzeros), plus the 2 % that two timings of one plan differ by; on the
# matrices of 1.5 M nonzeros, where an SpMM takes 12 to 60 us, within 8 us (largest in the table: 5.5).
MAX_GAP = 0.12
MAX_GAP_US = 8.0


def _bench():
    spec = importlib.util.spec_from_file_location("bench_module", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


@pytest.fixture(scope="module")
def bench():
    return _bench()


@pytest.mark.parametrize("scale", [0.015, 0.12])
@pytest.mark.parametrize("family", ["h1_prefattach", "h2_rmat", "h3_grid", "h4_bipartite", "h5_blocks", "h6_uniform100",
                                    "h7_groups"])
def test_held_out_family(pkg, oracle, gpu, bench, family, scale):
    import torch
    capi, graphs = pkg.capi, pkg.graphs
    g = graphs.make_graph(family, scale)
    assert 1.0e6 <= g.nnz <= 1.6e7
    stream = torch.cuda.current_stream()
    rp, ci, v = (torch.from_numpy(a).to(gpu) for a in (g.rowptr, g.col, g.val))
    for k in (32, 64, 128):
        B = graphs.make_dense(family, g.cols, k)
        Bd = torch.from_numpy(B).to(gpu)
        # parity: default plan, C poisoned first, the oracle on three slabs of rows
        C = torch.full((g.rows, k), float("nan"), device=gpu)
        plan = capi.Plan(g.rows, g.cols, rp, ci, k)
        capi.csr_spmm(plan, rp, ci, v, Bd, C)
        torch.cuda.synchronize()
        plan.destroy()
        assert not torch.isnan(C).any().item(), f"{family} x{scale} K={k}: C not fully written"
        slab = min(g.rows, 4096)
        for lo in (0, (g.rows - slab) // 2, g.rows - slab):
            got = C[lo:lo + slab].cpu().numpy()
            C64, S64 = oracle.csr_spmm_f64_rows(g.rowptr, g.col, g.val, B, lo, lo + slab)
            err, pos = oracle.max_norm_err(got, C64, S64)
            assert err <= TOL, f"{family} x{scale} K={k}: rows [{lo},{lo + slab}) normalised error {err:.3e} at {pos}"
        # choice: the default plan against every forced strategy
        t, chosen = bench.strategy_times(capi, g, rp, ci, v, Bd, C, k, stream)
        best_name, best = min(((n, x) for n, x in t.items() if n != "auto" and x is not None), key=lambda nx: nx[1])
        gap = t["auto"] - best
        if gap > max(MAX_GAP * best, MAX_GAP_US):
            # one more measurement before the verdict (the smaller of the two for every strategy): a single
            # timing of a 12-60 us SpMM can be off by more than the margin left on the closest lines
            t2, _ = bench.strategy_times(capi, g, rp, ci, v, Bd, C, k, stream)
            t = {n: (None if x is None or t2[n] is None else min(x, t2[n])) for n, x in t.items()}
            best_name, best = min(((n, x) for n, x in t.items() if n != "auto" and x is not None), key=lambda nx: nx[1])
            gap = t["auto"] - best
        assert gap <= max(MAX_GAP * best, MAX_GAP_US), (
            f"{family} x{scale} K={k}: default plan (strategy {chosen}) {t['auto']:.1f} us, "
            f"{best_name} forced {best:.1f} us; all: {t}")
        del Bd, C


def test_locality_of_the_stored_order_is_measured(pkg, gpu):
    """hpspmm_plan_info.stored_order_miss_share, the sampled share of the gathers that miss an L2 in
    stored order, on matrices whose answer is known: columns without any order, a B that fits the
    cache, a mesh (each row shares its columns with its neighbours), and no measurement for a small
    matrix or under a forcing flag."""
    import torch
    capi, graphs = pkg.capi, pkg.graphs

    def share(g, k=64, flags=0):
        rp, ci = (torch.from_numpy(a).to(gpu) for a in (g.rowptr, g.col))
        plan = capi.Plan(g.rows, g.cols, rp, ci, k, flags)
        info = plan.info
        plan.destroy()
        return info["stored_order_miss_share"], info["strategy"]

    uniform = graphs.uniform_rows(400_000, 400_000, 20, 5)      # 8 M nonzeros over 400k columns: nearly every gather misses
    m, _ = share(uniform)
    assert 0.85 <= m <= 1.0, m
    fits = graphs.uniform_rows(400_000, 20_000, 20, 5)          # 20k columns: all of them within reach
    m, _ = share(fits)
    assert 0.0 <= m <= 0.05, m
    mesh = graphs.make_graph("h3_grid", 0.12)                     # 9 of 13 entries per row shared with neighbouring rows
    m, strategy = share(mesh, k=128)
    assert 0.25 <= m <= 0.65, m
    assert strategy == capi.STRATEGY_ROWS                          # 12 M nonzeros x 128 columns: whole rows all the same
    m, _ = share(mesh, flags=capi.PLAN_FORCE_SEGMENTS)
    assert m == -1.0
    m, _ = share(graphs.make_graph("c1_citation"))
    assert m == -1.0
