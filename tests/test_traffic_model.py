"""The CPU-side cache model behind the traffic figures quoted for the routed strategy: the LRU
simulator against hand-worked streams, and the model's byte counts on a small R-MAT graph."""
import importlib

import numpy as np


def _tm():
    return importlib.import_module("hp-spmm-sddmm_amd.traffic_model")


def test_lru_known_answers():
    tm = _tm()
    # capacity 3: 0 1 2 miss, 0 1 2 hit, 3 misses and evicts 0, 0 misses again
    assert tm._lru_misses(np.array([0, 1, 2, 0, 1, 2, 3, 0]), 4, 3) == 5
    # a cyclic walk over capacity + 1 ids never hits
    assert tm._lru_misses(np.array([0, 1, 2, 3] * 5), 4, 3) == 20
    # ... and always hits after the first round when it fits
    assert tm._lru_misses(np.array([0, 1, 2, 3] * 5), 4, 4) == 4
    # negative ids are not gathers
    assert tm._lru_misses(np.array([-1, 5, -1, 5]), 8, 2) == 1
    # reuse distance exactly at capacity: 0 is the least recent of {0, 1, 2} when 3 arrives
    assert tm._lru_misses(np.array([0, 1, 2, 1, 0, 3, 2]), 4, 3) == 5
    rng = np.random.default_rng(3)
    ids = rng.integers(0, 50, 4000)
    # brute force LRU
    cache, misses = [], 0
    for c in ids:
        if c in cache:
            cache.remove(c)
        else:
            misses += 1
            if len(cache) == 7:
                cache.pop(0)
        cache.append(c)
    assert tm._lru_misses(ids, 50, 7) == misses


def test_routed_model_on_small_rmat(pkg):
    tm = _tm()
    g = pkg.graphs.make_graph("c4_rmat", 0.008)
    k = 128
    r = tm.routed_tiles_traffic(g, k, ranked_columns=1 << 12, lds_rows=64)
    assert r["tiles"] == 4
    assert r["hub_nnz"] + r["cold_nnz"] == g.nnz
    rowlen = np.diff(g.rowptr)
    assert r["hub_nnz"] == int(rowlen[rowlen >= 128].sum())
    assert r["stream_bytes"] == 4 * 8 * g.nnz and r["c_bytes"] == g.rows * k * 4
    # a cache cannot miss less often than once per distinct line, nor more often than once per gather
    assert r["hub_lines_first"] <= r["hub_lines_lru"] <= r["hub_nnz"]
    assert r["cold_lines_first"] <= r["cold_lines_lru"] <= r["cold_nnz"]
    assert r["compulsory"] <= r["lru"]
    # this graph's B tile (32768 rows of 128 bytes) fits one L2: every line is fetched once per XCD
    assert r["hub_lines_lru"] == r["hub_lines_first"] and r["cold_lines_lru"] == r["cold_lines_first"]
