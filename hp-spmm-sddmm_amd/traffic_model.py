"""CPU-side model of the L2 <-> fabric traffic of the routed strategy's column-tile kernel.

The kernel's gathers are replayed, XCD by XCD, through a fully associative LRU cache of one L2
(4 MB = 32768 lines of 128 bytes; a 32-column tile of a row of B is one line) in the order the
layout stores them: the nonzeros of the rows of at least `row_threshold` nonzeros by column slice
(slice = popularity rank mod 8 for the ranked columns, a hash of the index for the rest), each slice
in row order on its own XCD; the nonzeros of the shorter rows in row order, dealt to the XCDs
segment by segment.  Rows of B that the workgroups hold in LDS cost nothing.  Three figures come
out, in bytes per SpMM:

  compulsory   every byte the kernel needs, moved once: the entry and value streams once per column
               tile, every row of B once per tile and XCD that reads it, C and the partial results
               written once (and the partial results read once by the final kernel)
  lru          the same with the gathers of B as the LRU model misses them (the two streams of an
               XCD modelled with an L2 each: the kernel cannot do better than this order allows)
  lru_shared   the two streams of an XCD share its L2 in proportion to their lengths

This is a model of one layout, not a bound over all layouts: `compulsory` is the floor of the
routed layout, `lru` what its order of gathers costs on eight 4 MB caches."""
import ctypes

import numpy as np

from . import graphs

L2_LINES = (4 << 20) // 128
XCDS = 8


def _lru_misses(ids, id_range, capacity):
    lib = graphs.lib()
    lib.hpspmm_model_lru_misses.restype = ctypes.c_int64
    lib.hpspmm_model_lru_misses.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64]
    ids = np.ascontiguousarray(ids, dtype=np.int32)
    out = lib.hpspmm_model_lru_misses(ids.ctypes.data, ids.size, int(id_range), int(capacity))
    if out < 0:
        raise ValueError("hpspmm_model_lru_misses: bad arguments")
    return int(out)


def routed_tiles_traffic(g, k, tile_width=32, row_threshold=128, ranked_columns=1 << 18, lds_rows=696,
                         segment=512):
    """Model of one SpMM of the routed strategy in column tiles on the CSR matrix `g` (graphs.CSR).
    Returns a dict of byte counts and of the quantities they are made of."""
    tiles = k // tile_width
    line = tile_width * 4
    lines = (4 << 20) // line
    rowlen = np.diff(g.rowptr).astype(np.int64)
    row_of = np.repeat(np.arange(g.rows, dtype=np.int32), rowlen)
    col = g.col
    # popularity ranking and the slice of every column
    count = np.bincount(col, minlength=g.cols)
    order = np.argsort(-count, kind="stable")
    n_ranked = int(min(ranked_columns, np.count_nonzero(count)))
    slice_of = ((np.arange(g.cols, dtype=np.uint64) * np.uint64(2654435761)) >> np.uint64(29)).astype(np.int64) & 7
    slice_of[order[:n_ranked]] = np.arange(n_ranked) % XCDS
    in_lds = np.zeros(g.cols, dtype=bool)           # the most referenced rows of every slice
    in_lds[order[:min(lds_rows * XCDS, n_ranked)]] = True
    in_lds_cold = np.zeros(g.cols, dtype=bool)      # the cold workgroups hold an eighth as many per slice
    in_lds_cold[order[:min(lds_rows // XCDS * XCDS, n_ranked)]] = True

    routed = rowlen[row_of] >= row_threshold
    hub_col, hub_row = col[routed], row_of[routed]
    cold_col = col[~routed]
    n_hub, n_cold = hub_col.size, cold_col.size

    # hub classes: slice x on XCD x, in row order
    hub_miss = hub_first = 0
    partial_rows = 0
    per_xcd_hub = []
    for x in range(XCDS):
        m = slice_of[hub_col] == x
        stream = np.where(in_lds[hub_col[m]], -1, hub_col[m])
        per_xcd_hub.append(stream)
        hub_miss += _lru_misses(stream, g.cols, lines)
        hub_first += np.unique(stream[stream >= 0]).size
        partial_rows += np.unique(hub_row[m]).size  # one partial-result row per routed row and class it touches
    # cold class: segments dealt round robin
    seg = np.arange(n_cold) // segment
    cold_miss = cold_first = 0
    shared_miss = 0
    for x in range(XCDS):
        stream = cold_col[seg % XCDS == x]
        stream = np.where(in_lds_cold[stream], -1, stream)
        cold_miss += _lru_misses(stream, g.cols, lines)
        cold_first += np.unique(stream[stream >= 0]).size
        # the two streams of the XCD through one L2: interleaved in proportion to their lengths
        h = per_xcd_hub[x]
        both = np.empty(h.size + stream.size, dtype=np.int32)
        pos = (np.arange(h.size, dtype=np.float64) + 0.5) * (both.size / max(h.size, 1))
        is_h = np.zeros(both.size, dtype=bool)
        is_h[np.minimum(pos.astype(np.int64), both.size - 1)] = True
        # (positions may collide when h is the longer stream: fill by count instead)
        if is_h.sum() != h.size:
            is_h[:] = False
            is_h[np.round(np.linspace(0, both.size - 1, h.size)).astype(np.int64)] = True
            extra = h.size - int(is_h.sum())
            if extra > 0:
                free = np.flatnonzero(~is_h)[:extra]
                is_h[free] = True
        both[is_h] = h
        both[~is_h] = stream
        shared_miss += _lru_misses(both, g.cols, lines)

    short_rows = int(np.count_nonzero((rowlen > 0) & (rowlen < row_threshold)))
    empty_rows = int(np.count_nonzero(rowlen == 0))
    stream_bytes = tiles * 8 * (n_hub + n_cold)                  # entry word + value, once per tile
    c_bytes = g.rows * k * 4                                      # every row of C written once
    partial_bytes = 2 * partial_rows * k * 4                      # written by the main kernel, read by the final one
    out = {
        "tiles": tiles, "hub_nnz": int(n_hub), "cold_nnz": int(n_cold), "partial_rows": int(partial_rows),
        "short_rows": short_rows, "empty_rows": empty_rows,
        "hub_lines_first": int(hub_first), "cold_lines_first": int(cold_first),
        "hub_lines_lru": int(hub_miss), "cold_lines_lru": int(cold_miss), "lines_lru_shared": int(shared_miss),
        "stream_bytes": int(stream_bytes), "c_bytes": int(c_bytes), "partial_bytes": int(partial_bytes),
    }
    fixed = stream_bytes + c_bytes + partial_bytes
    out["compulsory"] = int(fixed + tiles * line * (hub_first + cold_first))
    out["lru"] = int(fixed + tiles * line * (hub_miss + cold_miss))
    out["lru_shared"] = int(fixed + tiles * line * shared_miss)
    return out
