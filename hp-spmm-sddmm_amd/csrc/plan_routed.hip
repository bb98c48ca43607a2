// Routed strategy: construction of the layout (column slices pinned to XCDs, class-major order of
// the nonzeros of the long rows, chunk tables of the per-call value sort).
#include "host.hpp"

#include "rank_kernels.hpp"
#include "routed_plan_kernels.hpp"

namespace hpspmm_host {

namespace {

// Rows of B kept in the compact buffer by the routed strategy (all slices together).
constexpr int kRoutedLog2Cached = 16;
// Automatic choice of the routed strategy (thresholds from measurements on the
// benchmark graphs: it pays on the 233k-vertex social graph at K = 32, 64 and
// 128 (1.34 -> 1.25 ms, 2.95 -> 2.05 ms, 6.6 -> 3.9 ms) and on the R-MAT graph
// (8.6 -> 6.1 ms); not on the co-purchase graph, whose columns are too evenly
// used (4.5 -> 5.5 ms)).
constexpr int64_t kRoutedMinNnz = (int64_t)1 << 22;
constexpr int64_t kRoutedMinBBytes = (int64_t)10 << 20;  // a B that one or two L2s hold needs no routing (social graph at 26 M nonzeros: B = 7 MB, routed 309 us against 246; B = 14 MB, 464 against 474)
constexpr double kRoutedMinShare = 0.35;     // of the nonzeros in the 64k most referenced columns
constexpr double kRoutedMinRowNnz = 32.0;    // mean nonzeros per non-empty row
constexpr int32_t kRoutedRowThreshold = 128;  // rows shorter than this are not split over the classes
constexpr double kRoutedMinRoutedShare = 0.3;  // of the nonzeros in rows of at least that length
constexpr double kRoutedMinRoutedShareTiles = 0.25;
// Phases: a slice of B larger than this is worked through in two phases, which halves the
// set of hot rows an L2 has to hold at a time.  Every phase adds a partial-result row per
// routed row, and more than two never paid: 233k-vertex social graph, K = 128 (15 MB a
// slice) 4.11 / 4.01 / 4.34 ms with 1 / 2 / 3 phases, K = 64 (7.5 MB a slice) 2.14 / 2.28 /
// 2.51 ms; R-MAT scale 22, K = 128 (268 MB a slice) 6.63 / 6.23 / 6.32 ms.
constexpr int64_t kRoutedPhaseBytes = (int64_t)8 << 20;
// Column-tile phases (see spmm_routed_tiles_kernel), chosen where the slices would otherwise need two
// phases: tiles of 32 columns; bytes of its slice's compact-buffer rows, within one tile, per XCD (what
// the 4 MB L2 keeps of them is up to its replacement: R-MAT scale 22, K = 128: 5.74 ms with 2 MB,
// 5.57 with 4 MB, 5.59 with 8 MB, against 6.08 ms for two phases over whole rows).
constexpr int kRoutedTileWidth = 32;
constexpr int64_t kRoutedTileHotBytes = (int64_t)4 << 20;

}  // namespace

// Builds the routed layout.  Returns HPSPMM_OK with p->strategy left at
// SEGMENTS when the graph does not qualify (and `forced` is false).
int build_routed(hpspmm_plan* p, const int32_t* d_rowptr, const int32_t* d_col, bool forced, const PlanOptions& opt,
                 ColumnRanking& rk, hipStream_t st) {
  // (the caller's sizes are heeded only with the forcing flag)
  const int log2_hubs = forced ? opt.hub_log2 : 0;
  const int log2_row_threshold = forced ? opt.routed_row_log2 : 0;
  const int want_sub = forced ? opt.routed_phases : 0;
  const bool sort_values = (opt.flags & HPSPMM_PLAN_ROUTED_SORT_VALUES) != 0;
  const int64_t rows = p->rows, nnz = p->nnz, k = p->k;
  if (!forced && (nnz < kRoutedMinNnz || p->cols * k * 4 < kRoutedMinBBytes)) return HPSPMM_OK;
  const int64_t nonempty = std::max<int64_t>(1, rows - p->empty_rows);
  if (!forced && (double)nnz / (double)nonempty < kRoutedMinRowNnz) return HPSPMM_OK;
  if (nnz > INT32_MAX - ((int64_t)1 << 24)) return HPSPMM_OK;  // virtual indices stay int32
  // Column-tile phases: all XCDs work through B and C one tile of tile_w columns after the other.
  // For a plan of whole rows of a tuned length only (not for one that is itself a column tile of a
  // wider product), and not with the values read in place (column-range slices).
  int tile_w = opt.routed_tile_width > 0    ? opt.routed_tile_width
               : opt.routed_tile_width == 0 ? (p->cols * k * 4 / hpspmm::kSlices > kRoutedPhaseBytes && !want_sub ? kRoutedTileWidth : 0)
                                            : 0;
  if (tile_w && (k % tile_w != 0 || k <= tile_w || p->k_full != k || p->cols >= ((int64_t)1 << 29))) tile_w = 0;
  const int64_t kw = tile_w ? tile_w : k;  // row length the kernel's sub-waves are made for
  // cached rows per class
  const int64_t default_cached = tile_w ? hpspmm::kSlices * kRoutedTileHotBytes / (tile_w * 4) : (int64_t)1 << kRoutedLog2Cached;
  const int64_t h = std::max<int64_t>(1, (log2_hubs ? (int64_t)1 << log2_hubs : default_cached) / hpspmm::kSlices);
  if (int rc = rank_columns(p, d_col, h * hpspmm::kSlices, st, rk)) return rc;
  if (!forced && (double)rk.served < kRoutedMinShare * (double)nnz) return HPSPMM_OK;
  const int32_t n_ids = (int32_t)rk.n_ids;

  const int64_t slice_bytes = p->cols * k * 4 / hpspmm::kSlices;
  int nsub = slice_bytes > kRoutedPhaseBytes ? 2 : 1;
  if (want_sub) nsub = std::min(want_sub, hpspmm::kMaxSub);
  if (tile_w) nsub = 1;  // the tiles are the phases

  const int64_t n_bhot = h * hpspmm::kSlices;

  const int nhub = hpspmm::kSlices * nsub;
  const int32_t min_row_nnz =
      std::max<int32_t>(1, forced && log2_row_threshold ? (1 << log2_row_threshold) : kRoutedRowThreshold);

  // Column-range slices: the columns cut into 8 * nsub consecutive ranges of equal nonzero count
  // instead of spread by rank and hash.  In a row with sorted columns the nonzeros of one class are
  // then consecutive, so the kernel reads the values where the caller keeps them and the per-call
  // re-ordering of the values (0.21 ms of the social graph's 1.2 ms at K = 32) goes away.  Only when
  // the hot columns spread evenly over the ranges (random vertex labels do that; R-MAT's hot
  // columns all have small indices and would land in one slice, whose L2 could not hold them) and
  // with one phase: with two the runs are half as long, the value loads fetch 1.8 lines per run, and
  // what the re-ordering pass saved is spent inside the main kernel (social graph, K = 128: 3.73 ms
  // either way; R-MAT: 6.0 -> 6.85 ms).
  // temporaries of the layout construction (freed by the guard on every way out)
  uint8_t* d_colrange = nullptr;
  int32_t* d_colmap = nullptr;
  int32_t* d_bhot_src_tmp = nullptr;  // [n_bhot], handed to the plan once the layout is accepted
  uint32_t* d_ridx = nullptr;     // [rows + 1] routed flag, then (scanned in place) routed-row number
  uint32_t* d_cnt = nullptr;      // [nhub * n_routed + 1] class-major counts, then their scan
  uint32_t* d_coldcnt = nullptr;  // [rows + 1] cold-class count per row, then its scan
  uint8_t* d_action = nullptr;    // [rows]
  int32_t* d_counts = nullptr;    // [2] list lengths
  int32_t* d_vpos = nullptr;      // [nnz] position of every stored nonzero in the class-major order
  int32_t* d_rlist = nullptr;     // [n_routed] row of every routed-row number
  uint32_t* d_chunk_base = nullptr;  // [n_routed + 1] chunks per routed row, then (scanned) its first chunk
  int32_t* d_chunk_row = nullptr;    // [n_chunks] routed-row number of every chunk
  struct Guard {
    void** q[12];
    ~Guard() {
      for (void** x : q)
        if (*x) (void)hipFree(*x);
    }
  } guard{{(void**)&d_colmap, (void**)&d_ridx, (void**)&d_cnt, (void**)&d_coldcnt, (void**)&d_action,
           (void**)&d_counts, (void**)&d_vpos, (void**)&d_colrange, (void**)&d_bhot_src_tmp, (void**)&d_rlist,
           (void**)&d_chunk_base, (void**)&d_chunk_row}};

  bool inplace = false;
  if (!sort_values && !tile_w && nsub == 1 && nnz > 0 && p->cols * p->k_full * 4 < ((int64_t)1 << 32) &&
      columns_sorted(p, d_rowptr, d_col, st)) {
    const int groups = nhub;
    const int64_t target = ceil_div(rk.sampled, groups);  // the column counts are those of the sample
    uint32_t* d_before = nullptr;
    uint32_t* d_hot = nullptr;
    uint32_t hot[hpspmm::kMaxHub] = {0};
    hipError_t e = hipMalloc(&d_before, (size_t)(p->cols + 1) * sizeof(uint32_t));
    if (e == hipSuccess) e = hipMalloc(&d_hot, sizeof hot);
    if (e == hipSuccess) e = hipMalloc(&d_colrange, (size_t)p->cols);
    if (e == hipSuccess) e = hipMemsetAsync(d_hot, 0, sizeof hot, st);
    int rc = HPSPMM_OK;
    if (e == hipSuccess)  // the counts are non-negative: scanned as uint32 (one spare slot keeps the scan's tail in bounds)
      rc = exclusive_scan_u32(reinterpret_cast<const uint32_t*>(rk.d_count), d_before, p->cols, st);
    if (e == hipSuccess && rc == HPSPMM_OK) {
      hipLaunchKernelGGL(hpspmm::column_range_kernel, dim3((unsigned)ceil_div(p->cols, hpspmm::kBlock)),
                         dim3(hpspmm::kBlock), 0, st, p->cols, d_before, target, groups, d_colrange);
      if (n_ids > 0)
        hipLaunchKernelGGL(hpspmm::range_hot_count_kernel, dim3((unsigned)ceil_div(n_ids, hpspmm::kBlock)),
                           dim3(hpspmm::kBlock), 0, st, n_ids, rk.d_ids, d_colrange, d_hot);
      e = hipMemcpyAsync(hot, d_hot, sizeof hot, hipMemcpyDeviceToHost, st);
      if (e == hipSuccess) e = hipStreamSynchronize(st);
    }
    if (d_before) (void)hipFree(d_before);
    if (d_hot) (void)hipFree(d_hot);
    if (rc) return rc;
    if (e != hipSuccess) return fail(HPSPMM_ERR_HIP, "column ranges: %s", hipGetErrorString(e));
    const int64_t most = *std::max_element(hot, hot + groups);
    inplace = most * 2 * groups <= 3 * (int64_t)n_ids + 32 * groups;
    if (!inplace) {
      (void)hipFree(d_colrange);
      d_colrange = nullptr;
    }
  }
  // Evenly spread hot columns also mean that their rows of B do not crowd a few memory channels, which
  // is what the compact buffer is for (R-MAT): without it (social graph, K = 32: 1.128 against
  // 1.135 ms with it) the kernel's gather address is a 32-bit offset from B and the hot rows need
  // no copying at the start of every SpMM.

  // popularity rank s -> slice s % 8, compact-buffer row (s % 8) * h + s / 8 (none with column ranges)
  HPSPMM_HIP(hipMalloc(&d_colmap, (size_t)std::max<int64_t>(1, p->cols) * sizeof(int32_t)));
  HPSPMM_HIP(hipMalloc(&d_bhot_src_tmp, (size_t)n_bhot * sizeof(int32_t)));
  HPSPMM_HIP(hipMemsetAsync(d_colmap, 0xFF, (size_t)std::max<int64_t>(1, p->cols) * sizeof(int32_t), st));
  HPSPMM_HIP(hipMemsetAsync(d_bhot_src_tmp, 0xFF, (size_t)n_bhot * sizeof(int32_t), st));
  if (!inplace && n_ids > 0)
    hipLaunchKernelGGL(hpspmm::hot_slots_kernel, dim3((unsigned)ceil_div(n_ids, hpspmm::kBlock)), dim3(hpspmm::kBlock), 0,
                       st, n_ids, rk.d_ids, hpspmm::kSlices, (int32_t)h, d_colmap, d_bhot_src_tmp);
  HPSPMM_HIP(hipMalloc(&d_ridx, (size_t)(rows + 1) * sizeof(uint32_t)));
  HPSPMM_HIP(hipMalloc(&d_coldcnt, (size_t)(rows + 1) * sizeof(uint32_t)));
  HPSPMM_HIP(hipMalloc(&d_action, (size_t)rows));
  HPSPMM_HIP(hipMalloc(&d_counts, 2 * sizeof(int32_t)));

  // number the routed rows
  hipLaunchKernelGGL(hpspmm::routed_flag_kernel, dim3((unsigned)ceil_div(rows + 1, hpspmm::kBlock)),
                     dim3(hpspmm::kBlock), 0, st, rows, d_rowptr, min_row_nnz, d_ridx);
  if (int rc = exclusive_scan_u32(d_ridx, d_ridx, rows + 1, st)) return rc;
  uint32_t n_routed_u = 0;
  HPSPMM_HIP(hipMemcpyAsync(&n_routed_u, d_ridx + rows, sizeof(uint32_t), hipMemcpyDeviceToHost, st));
  HPSPMM_HIP(hipStreamSynchronize(st));
  const int64_t n_routed = n_routed_u;

  // class counts and their scans: a wavefront per chunk of a routed row, a thread per short row
  HPSPMM_HIP(hipMalloc(&d_rlist, (size_t)std::max<int64_t>(n_routed, 1) * sizeof(int32_t)));
  HPSPMM_HIP(hipMalloc(&d_chunk_base, (size_t)(n_routed + 1) * sizeof(uint32_t)));
  const unsigned thread_per_row_grid = (unsigned)ceil_div(rows + 1, hpspmm::kBlock);
  const unsigned thread_per_routed_grid = (unsigned)ceil_div(n_routed + 1, hpspmm::kBlock);
  hipLaunchKernelGGL(hpspmm::routed_list_kernel, dim3(thread_per_row_grid), dim3(hpspmm::kBlock), 0, st, rows, d_rowptr,
                     min_row_nnz, d_ridx, d_rlist);
  hipLaunchKernelGGL(hpspmm::routed_cold_count_kernel, dim3(thread_per_row_grid), dim3(hpspmm::kBlock), 0, st, rows,
                     d_rowptr, min_row_nnz, d_coldcnt);
  hipLaunchKernelGGL(hpspmm::routed_row_chunks_kernel, dim3(thread_per_routed_grid), dim3(hpspmm::kBlock), 0, st,
                     n_routed, d_rlist, d_rowptr, d_chunk_base);
  if (int rc = exclusive_scan_u32(d_chunk_base, d_chunk_base, n_routed + 1, st)) return rc;
  uint32_t n_chunks_u = 0;
  HPSPMM_HIP(hipMemcpyAsync(&n_chunks_u, d_chunk_base + n_routed, sizeof(uint32_t), hipMemcpyDeviceToHost, st));
  HPSPMM_HIP(hipStreamSynchronize(st));
  const int64_t n_chunks = n_chunks_u;
  HPSPMM_HIP(hipMalloc(&d_chunk_row, (size_t)std::max<int64_t>(n_chunks, 1) * sizeof(int32_t)));
  const int64_t ncnt = (int64_t)nhub * n_chunks + 1;
  HPSPMM_HIP(hipMalloc(&d_cnt, (size_t)ncnt * sizeof(uint32_t)));
  const unsigned chunk_grid = (unsigned)std::max<int64_t>(1, ceil_div(n_chunks, hpspmm::kWavesPerBlock));
  hipLaunchKernelGGL(hpspmm::routed_chunk_rows_kernel, dim3(thread_per_routed_grid), dim3(hpspmm::kBlock), 0, st,
                     n_routed, d_chunk_base, d_chunk_row);
  hipLaunchKernelGGL(hpspmm::routed_count_kernel, dim3(chunk_grid), dim3(hpspmm::kBlock), 0, st, n_chunks, d_chunk_row,
                     d_chunk_base, d_rlist, d_rowptr, d_col, d_colmap, (int32_t)h, nsub, (const uint8_t*)d_colrange,
                     min_row_nnz, d_cnt);
  if (int rc = exclusive_scan_u32(d_cnt, d_cnt, ncnt, st)) return rc;
  if (int rc = exclusive_scan_u32(d_coldcnt, d_coldcnt, rows + 1, st)) return rc;

  // class sizes = differences of the scan at the class origins
  uint32_t origin[hpspmm::kMaxHub + 1];
  for (int x = 0; x <= nhub; ++x)
    HPSPMM_HIP(hipMemcpyAsync(&origin[x], d_cnt + (int64_t)x * n_chunks, sizeof(uint32_t), hipMemcpyDeviceToHost, st));
  uint32_t cold_total = 0;
  HPSPMM_HIP(hipMemcpyAsync(&cold_total, d_coldcnt + rows, sizeof(uint32_t), hipMemcpyDeviceToHost, st));
  HPSPMM_HIP(hipStreamSynchronize(st));
  if ((int64_t)origin[nhub] + (int64_t)cold_total != nnz)
    return fail(HPSPMM_ERR_HIP, "routed plan: class counts do not add up to nnz");
  // routing only moves the nonzeros of the routed rows; if those are few the layout buys nothing
  // (in column tiles the rows that stay whole are served from the same tile of B as the routed ones:
  // users x items with Zipf popularity, 102 M nonzeros of which 0.30 in such rows, K = 128: 3.79 ms
  // against 4.41 for whole rows and 4.43 for segments)
  if (!forced && (double)origin[nhub] < (tile_w ? kRoutedMinRoutedShareTiles : kRoutedMinRoutedShare) * (double)nnz) return HPSPMM_OK;

  hpspmm::RoutedLayout& lay = p->lay;
  lay = hpspmm::RoutedLayout{};
  lay.rows = rows;
  lay.n_routed = n_routed;
  lay.shift = p->shift;
  lay.nsub = nsub;
  lay.nhub = nhub;
  lay.tile_width = tile_w;
  lay.rows_of_b = p->cols;
  lay.hub_rows_per_slice = h;
  int tile_waves = hpspmm::kWavesPerBlock;
  if (tile_w) {
    // workgroups of 16 wavefronts, one per CU, whose LDS - what the staging tiles leave of it - holds
    // the most referenced rows of the class (a multiple of 8 of them: the cold class takes an eighth per slice)
    tile_waves = hpspmm::kRoutedTileWaves;
    int room = 0;
    if (int rc = routed_tiles_prepare(tile_w, &room)) return rc;
    int lds_rows = opt.routed_lds_rows < 0 ? 0 : opt.routed_lds_rows > 0 ? std::min(opt.routed_lds_rows, room) : room;
    lds_rows = (int)std::min<int64_t>(lds_rows, h) / hpspmm::kSlices * hpspmm::kSlices;
    lay.tile_waves = tile_waves;
    lay.lds_rows = lds_rows;
  }
  lay.tiles = tile_w ? (int)(k / tile_w) : 1;
  const int64_t subwaves = 64 / (kw / 4);
  const int64_t quantum = ((int64_t)1 << p->shift) * subwaves * tile_waves;  // nonzeros per workgroup
  int64_t at = 0;
  for (int x = 0; x <= nhub; ++x) {
    const int64_t n_x = x < nhub ? (int64_t)origin[x + 1] - (int64_t)origin[x] : (int64_t)cold_total;
    lay.cls_begin[x] = at;
    lay.cls_end[x] = at + n_x;
    lay.cls_blocks[x] = ceil_div(n_x, quantum);
    at += lay.cls_blocks[x] * quantum;
  }
  const int64_t vtotal = std::max<int64_t>(at, 1);
  // a phase's workgroups are interleaved by slice, so it takes 8 x its largest class
  int64_t grid = 0;
  for (int ph = 0; ph < nsub; ++ph) {
    lay.phase_begin[ph] = grid;
    int64_t most = 0;
    for (int x = 0; x < hpspmm::kSlices; ++x) most = std::max(most, lay.cls_blocks[ph * hpspmm::kSlices + x]);
    grid += most * hpspmm::kSlices;
  }
  lay.phase_begin[nsub] = grid;
  p->routed_grid = grid + lay.cls_blocks[nhub];
  if (tile_w) {
    // every tile's range of workgroups begins at a multiple of 8, so that workgroup -> XCD stays slice
    lay.cold_grid = ceil_div(lay.cls_blocks[nhub], hpspmm::kXcds) * hpspmm::kXcds;
    lay.n_zero = p->empty_rows;
    const int64_t zero_per_block = (int64_t)tile_waves * subwaves * hpspmm::kTileZeroRows;
    lay.hub_grid = grid;
    lay.tile_grid = grid + lay.cold_grid + ceil_div(ceil_div(p->empty_rows, zero_per_block), hpspmm::kXcds) * hpspmm::kXcds;
    p->routed_grid = lay.tile_grid * lay.tiles;
  }
  if (vtotal >= INT32_MAX || p->routed_grid > INT32_MAX) return HPSPMM_OK;

  const int64_t nseg = vtotal >> p->shift;
  const size_t rvptr_bytes = (size_t)(n_routed + 1) * (size_t)nhub * sizeof(int32_t);
  const size_t coldptr_bytes = (size_t)(rows + 1) * sizeof(int32_t);
  const size_t v_bytes = (size_t)vtotal * sizeof(int32_t);
  const size_t vpos_bytes = (size_t)std::max<int64_t>(nnz, 1) * sizeof(int32_t);
  const int64_t nchunks = ceil_div(nnz, hpspmm::kPermChunk);
  const size_t lslot_bytes = (size_t)std::max<int64_t>(nnz, 1) * sizeof(uint16_t);
  const size_t chunk_bytes = (size_t)std::max<int64_t>(nchunks, 1) * (size_t)(nhub + 1) * sizeof(int32_t);
  const size_t partial_bytes = (size_t)std::max<int64_t>(n_routed, 1) * (size_t)nhub * (size_t)k * sizeof(float);
  const size_t carry_bytes = (size_t)std::max<int64_t>(nseg, 1) * 2 * (size_t)k * sizeof(float);
  const size_t bhot_bytes = (size_t)n_bhot * (size_t)k * sizeof(float);
  const size_t list_bytes = (size_t)std::max<int64_t>(rows, 1) * sizeof(int32_t);
  const size_t routed_rows_bytes = (size_t)std::max<int64_t>(n_routed, 1) * sizeof(int32_t);
  // the segments strategy's carry slots are not needed any more (the row of every nonzero is, for the fill)
  if (p->d_carry) { (void)hipFree(p->d_carry); p->d_carry = nullptr; }
  if (int rc = ensure_row_expansion(p, d_rowptr, st)) return rc;
  const size_t total_bytes = rvptr_bytes + coldptr_bytes + (tile_w ? 2 : 3) * v_bytes +
                             (inplace ? 0 : lslot_bytes + 2 * chunk_bytes) + partial_bytes + carry_bytes +
                             bhot_bytes + (size_t)n_bhot * 4 + 2 * list_bytes + routed_rows_bytes;
  // (the order of these allocations is felt: with the values allocated after the rows instead of
  // between columns and rows the social graph at K = 32 ran 3 % slower - where the three streams
  // that a sub-wave reads in step lie relative to each other decides how they share the channels)
  bool ok = hipMalloc(&p->d_rvptr, rvptr_bytes) == hipSuccess && hipMalloc(&p->d_coldptr, coldptr_bytes) == hipSuccess &&
            hipMalloc(&p->d_vcol, v_bytes) == hipSuccess &&
            hipMalloc(inplace ? (void**)&p->d_vsrc : (void**)&p->d_vval, v_bytes) == hipSuccess &&
            hipMalloc(&p->d_vrow, v_bytes) == hipSuccess && hipMalloc(&d_vpos, vpos_bytes) == hipSuccess;
  if (ok && !inplace)
    ok = hipMalloc(&p->d_lslot, lslot_bytes) == hipSuccess && hipMalloc(&p->d_chunk_base, chunk_bytes) == hipSuccess &&
         hipMalloc(&p->d_chunk_pref, chunk_bytes) == hipSuccess;
  if (!ok ||
      hipMalloc(&p->d_partial, partial_bytes) != hipSuccess || hipMalloc(&p->d_carry, carry_bytes) != hipSuccess ||
      hipMalloc(&p->d_bhot, bhot_bytes) != hipSuccess ||
      hipMalloc(&p->d_routed_rows, routed_rows_bytes) != hipSuccess ||
      hipMalloc(&p->d_cross_rows, list_bytes) != hipSuccess || hipMalloc(&p->d_zero_rows, list_bytes) != hipSuccess) {
    (void)hipGetLastError();
    return fail(HPSPMM_ERR_ALLOC, "device allocation for the routed plan failed (%zu bytes)", total_bytes);
  }
  p->workspace_bytes = (int64_t)total_bytes;
  p->d_bhot_src = d_bhot_src_tmp;  // the plan owns it from here on
  d_bhot_src_tmp = nullptr;
  // unused compact-buffer rows and the padding between the classes are never used; keep them defined anyway
  HPSPMM_HIP(hipMemsetAsync(p->d_bhot, 0, bhot_bytes, st));
  HPSPMM_HIP(hipMemsetAsync(inplace ? (void*)p->d_vsrc : (void*)p->d_vval, 0, v_bytes, st));
  HPSPMM_HIP(hipMemsetAsync(d_counts, 0, 2 * sizeof(int32_t), st));
  const int64_t nrv = (n_routed + 1) * nhub;
  hipLaunchKernelGGL(hpspmm::routed_vptr_kernel, dim3((unsigned)ceil_div(nrv, hpspmm::kBlock)), dim3(hpspmm::kBlock),
                     0, st, lay, n_chunks, d_chunk_base, d_cnt, p->d_rvptr);
  hipLaunchKernelGGL(hpspmm::routed_coldptr_kernel, dim3((unsigned)ceil_div(rows + 1, hpspmm::kBlock)),
                     dim3(hpspmm::kBlock), 0, st, rows, lay.cls_begin[nhub], d_coldcnt, p->d_coldptr);
  HPSPMM_HIP(hipMemcpyAsync(p->d_routed_rows, d_rlist, (size_t)n_routed * sizeof(int32_t), hipMemcpyDeviceToDevice, st));
  hipLaunchKernelGGL(hpspmm::routed_fill_kernel, dim3(chunk_grid), dim3(hpspmm::kBlock), 0, st, lay, n_chunks,
                     d_chunk_row, d_chunk_base, d_cnt, d_rlist, d_rowptr, d_col, d_colmap, (int32_t)h,
                     (const uint8_t*)d_colrange, min_row_nnz, p->d_vcol, d_vpos, p->d_vsrc, p->d_vrow);
  if (nnz > 0)
    hipLaunchKernelGGL(hpspmm::routed_fill_cold_kernel, dim3((unsigned)ceil_div(nnz, hpspmm::kBlock)),
                       dim3(hpspmm::kBlock), 0, st, nnz, p->d_nnz_row, d_rowptr, d_col, d_colmap, min_row_nnz,
                       p->d_coldptr, p->d_vcol, d_vpos, p->d_vsrc, p->d_vrow);
  hipLaunchKernelGGL(hpspmm::routed_action_kernel, dim3((unsigned)ceil_div(rows, hpspmm::kBlock)), dim3(hpspmm::kBlock),
                     0, st, rows, d_rowptr, min_row_nnz, p->d_coldptr, p->shift, d_action);
  // chunk tables of the value scatter
  if (nchunks > INT32_MAX) return fail(HPSPMM_ERR_INVALID_ARG, "grid too large");
  if (!inplace)
    hipLaunchKernelGGL(hpspmm::routed_chunk_kernel, dim3((unsigned)nchunks), dim3(hpspmm::kBlock), 0, st, lay, nnz,
                       d_vpos, p->d_lslot, p->d_chunk_base, p->d_chunk_pref);
  // compact lists of the short rows the final kernel has to visit
  const unsigned cgrid = (unsigned)ceil_div(std::max<int64_t>(rows, 1), hpspmm::kCollectRows);
  hipLaunchKernelGGL(hpspmm::routed_collect_rows_kernel, dim3(cgrid), dim3(hpspmm::kBlock), 0, st, rows, d_action,
                     hpspmm::kActionCross, p->d_cross_rows, d_counts);
  hipLaunchKernelGGL(hpspmm::routed_collect_rows_kernel, dim3(cgrid), dim3(hpspmm::kBlock), 0, st, rows, d_action,
                     hpspmm::kActionZero, p->d_zero_rows, d_counts + 1);
  int32_t counts[2] = {0, 0};
  HPSPMM_HIP(hipMemcpyAsync(counts, d_counts, sizeof counts, hipMemcpyDeviceToHost, st));
  HPSPMM_HIP(hipStreamSynchronize(st));
  HPSPMM_HIP(hipGetLastError());
  p->n_cross = counts[0];
  p->n_zero = counts[1];
  p->lay.n_zero = std::min<int64_t>(counts[1], p->lay.n_zero);  // (the tile grid was sized for the latter)
  (void)hipFree(p->d_nnz_row);  // the row of every nonzero served the fill; the class-major arrays replace it
  p->d_nnz_row = nullptr;
  if (tile_w) {
    // The row of every entry becomes a flag in its entry word and one row per run; the row array goes.
    DeviceTemps tmp;
    uint32_t *d_flag = nullptr, *d_before = nullptr;
    if (int rc = tmp.alloc(&d_flag, (size_t)vtotal + 1)) return rc;
    if (int rc = tmp.alloc(&d_before, (size_t)vtotal + 1)) return rc;
    hipLaunchKernelGGL(hpspmm::routed_run_flags_kernel, dim3(grid_for(vtotal + 1, 1 << 16)), dim3(hpspmm::kBlock), 0, st,
                       lay, vtotal, p->d_vrow, d_flag);
    if (int rc = exclusive_scan_u32(d_flag, d_before, vtotal + 1, st)) return rc;
    uint32_t n_runs = 0;
    HPSPMM_HIP(hipMemcpyAsync(&n_runs, d_before + vtotal, sizeof n_runs, hipMemcpyDeviceToHost, st));
    HPSPMM_HIP(hipStreamSynchronize(st));
    const size_t run_bytes = (size_t)std::max<uint32_t>(n_runs, 1) * sizeof(int32_t);
    const size_t seg_bytes = (size_t)std::max<int64_t>(nseg, 1) * sizeof(int32_t);
    if (hipMalloc(&p->d_run_row, run_bytes) != hipSuccess || hipMalloc(&p->d_seg_run, seg_bytes) != hipSuccess) {
      (void)hipGetLastError();
      return fail(HPSPMM_ERR_ALLOC, "device allocation for the routed plan failed (%zu bytes)", run_bytes + seg_bytes);
    }
    HPSPMM_HIP(hipMemsetAsync(p->d_seg_run, 0, seg_bytes, st));
    hipLaunchKernelGGL(hpspmm::routed_runs_kernel, dim3(grid_for(vtotal, 1 << 16)), dim3(hpspmm::kBlock), 0, st, lay,
                       vtotal, d_flag, d_before, p->d_vrow, p->d_vcol, p->d_run_row, p->d_seg_run);
    HPSPMM_HIP(hipStreamSynchronize(st));
    HPSPMM_HIP(hipGetLastError());
    (void)hipFree(p->d_vrow);
    p->d_vrow = nullptr;
    p->n_runs = n_runs;
    p->workspace_bytes += (int64_t)(run_bytes + seg_bytes);
  }
  p->n_bhot = inplace ? 0 : n_bhot;
  p->n_hub = inplace ? 0 : (int64_t)n_ids;
  p->nseg = nseg;
  p->routed_split_launch = opt.routed_split_launch;
  p->strategy = HPSPMM_STRATEGY_ROUTED;
  return HPSPMM_OK;
}

}  // namespace hpspmm_host
