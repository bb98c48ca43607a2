// hpspmm_plan_create and the other entry points about plans: validation, the choice of strategy,
// the hub cache, plan info, value binding, destruction.
#include "host.hpp"

#include "rank_kernels.hpp"
#include "routed_plan_kernels.hpp"
#include "rowtile_kernels.hpp"

#include <new>

using namespace hpspmm_host;

namespace {

// Width of the column tiles by which a tuned layout can serve row length k (0: none, or k is tuned
// itself): any multiple of 4 from 16 up - the last tile may be narrower than the layout's width, the
// lanes beyond it idle.  The width that costs least, a tile of 32 / 64 / 128 columns weighed as the
// tuned sizes relate on the benchmark graphs (1 : 1.56 : 2.75): 40 -> one tile of 64, 96 -> one of
// 128, 160 -> 64 + 64 + 32 of 64, 200 -> 128 + 72 of 128, 256 -> two of 128.
inline int64_t tile_width(int64_t k) {
  if (fast_k(k) || k < 16 || k % 4 != 0) return 0;
  const int64_t width[3] = {128, 64, 32};
  const double cost[3] = {2.75, 1.56, 1.0};
  int best = 0;
  for (int i = 1; i < 3; ++i)
    if ((double)((k + width[i] - 1) / width[i]) * cost[i] < (double)((k + width[best] - 1) / width[best]) * cost[best]) best = i;
  return width[best];
}

// Row tiles (32-column tiles of B and C) serve every row length
// (hpspmm_plan_options.row_tiles_min_k: only from there up, for comparisons).
inline bool row_tiles_serve(int64_t k, const PlanOptions& opt) {
  if (fast_k(k)) return true;
  if (k >= ((int64_t)1 << 22)) return false;
  return k >= opt.row_tiles_min_k;
}

using hpspmm::kRowTileWorkgroupRows;  // rows beyond this many nonzeros get a whole workgroup
// automatic use of the rows strategy beyond tiny matrices
constexpr int64_t kRowsAutoMaxNnz = 1 << 24;
constexpr int64_t kRowsAutoMaxWork = (int64_t)3 << 28;  // nnz * K, matrices of short rows
constexpr double kRowsAutoLongMean = 128.0;             // mean nonzeros per non-empty row beyond which ...
constexpr double kRowsAutoLongWork = 2.0e15;            // ... nnz^2 * K decides instead
constexpr int64_t kRowsAutoMaxRow = 1 << 16;
constexpr int64_t kRowsAutoAnyKNnz = 1 << 25;            // K outside the tuned set, rows of even lengths: row tiles up to here
constexpr int64_t kRowsAutoFewPerRowNnz = 1 << 22;      // rows of <= 8 nonzeros, K > 32 and not a multiple of 32
constexpr int64_t kRowTilePadMinNnz = 1 << 19;  // row tiles: matrices from here up read a B of odd row length through a padded copy

// Segment length: long enough that the carry traffic (two K-float partials per
// segment, against S*(K+2) floats of gather) is small, short enough that there
// are several waves of work per SIMD.
int choose_shift(int64_t nnz, int64_t k, int64_t max_row_nnz) {
  const int64_t subwaves = fast_k(k) ? 64 / (k / 4) : 64 / anyk_lanes(k);
  const int64_t target_waves = 256 /*CUs*/ * 4 /*SIMDs*/ * 16;
  int shift = 5;
  while (shift < 9 && (nnz >> (shift + 1)) / subwaves >= target_waves) ++shift;
  // a row cut into n segments is put together again by one sub-wave reading n carry slots one batch
  // after the other: keep that chain short (a dense row of 3M nonzeros in a matrix of 6M: 3.5 ms
  // with 32-nonzero segments, 0.9 ms with 512)
  while (shift < 9 && (max_row_nnz >> shift) > 2048) ++shift;
  return shift;
}

// Automatic clustering is tried for graphs of at least this size ...
constexpr int64_t kClusterMinNnz = (int64_t)1 << 22;
constexpr int64_t kClusterMinBBytes = (int64_t)12 << 20;  // co-purchase graph, 6 M nonzeros, K = 32 (B = 16 MB): 65 us against 87 for whole rows
// The sweep is chosen where it is expected to take this share of the time of whole rows: at once,
// and once the ordered strategy has been tried.
constexpr double kSweepSureGain = 0.7, kSweepMinGain = 0.9;
constexpr int64_t kOtherLayoutsMinNnz = (int64_t)1 << 21;  // below: whole rows without looking further
constexpr int64_t kRowTileChunksMinNnz = (int64_t)1 << 21;  // row tiles dealt to the XCDs in chunks from here up
// A matrix whose stored order is local already has its communities side by side; another order pays
// only where B is far beyond every cache (blocks of 8 to 4096 vertices along the diagonal with 10 % of
// the entries elsewhere, K = 32 / 64 / 128: at 10 M nonzeros (B = 38 / 77 / 154 MB) ordered 109 / 193 /
// 377 us against 99 / 183 / 380 for whole rows; at 85 M (320 / 640 / 1280 MB) 0.95 / 1.66 / 3.17 ms
// against 0.93 / 1.80 / 3.95).
constexpr int64_t kClusterLocalMinBBytes = (int64_t)256 << 20;
constexpr double kLocalMissShare = 0.3;  // stored order counts as local up to this share of missing gathers
constexpr double kRowsFallbackMissShare = 0.85;
constexpr double kRowsHitPs = 7.0, kRowsMissPs = 20.7;  // rows strategy: per nonzero and 32 columns of B
constexpr double kClusterMinIntra = 0.15;   // share of the nonzeros inside such clusters for the order to be used
// Rows of fewer nonzeros than this on average are left to the row tiles: what the ordered strategy spends per
// row (a run's row and value offset, a store of C per ~13 gathers) outweighs the gathers it saves (9-point mesh
// with two long-range entries per row, 12 M nonzeros, clusters found once the diagonal has no vote: 192 / 387 /
// 742 us against 128 / 253 / 590 for whole rows in stored order).
constexpr int64_t kClusterMinMeanNnz = 16;
// ... and its order is kept if this share of the nonzeros then reads B from LDS.
constexpr double kClusterMinServed = 0.15;

// Automatic hub cache: only when the cached rows would serve at least this share of the nonzeros.
constexpr double kHubMinShare = 0.25;

// Picks the most referenced columns of A (by nonzero count; ties by lower index, so
// the choice is reproducible), gives each a slot in a compact copy of B and
// rewrites the column array accordingly.  log2_hubs = 0 picks the default size.
int build_hub_cache(hpspmm_plan* p, const int32_t* d_col, int log2_hubs, bool forced, ColumnRanking& rk,
                    hipStream_t st) {
  if (log2_hubs == 0) log2_hubs = 16;
  if (log2_hubs < 4 || log2_hubs > 24) return fail(HPSPMM_ERR_INVALID_ARG, "hub cache size 2^%d outside [2^4, 2^24]", log2_hubs);
  if (int rc = rank_columns(p, d_col, (int64_t)1 << log2_hubs, st, rk)) return rc;
  if (rk.n_ids == 0) return HPSPMM_OK;
  // worth the extra column array only when the cached rows serve a good part of the gathers
  if (!forced && (double)rk.served < kHubMinShare * (double)p->nnz) return HPSPMM_OK;

  const int64_t n_hub = rk.n_ids;
  HPSPMM_HIP(hipMalloc(&p->d_hub_ids, (size_t)n_hub * sizeof(int32_t)));
  HPSPMM_HIP(hipMalloc(&p->d_hub_col, (size_t)p->nnz * sizeof(int32_t)));
  HPSPMM_HIP(hipMalloc(&p->d_bhot, (size_t)n_hub * (size_t)p->k * sizeof(float)));
  p->workspace_bytes += n_hub * 4 + p->nnz * 4 + n_hub * p->k * 4;
  HPSPMM_HIP(hipMemcpyAsync(p->d_hub_ids, rk.d_ids, (size_t)n_hub * sizeof(int32_t), hipMemcpyDeviceToDevice, st));
  int32_t* d_colmap = nullptr;
  HPSPMM_HIP(hipMalloc(&d_colmap, (size_t)p->cols * sizeof(int32_t)));
  hipError_t e = hipMemsetAsync(d_colmap, 0xFF, (size_t)p->cols * sizeof(int32_t), st);
  if (e == hipSuccess) {
    hipLaunchKernelGGL(hpspmm::hot_index_kernel, dim3((unsigned)ceil_div(n_hub, hpspmm::kBlock)), dim3(hpspmm::kBlock), 0,
                       st, (int32_t)n_hub, rk.d_ids, d_colmap);
    hipLaunchKernelGGL(hpspmm::remap_columns_kernel, dim3(grid_for(p->nnz, 1 << 16)), dim3(hpspmm::kBlock), 0, st,
                       p->nnz, d_col, d_colmap, p->d_hub_col);
    e = hipStreamSynchronize(st);
  }
  (void)hipFree(d_colmap);
  if (e != hipSuccess) return fail(HPSPMM_ERR_HIP, "column remap failed: %s", hipGetErrorString(e));
  p->n_hub = n_hub;
  return HPSPMM_OK;
}

// Column tiles are tried for matrices of at least this many nonzeros (below, whole rows or plain
// segments at the full row length are as good), or when the caller forces one of the layouts.
constexpr int64_t kTiledMinNnz = (int64_t)1 << 22;

// k_full = 0: the plan is for row length k.  Otherwise: a plan of tile width k for B and C of row
// length k_full (see hpspmm_plan::k_full).
int plan_create_impl(int64_t rows, int64_t cols, int64_t nnz, const int32_t* d_rowptr, const int32_t* d_col,
                     int64_t k, const PlanOptions& opt, void* stream, hpspmm_plan** plan_out, int64_t k_full = 0) {
  const uint32_t flags = opt.flags;
  const int32_t* d_order = opt.d_row_order;
  if (!plan_out) return fail(HPSPMM_ERR_INVALID_ARG, "plan_out is NULL");
  *plan_out = nullptr;
  if (int rc = check_dims(rows, cols, nnz, k)) return rc;
  if (!d_rowptr) return fail(HPSPMM_ERR_INVALID_ARG, "d_rowptr is NULL");
  if (nnz > 0 && !d_col) return fail(HPSPMM_ERR_INVALID_ARG, "d_col is NULL with nnz > 0");
  hipStream_t st = (hipStream_t)stream;

  // Not a tuned row length: the layouts built for a tuned length (sweep, routed, ordered) serve it
  // tile by tile, if the matrix gets one of them; if not, the plan is built for the full length as
  // for any other row length.  A row length that is not a multiple of 4 (from 16 up) is rounded up
  // to one for that: 16-byte gathers at 4-byte alignment cost about twice, so B is read through a
  // padded copy made at the start of every SpMM (0.02 ms for 233k rows of 41 floats; C is written
  // in place, its stores are few).
  // (hpspmm_plan_options.no_column_tiles switches this off, for comparisons)
  const int64_t kp = (k + 3) & ~(int64_t)3;
  const int64_t kw = fast_k(kp) ? kp : tile_width(kp);
  if (k_full == 0 && !fast_k(k) && kw > 0 && (k % 4 == 0 || k >= 16) && nnz > 0 &&
      opt.column_tiles &&
      (nnz >= kTiledMinNnz || d_order ||
       (flags & (HPSPMM_PLAN_FORCE_ROUTED | HPSPMM_PLAN_FORCE_SWEEP | HPSPMM_PLAN_CLUSTER)))) {
    hpspmm_plan* tiled = nullptr;
    int rc = plan_create_impl(rows, cols, nnz, d_rowptr, d_col, kw, opt, stream, &tiled, kp);
    if (rc == HPSPMM_OK && tiled &&
        (tiled->strategy == HPSPMM_STRATEGY_SWEEP || tiled->strategy == HPSPMM_STRATEGY_ROUTED ||
         tiled->strategy == HPSPMM_STRATEGY_ORDERED)) {
      if (kp != k) {
        const size_t pad_bytes = (size_t)std::max<int64_t>(cols, 1) * (size_t)kp * sizeof(float);
        if (hipMalloc(&tiled->d_bpad, pad_bytes) != hipSuccess) {
          (void)hipGetLastError();
          tiled->d_bpad = nullptr;
          hpspmm_plan_destroy(tiled);
          return fail(HPSPMM_ERR_ALLOC, "device allocation of %zu bytes for the padded copy of B failed", pad_bytes);
        }
        tiled->workspace_bytes += (int64_t)pad_bytes;
        tiled->k_user = k;
      }
      *plan_out = tiled;
      return HPSPMM_OK;
    }
    if (tiled) hpspmm_plan_destroy(tiled);
    if (rc == HPSPMM_ERR_BAD_CSR || rc == HPSPMM_ERR_NO_DEVICE) return rc;
  }

  int ndev = 0;
  if (hipGetDeviceCount(&ndev) != hipSuccess || ndev == 0) {
    (void)hipGetLastError();
    return fail(HPSPMM_ERR_NO_DEVICE, "no HIP device available");
  }

  // validation flags + row statistics, one small device buffer
  int32_t* d_meta = nullptr;
  HPSPMM_HIP(hipMalloc(&d_meta, 4 * sizeof(int32_t)));
  struct MetaGuard {
    int32_t* p;
    ~MetaGuard() { (void)hipFree(p); }
  } meta_guard{d_meta};
  HPSPMM_HIP(hipMemsetAsync(d_meta, 0, 4 * sizeof(int32_t), st));
  if (!(flags & HPSPMM_PLAN_NO_VALIDATE)) {
    const int64_t work = rows > nnz ? rows : nnz;
    hipLaunchKernelGGL(hpspmm::validate_csr_kernel, dim3(grid_for(work, 8192)), dim3(hpspmm::kBlock), 0, st, rows,
                       cols, nnz, d_rowptr, d_col, d_meta);
    int32_t bad = 0;
    HPSPMM_HIP(hipMemcpyAsync(&bad, d_meta, sizeof bad, hipMemcpyDeviceToHost, st));
    HPSPMM_HIP(hipStreamSynchronize(st));
    if (bad)
      return fail(HPSPMM_ERR_BAD_CSR, "invalid CSR:%s%s%s%s", (bad & 1) ? " rowptr[0] != 0;" : "",
                  (bad & 2) ? " rowptr decreases;" : "", (bad & 4) ? " rowptr[rows] != nnz;" : "",
                  (bad & 8) ? " column index out of range;" : "");
  }
  int32_t stats[2] = {0, 0};
  if (rows > 0) {
    hipLaunchKernelGGL(hpspmm::row_stats_kernel, dim3(grid_for(rows, 4096)), dim3(hpspmm::kBlock), 0, st, rows,
                       d_rowptr, d_meta + 1);
    HPSPMM_HIP(hipMemcpyAsync(stats, d_meta + 1, sizeof stats, hipMemcpyDeviceToHost, st));
    HPSPMM_HIP(hipStreamSynchronize(st));
  }

  hpspmm_plan* p = new (std::nothrow) hpspmm_plan;
  if (!p) return fail(HPSPMM_ERR_ALLOC, "out of host memory");
  // every exit but the last - an error return or an exception - frees the plan and what it owns
  struct PlanHolder {
    hpspmm_plan* plan;
    ~PlanHolder() { hpspmm_plan_destroy(plan); }
  } holder{p};
  p->rows = rows;
  p->cols = cols;
  p->nnz = nnz;
  p->k = k;
  p->k_full = k_full ? k_full : k;
  p->tiles = (int)ceil_div(p->k_full, k);
  p->k_user = p->k_full;
  p->max_row_nnz = stats[0];
  p->empty_rows = stats[1];
  p->src_rowptr = d_rowptr;
  p->src_col = d_col;
  p->allow_moved = (flags & HPSPMM_PLAN_ALLOW_MOVED_CSR) != 0;
  // strategies that place work on particular XCDs are used only where the dealing of workgroups to
  // XCDs they assume has been observed on this device
  const bool xcd_ok = xcd_dealing_holds(st, opt.xcd_dealing);
  p->xcd_remap = !(flags & HPSPMM_PLAN_NO_XCD_REMAP) && xcd_ok;

  // Automatic choice, in this order: tiny matrix -> rows; sweep where its expected time is well
  // below that of whole rows; a matrix in the rows strategy's range (`rows_range`: by size, or at any
  // size when its stored order is local) -> ordered if it has communities, else sweep if that is
  // still expected to pay, else rows; beyond that range -> routed if a few columns take most of the
  // nonzeros, else ordered if it has communities, else sweep as before, else rows where the rows
  // are even and not all gathers miss (`rows_fallback`), else segments.
  ColumnRanking ranking;         // column popularity, shared by the routed and the hub-cache decisions
  bool rows_need_tiles = false;  // rows strategy chosen on the strength of the row tiles
  bool rows_range = false;       // provisional segments; rows unless the ordered strategy qualifies
  bool want_row_tiles = true;    // rows strategy: over row tiles if they can be built
  double miss = 1.0;             // share of the gathers that miss an L2 when the rows are taken in stored order
  double rows_us = 0.0;          // what the rows strategy is expected to take (0: no estimate)
  bool rows_fallback = false;    // whole rows rather than segments if no other layout qualifies
  if (!row_tiles_serve(k, opt)) {
    // a row length that not even the row tiles serve: whole rows over the CSR arrays for small
    // matrices (one launch), segments beyond (balanced over any degree distribution)
    const bool small = nnz < (1 << 21) && p->max_row_nnz <= 4096;
    p->strategy = (flags & HPSPMM_PLAN_FORCE_SEGMENTS)                   ? HPSPMM_STRATEGY_SEGMENTS
                  : ((flags & HPSPMM_PLAN_FORCE_ROWS) || nnz == 0 || small) ? HPSPMM_STRATEGY_ROWS
                                                                           : HPSPMM_STRATEGY_SEGMENTS;
  } else if (d_order && nnz > 0 && fast_k(k)) {
    if (int rc = build_ordered(p, d_rowptr, d_col, d_order, 0.0, st)) {
      return rc;
    }
    holder.plan = nullptr;
    *plan_out = p;
    return HPSPMM_OK;
  } else if (flags & HPSPMM_PLAN_FORCE_ROWS) {
    p->strategy = HPSPMM_STRATEGY_ROWS;
  } else if (flags & (HPSPMM_PLAN_FORCE_SEGMENTS | HPSPMM_PLAN_FORCE_ROUTED | HPSPMM_PLAN_FORCE_SWEEP)) {
    p->strategy = HPSPMM_STRATEGY_SEGMENTS;  // the routed and sweep layouts are built on top of it below
  } else {
    // Whole rows (one launch) while the matrix is small enough that the second and third launch of
    // the other strategies are felt and L2 reuse across rows is not yet what decides.  Measured
    // against segments and routed on scaled copies of the benchmark graphs: with short rows (means
    // of 30 and 50 nonzeros) row tiles win up to nnz * K = 2^29.5 (R-MAT, 15 M nonzeros, K=32:
    // 188 us against 258 us routed; 7.6 M nonzeros, K=128: 403 against 346 us); with long rows
    // (mean 400: every row a chain of tiles on one wavefront) they win at 4.3 M nonzeros and lose
    // at 9.6 M for every K, the crossing near nnz * sqrt(K) = 4.5e7.
    const bool tiny = nnz < (1 << 21) && p->max_row_nnz <= 4096;  // fine even over the CSR arrays
    const double mean_row = (double)nnz / (double)std::max<int64_t>(1, rows - p->empty_rows);
    const bool fits = mean_row > kRowsAutoLongMean ? (double)nnz * (double)nnz * (double)k < kRowsAutoLongWork
                                                   : nnz * k < kRowsAutoMaxWork;
    // (A row length outside the tuned set, on a matrix that has not got one of the tiled layouts:
    // the alternative to row tiles is the run-time-K segments kernel, which they beat at every size
    // measured - R-MAT graph, 7.6 M nonzeros, K = 48: 206 against 817 us; 0.9 M, K = 96: 25 against 521.)
    // The exception are large matrices of few nonzeros per row, whose B is far beyond the L2s: what
    // decides there is the traffic, every 128-byte gather of a row of B that is not a whole number
    // of lines touches two, and the segments kernel, whose sub-waves read whole rows of B, is ahead
    // (citation graph at 64 times its size, 6.5 M nonzeros, K = 100: 774 us against 542; K = 41: 496
    // against 370; at 16 times, 1.6 M: 148 against 142 for the rows kernel over the CSR arrays,
    // K = 172: 231 against 273), while a padded copy of B costs more than it saves.
    const bool few_per_row = mean_row <= 8.0;
    // (K < 4, which row tiles read through a padded copy of B: 1.6 M nonzeros, K = 1: 30 against 18 us.)
    // On the largest matrices the segments kernel is level or ahead as well, unless the row lengths
    // are very uneven (social graph, 115 M nonzeros, K = 8: 0.97 ms against 1.12 for row tiles, K = 1:
    // 0.68 against 1.01; at 26 M nonzeros 0.38 against 0.24, 0.31 against 0.22; R-MAT at 31 M,
    // K = 1: 1.05 against 0.29).
    const bool uneven = (double)p->max_row_nnz >= 64.0 * mean_row;
    const bool any_k_range = !few_per_row  ? nnz < kRowTileMaxNnz && (uneven || nnz < (k < 4 ? kRowsAutoAnyKNnz / 4 : kRowsAutoAnyKNnz))
                             : k % 32 == 0 ? nnz < kRowsAutoMaxNnz && fits
                             : k < 4       ? nnz < kRowTilePadMinNnz
                                           : k <= 32 || nnz < kRowsAutoFewPerRowNnz;
    const bool in_range = fast_k(k) ? nnz < kRowsAutoMaxNnz && fits : any_k_range;
    // (a row gets at most one workgroup of 16 wavefronts; at K outside the tuned set that still beats
    // the segments kernel with a row of 163k nonzeros - R-MAT, 128 M nonzeros, K = 8: 1.72 against 2.27 ms)
    const int64_t longest_ok = fast_k(k) || k < 4 ? kRowsAutoMaxRow : 4 * kRowsAutoMaxRow;
    // How local the stored order is decides between strategies from here on.  The rows strategy over
    // matrices of 25 to 200 uniformly placed nonzeros per row takes, per nonzero and 32 columns of B,
    // 7.5 ps when the 32-column tile of B is 4 MB, 11.5 at 8 MB, 15.3 at 15 MB, 17.7 at 32 MB and
    // 19.2 at 64 MB (the same for K = 32, 64 and 128): 7 ps for a gather that hits, 20.7 for one that
    // does not.
    if (!tiny && nnz > 0 && fast_k(k)) {
      if (int rc = stored_order_miss_share(p, d_col, st, &miss)) return rc;
      p->stored_miss = miss;
      rows_us = (double)nnz * (double)(k / 32) * (kRowsHitPs + (kRowsMissPs - kRowsHitPs) * miss) * 1e-6;
    }
    if (opt.report && rows_us > 0)
      fprintf(stderr, "plan: %.3f of the gathers miss in stored order, whole rows expected to take %.1f us\n", miss, rows_us);
    const bool short_rows = mean_row <= kRowsAutoLongMean;
    const bool mid = in_range && p->max_row_nnz <= longest_ok && !(flags & HPSPMM_PLAN_NO_ROW_TILES);
    // Beyond that range, when none of the other layouts qualifies, the choice is between whole rows
    // and segments.  A matrix whose stored order is local (banded, a mesh, blocks along the diagonal)
    // is served best by whole rows at any size (9-point mesh with 2 random entries per row, 102 M
    // nonzeros, K = 32 / 64 / 128: 1.27 / 2.58 / 5.75 ms against 1.81 / 3.31 / 6.44 for segments); a few
    // missing gathers alone do not say that, though (R-MAT at 7.6 M nonzeros: 0.21 of them miss, for the
    // popularity of its columns, and the routed strategy is 10 % ahead of whole rows at K = 128), so
    // the other layouts are tried first.  Row tiles are taken in stored order by all the CUs side by side, so that rows
    // that share columns with their neighbours meet them in the L2; segments are long runs of
    // nonzeros far apart from each other, which gain nothing from that order, but read the sparse
    // matrix once instead of once per 32 columns.  Measured (rows against segments, K = 32 / 64 / 128):
    // 9-point mesh with 2 / 8 random entries per row, 52 / 100 M nonzeros: 0.66 / 1.31 / 2.84 against
    // 0.94 / 1.84 / 3.49 ms and 1.49 / 3.43 / 7.51 against 2.12 / 3.71 / 7.69; 20 uniformly placed
    // nonzeros in each of 4 M rows: 1.61 / 3.70 / 8.33 against 1.69 / 3.68 / 7.98; preferential
    // attachment, 101 M: 1.93 / 3.97 / 8.89 against 2.13 / 3.80 / 7.47.
    // (a row is a chain of tiles on one wavefront: long rows only where they are all of a length)
    const bool even_enough = (double)p->max_row_nnz < (short_rows ? 512.0 : 16.0) * mean_row;
    rows_fallback = fast_k(k) && even_enough && nnz < kRowTileMaxNnz && p->max_row_nnz <= longest_ok &&
                    !(flags & HPSPMM_PLAN_NO_ROW_TILES) && (miss <= kRowsFallbackMissShare || k == 32);
    if (nnz == 0 || tiny || (mid && nnz < kOtherLayoutsMinNnz)) {
      p->strategy = HPSPMM_STRATEGY_ROWS;
      rows_need_tiles = !(nnz == 0 || tiny);
      want_row_tiles = mid;
    } else {
      p->strategy = HPSPMM_STRATEGY_SEGMENTS;
      rows_range = mid;
    }
  }

  if (p->strategy == HPSPMM_STRATEGY_ROWS && want_row_tiles && row_tiles_serve(k, opt) && rows > 0 && nnz < kRowTileMaxNnz &&
      !(flags & HPSPMM_PLAN_NO_ROW_TILES)) {
    if (int rc = build_row_tiles(p, d_rowptr, d_col, st)) {
      return rc;
    }
  }
  if (p->strategy == HPSPMM_STRATEGY_ROWS && rows_need_tiles && !p->d_tent) p->strategy = HPSPMM_STRATEGY_SEGMENTS;

  if (p->strategy == HPSPMM_STRATEGY_SEGMENTS) {
    const int forced = opt.segment_shift;
    if (forced && (forced < 3 || forced > 15)) {
      return fail(HPSPMM_ERR_INVALID_ARG, "forced segment shift %d outside [3, 15]", forced);
    }
    p->shift = forced ? forced : choose_shift(nnz, k, p->max_row_nnz);
    p->nseg = ceil_div(nnz, (int64_t)1 << p->shift);
    // what the segments kernels need (the row of every nonzero, the carry slots) is allocated at the
    // end, if the plan is still a segments plan then: the layouts tried below mostly replace both
  }
  const bool want_cluster = (flags & HPSPMM_PLAN_CLUSTER) != 0;
  // large enough for an order of its rows by community to pay, if it has communities (a square matrix
  // is taken as a graph on its rows, any other as the bipartite graph of its rows and columns)
  const bool cluster_candidate = nnz >= kClusterMinNnz && nnz >= rows * kClusterMinMeanNnz &&
                                 cols * k * 4 >= (miss <= kLocalMissShare ? kClusterLocalMinBBytes : kClusterMinBBytes) &&
                                 !(flags & HPSPMM_PLAN_NO_CLUSTER);
  // Long rows over a B that is small against the gather volume: every wavefront walks B window by
  // window (tried first: where it qualifies it beats the routed strategy - social graph, 233k
  // vertices, K = 32 / 64 / 128: 1.09 / 1.68 / 2.86 ms against 1.11 / 1.92 / 3.72).  When the matrix
  // does not qualify, or cannot be laid out that way (unsorted columns, more than 2^24 columns),
  // the plan stays what it was.
  if (p->strategy == HPSPMM_STRATEGY_SEGMENTS && fast_k(k) && nnz > 0 && !(flags & HPSPMM_PLAN_NO_SWEEP) &&
      ((flags & HPSPMM_PLAN_FORCE_SWEEP) ||
       !(flags & (HPSPMM_PLAN_FORCE_SEGMENTS | HPSPMM_PLAN_FORCE_ROUTED | HPSPMM_PLAN_CLUSTER)))) {
    // (where the gain expected is small, a matrix that may have communities is served better by the
    // ordered strategy, which is tried first then: co-purchase graph at 6 M nonzeros, K = 32: sweep
    // 87 us, whole rows 87, ordered 65)
    if (int rc = build_sweep(p, d_rowptr, d_col, (flags & HPSPMM_PLAN_FORCE_SWEEP) != 0,
                             (cluster_candidate ? kSweepSureGain : kSweepMinGain) * rows_us, opt, st))
      return rc;
  }
  if (p->strategy == HPSPMM_STRATEGY_SEGMENTS && fast_k(k) && !(flags & HPSPMM_PLAN_NO_ROUTED) && nnz > 0 &&
      !rows_range &&
      (xcd_ok || (flags & HPSPMM_PLAN_FORCE_ROUTED)) &&
      !(flags & HPSPMM_PLAN_FORCE_SEGMENTS && !(flags & HPSPMM_PLAN_FORCE_ROUTED))) {
    if (int rc = build_routed(p, d_rowptr, d_col, (flags & HPSPMM_PLAN_FORCE_ROUTED) != 0, opt, ranking, st)) return rc;
  }
  // Community structure: not routed and B does not fit the L2s - look for clusters of rows that
  // share columns.  Tried before the hub cache: a graph can have
  // both popular columns and communities (the co-purchase graph at a quarter of its size: the 64k
  // most referenced columns take a quarter of the nonzeros there), and the ordered strategy is then
  // the faster of the two (0.73 ms against 1.15 ms for segments with the hub cache).
  if (p->strategy == HPSPMM_STRATEGY_SEGMENTS && fast_k(k) && nnz > 0 &&
      !(flags & HPSPMM_PLAN_NO_CLUSTER) && (want_cluster || (!(flags & HPSPMM_PLAN_FORCE_SEGMENTS) && cluster_candidate))) {
    int32_t* d_order = nullptr;
    double intra_share = 0.0;
    int rc = cluster_rows(p, d_rowptr, d_col, opt, st, &d_order, &intra_share);
    if (rc == HPSPMM_OK && d_order && (want_cluster || intra_share >= kClusterMinIntra))
      rc = build_ordered(p, d_rowptr, d_col, d_order, want_cluster ? 0.0 : kClusterMinServed, st);
    if (d_order) (void)hipFree(d_order);
    if (rc) {
      return rc;
    }
  }
  if (p->strategy == HPSPMM_STRATEGY_SEGMENTS && fast_k(k) && nnz > 0 && rows_us > 0 &&
      !(flags & (HPSPMM_PLAN_NO_SWEEP | HPSPMM_PLAN_FORCE_SEGMENTS | HPSPMM_PLAN_FORCE_ROUTED | HPSPMM_PLAN_CLUSTER))) {
    if (int rc = build_sweep(p, d_rowptr, d_col, false, kSweepMinGain * rows_us, opt, st)) return rc;
  }
  if (p->strategy == HPSPMM_STRATEGY_SEGMENTS && (rows_range || rows_fallback) && row_tiles_serve(k, opt)) {
    // no communities: whole rows after all, if the row tiles get built
    if (int rc = build_row_tiles(p, d_rowptr, d_col, st)) {
      return rc;
    }
    if (p->d_tent) {
      if (p->d_nnz_row) {  // a layout tried above has asked for it
        (void)hipFree(p->d_nnz_row);
        p->d_nnz_row = nullptr;
        p->workspace_bytes -= (int64_t)((size_t)std::max<int64_t>(nnz, 1) * sizeof(int32_t));
      }
      p->nseg = 0;
      p->shift = 0;
      p->strategy = HPSPMM_STRATEGY_ROWS;
    }
  }
  if (p->d_tent && fast_k(k)) {
    // 2^n consecutive groups of row tiles to an XCD at a time instead of one (n by the size, at the
    // launch): rows that share columns with their neighbours then share an L2.  Mesh with 2 random
    // entries per row, 1.5 / 12 M nonzeros, K = 32 / 64 / 128: 20 / 36 / 64 -> 17 / 31 / 59 and 148 / 268 /
    // 600 -> 127 / 253 / 589 us; blocks along the diagonal, 10 M: 98 / 178 / 377 -> 86 / 169 / 373; 85 M:
    // -1 to -2 %.  Matrices without such an order pay up to 3 % (R-MAT at 0.9 to 7.6 M nonzeros +2 to
    // +3 %, users x items +1 to +2 %, the mesh at 102 M +0 to +2 %, the others +-1 %), a launch of
    // microseconds more (the 20k-vertex citation graph +2 to +5 %): from 2^21 nonzeros only.
    // (One contiguous range of the tiles per XCD does the same for the mesh, -14 to -24 %, but costs
    // the others up to 30 %: the tiles lie sorted by the length class of their rows, so the ranges
    // are not equally heavy, also when cut by estimated work.)
    p->rt_chunk_log2 = opt.row_tiles_chunk_log2 > 0   ? opt.row_tiles_chunk_log2
                       : opt.row_tiles_chunk_log2 < 0 ? 0
                       : nnz >= kRowTileChunksMinNnz  ? -1
                                                      : 0;
  }
  if (p->d_tent && !fast_k(k)) {
    // Row tiles at a row length of its own.  The gathers are fastest when every 32-column tile of a
    // row of B is one aligned 128-byte line (R-MAT graph, 3.7 M nonzeros: K = 96 131 us, K = 100
    // 186 us as it lies).  A B whose rows do not even start at multiples of 32 bytes is therefore
    // read through a copy with rows padded to a multiple of 32 floats, refreshed at the start of
    // every SpMM, where that copy is cheap against the gathers - 40 nonzeros for every row of B,
    // 2^20 in all (co-purchase graph, 2.5 M nonzeros, K = 100: 140 -> 118 us, K = 41: 77 -> 66;
    // but K = 200: 267 -> 319, K = 48: 58 -> 64; R-MAT, 28 nonzeros a row, K = 172: 291 -> 342;
    // co-purchase graph at 0.6 M nonzeros, K = 41: 16.5 -> 20.2).  hpspmm_plan_options.row_tiles_pad:
    // never / whenever the length is not a multiple of 32, for comparisons.
    // Otherwise the rows stay as they lie; a length that is not a multiple of 4 is then gathered
    // with 16-byte loads at 4-byte alignment - except below 4 columns, where a row is shorter than
    // one such load: the copy then has rows of 4 floats.
    const bool pad = k < 4 || (k % 32 != 0 && (opt.row_tiles_pad >= 0 ? opt.row_tiles_pad != 0
                                                                      : (k > 32 && k % 8 != 0 && nnz >= 2 * kRowTilePadMinNnz &&
                                                                         nnz >= 40 * cols)));
    p->rt_ldb = (uint32_t)(k < 4 ? 4 : pad ? (k + 31) & ~(int64_t)31 : k);
    p->rt_mode = pad ? 2 : k % 4 ? 3 : 1;
    // lanes per entry: 8 (32 columns at a time), or 4 / 1 when there are at most 16 / 4 columns, so that
    // a slot works on 2 / 8 of its entries at a time
    p->rt_sub = !opt.row_tiles_narrow ? 8 : k <= 4 ? 1 : k <= 16 ? 4 : 8;
    p->rt_same_xcd = opt.row_tiles_same_xcd;
    if (pad) {
      const size_t pad_bytes = (size_t)std::max<int64_t>(cols, 1) * (size_t)p->rt_ldb * sizeof(float);
      if (hipMalloc(&p->d_bpad, pad_bytes) != hipSuccess) {
        (void)hipGetLastError();
        p->d_bpad = nullptr;
        return fail(HPSPMM_ERR_ALLOC, "device allocation of %zu bytes for the padded copy of B failed", pad_bytes);
      }
      p->workspace_bytes += (int64_t)pad_bytes;
    }
  }
  if (p->strategy == HPSPMM_STRATEGY_SEGMENTS && fast_k(k) && !(flags & HPSPMM_PLAN_NO_HUB_CACHE) && nnz > 0) {
    if (int rc = build_hub_cache(p, d_col, opt.hub_log2, (flags & HPSPMM_PLAN_HUB_CACHE) != 0, ranking, st)) {
      return rc;
    }
  }
  if (p->strategy == HPSPMM_STRATEGY_ROWS && !p->d_tent && p->max_row_nnz > kLongRowThreshold) {
    // list of the rows that get a whole wavefront; d_meta[3] counts them
    p->long_threshold = kLongRowThreshold;
    const int64_t cap = nnz / (kLongRowThreshold + 1) + 1;  // cannot be more rows than that
    if (hipMalloc(&p->d_long_rows, (size_t)cap * sizeof(int32_t)) != hipSuccess) {
      (void)hipGetLastError();
      return fail(HPSPMM_ERR_ALLOC, "device allocation of the long-row list failed");
    }
    p->workspace_bytes += cap * (int64_t)sizeof(int32_t);
    hipLaunchKernelGGL(hpspmm::collect_long_rows_kernel, dim3((unsigned)ceil_div(rows, hpspmm::kBlock)),
                       dim3(hpspmm::kBlock), 0, st, rows, d_rowptr, p->long_threshold, p->d_long_rows, d_meta + 3);
    int32_t n_long = 0;
    hipError_t e = hipMemcpyAsync(&n_long, d_meta + 3, sizeof n_long, hipMemcpyDeviceToHost, st);
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    if (e != hipSuccess || n_long < 0 || n_long > cap) {
      return fail(HPSPMM_ERR_HIP, "long-row collection failed: %s", hipGetErrorString(e));
    }
    p->n_long = n_long;
  }
  if (p->strategy == HPSPMM_STRATEGY_SEGMENTS) {
    if (int rc = ensure_row_expansion(p, d_rowptr, st)) return rc;
    // (a carry slot holds a row of K rounded up to 4 floats, so that slots stay 16-byte aligned for any K)
    const size_t carry_bytes = (size_t)std::max<int64_t>(p->nseg, 1) * 2 * (size_t)((k + 3) & ~(int64_t)3) * sizeof(float);
    if (!p->d_carry) {
      if (hipMalloc(&p->d_carry, carry_bytes) != hipSuccess) {
        (void)hipGetLastError();
        p->d_carry = nullptr;
        return fail(HPSPMM_ERR_ALLOC, "device allocation of %zu bytes for the plan failed", carry_bytes);
      }
      p->workspace_bytes += (int64_t)carry_bytes;
    }
    const hipError_t e = hipStreamSynchronize(st);
    if (e != hipSuccess) return fail(HPSPMM_ERR_HIP, "row expansion failed: %s", hipGetErrorString(e));
  }
  holder.plan = nullptr;
  *plan_out = p;
  return HPSPMM_OK;
}

// No C++ exception crosses the C ABI: the host-side steps of plan construction allocate vectors
// sized by the input, and a failed allocation there becomes HPSPMM_ERR_ALLOC; the plan under
// construction and the temporaries of the step that threw are freed by their guards.
int plan_create_guarded(int64_t rows, int64_t cols, int64_t nnz, const int32_t* d_rowptr, const int32_t* d_col,
                        int64_t k, const PlanOptions& opt, void* stream, hpspmm_plan** plan_out) {
  int rc;
  try {
    rc = plan_create_impl(rows, cols, nnz, d_rowptr, d_col, k, opt, stream, plan_out);
  } catch (const std::bad_alloc&) {
    if (plan_out) *plan_out = nullptr;
    rc = fail(HPSPMM_ERR_ALLOC, "out of host memory while building the plan");
  } catch (const std::exception& e) {
    if (plan_out) *plan_out = nullptr;
    rc = fail(HPSPMM_ERR_ALLOC, "plan construction failed: %s", e.what());
  }
  return rc;
}

// The sizes packed into a flag word (segment length, hub rows, routed row length and phases).
PlanOptions options_from_flags(uint32_t flags) {
  PlanOptions o;
  o.flags = flags;
  o.segment_shift = (int)((flags >> 8) & 0xFu);
  o.hub_log2 = (int)((flags >> 16) & 0x1Fu);
  o.routed_row_log2 = (int)((flags >> 24) & 0x1Fu);
  o.routed_phases = (int)((flags >> 29) & 0x7u);
  return o;
}

}  // namespace

HPSPMM_API int hpspmm_plan_create(int64_t rows, int64_t cols, int64_t nnz, const int32_t* d_rowptr,
                                  const int32_t* d_col, int64_t k, uint32_t flags, void* stream,
                                  hpspmm_plan** plan_out) {
  return plan_create_guarded(rows, cols, nnz, d_rowptr, d_col, k, options_from_flags(flags), stream, plan_out);
}

HPSPMM_API int hpspmm_plan_create_ordered(int64_t rows, int64_t cols, int64_t nnz, const int32_t* d_rowptr,
                                          const int32_t* d_col, int64_t k, uint32_t flags,
                                          const int32_t* d_row_order, void* stream, hpspmm_plan** plan_out) {
  if (rows > 0 && !d_row_order) return fail(HPSPMM_ERR_INVALID_ARG, "d_row_order is NULL");
  PlanOptions o = options_from_flags(flags);
  o.d_row_order = d_row_order;
  return plan_create_guarded(rows, cols, nnz, d_rowptr, d_col, k, o, stream, plan_out);
}

HPSPMM_API int hpspmm_plan_create_ex(int64_t rows, int64_t cols, int64_t nnz, const int32_t* d_rowptr,
                                     const int32_t* d_col, int64_t k, const hpspmm_plan_options* options,
                                     void* stream, hpspmm_plan** plan_out) {
  hpspmm_plan_options in;
  std::memset(&in, 0, sizeof in);
  if (options) {
    // a caller compiled against an older header passes a shorter struct: what it lacks stays zero
    if (options->struct_size < 2 * sizeof(uint32_t) || options->struct_size % 4 != 0)
      return fail(HPSPMM_ERR_INVALID_ARG, "hpspmm_plan_options.struct_size = %u is not the size of such a struct",
                  options->struct_size);
    std::memcpy(&in, options, std::min<size_t>(options->struct_size, sizeof in));
  }
  PlanOptions o = options_from_flags(in.flags);
  o.d_row_order = in.d_row_order;
  if (in.segment_shift) o.segment_shift = in.segment_shift;
  if (in.hub_log2) o.hub_log2 = in.hub_log2;
  if (in.routed_row_log2) o.routed_row_log2 = in.routed_row_log2;
  if (in.routed_phases) o.routed_phases = in.routed_phases;
  o.routed_tile_width = in.routed_tile_width;
  if (!(o.routed_tile_width == 0 || o.routed_tile_width == -1 || o.routed_tile_width == 32 || o.routed_tile_width == 64))
    return fail(HPSPMM_ERR_INVALID_ARG, "routed_tile_width must be 0, -1, 32 or 64, got %d", o.routed_tile_width);
  o.routed_split_launch = in.routed_split_launch != 0;
  o.routed_lds_rows = in.routed_lds_rows;
  if (in.xcd_dealing < 0 || in.xcd_dealing > 2) return fail(HPSPMM_ERR_INVALID_ARG, "xcd_dealing must be 0, 1 or 2");
  o.xcd_dealing = in.xcd_dealing == 0 ? -1 : in.xcd_dealing == 1 ? 1 : 0;
  o.column_tiles = in.no_column_tiles == 0;
  if (in.row_tiles_min_k > 0) o.row_tiles_min_k = in.row_tiles_min_k;
  if (in.row_tiles_pad < 0 || in.row_tiles_pad > 2) return fail(HPSPMM_ERR_INVALID_ARG, "row_tiles_pad must be 0, 1 or 2");
  o.row_tiles_pad = in.row_tiles_pad == 0 ? -1 : in.row_tiles_pad == 1 ? 0 : 1;
  o.row_tiles_narrow = in.row_tiles_wide == 0;
  o.row_tiles_same_xcd = in.row_tiles_round_robin == 0;
  o.sweep_window_log2 = std::max(0, in.sweep_window_log2);
  o.sweep_lead = std::max(0, in.sweep_lead);
  o.sweep_spin = in.sweep_spin == 0 ? -1 : std::max(0, in.sweep_spin);
  o.sweep_limit = std::max(0, in.sweep_limit);
  o.sweep_priorities = in.sweep_no_priorities ? 0 : -1;
  o.cluster_sweeps = std::max(0, in.cluster_sweeps);
  o.report = in.report != 0;
  if (in.row_tiles_chunk_log2 < -1 || in.row_tiles_chunk_log2 > 16)
    return fail(HPSPMM_ERR_INVALID_ARG, "row_tiles_chunk_log2 must be -1 .. 16");
  o.row_tiles_chunk_log2 = in.row_tiles_chunk_log2;
  return plan_create_guarded(rows, cols, nnz, d_rowptr, d_col, k, o, stream, plan_out);
}

HPSPMM_API int hpspmm_plan_get_info(const hpspmm_plan* plan, hpspmm_plan_info* out) {
  if (!plan || !out) return fail(HPSPMM_ERR_INVALID_ARG, "plan or info_out is NULL");
  std::memset(out, 0, sizeof *out);
  out->rows = plan->rows;
  out->cols = plan->cols;
  out->nnz = plan->nnz;
  out->k = plan->k_user;
  out->strategy = plan->strategy;
  const bool segmented = plan->strategy == HPSPMM_STRATEGY_SEGMENTS || plan->strategy == HPSPMM_STRATEGY_ROUTED ||
                         plan->strategy == HPSPMM_STRATEGY_ORDERED;
  out->segment_length = segmented ? (1 << plan->shift) : 0;
  out->num_segments = plan->nseg;
  out->max_row_nnz = plan->max_row_nnz;
  out->empty_rows = plan->empty_rows;
  out->workspace_bytes = plan->workspace_bytes;
  out->launches_per_spmm = plan->strategy == HPSPMM_STRATEGY_ROUTED    ? (plan->d_vsrc ? 2 : 3)
                           : plan->strategy == HPSPMM_STRATEGY_ORDERED ? 2
                           : plan->strategy == HPSPMM_STRATEGY_SWEEP   ? 2
                           : plan->strategy == HPSPMM_STRATEGY_SEGMENTS ? (plan->n_hub > 0 ? 3 : 2)
                                                                        : 1;
  out->launches_per_spmm *= plan->tiles;  // one pass per column tile
  if (plan->d_bpad) out->launches_per_spmm += 1;  // the padded copy of B
  out->column_tiles = plan->tiles;
  out->hub_rows = plan->n_hub;
  out->lds_served_nnz = plan->oserved;
  out->row_tiles = plan->d_tent ? plan->rt_tiles : 0;
  out->stored_order_miss_share = plan->stored_miss;
  return HPSPMM_OK;
}

HPSPMM_API int hpspmm_plan_destroy(hpspmm_plan* plan) {
  if (!plan) return HPSPMM_OK;
  if (plan->d_nnz_row) (void)hipFree(plan->d_nnz_row);
  if (plan->d_carry) (void)hipFree(plan->d_carry);
  if (plan->d_long_rows) (void)hipFree(plan->d_long_rows);
  if (plan->d_hub_ids) (void)hipFree(plan->d_hub_ids);
  if (plan->d_hub_col) (void)hipFree(plan->d_hub_col);
  if (plan->d_bhot) (void)hipFree(plan->d_bhot);
  if (plan->d_bpad) (void)hipFree(plan->d_bpad);
  for (void* q : {(void*)plan->d_rvptr, (void*)plan->d_coldptr, (void*)plan->d_vcol, (void*)plan->d_lslot,
                  (void*)plan->d_chunk_base, (void*)plan->d_chunk_pref,
                  (void*)plan->d_vval, (void*)plan->d_vsrc, (void*)plan->d_vrow, (void*)plan->d_run_row,
                  (void*)plan->d_seg_run, (void*)plan->d_bhot_src, (void*)plan->d_partial,
                  (void*)plan->d_routed_rows, (void*)plan->d_cross_rows, (void*)plan->d_zero_rows,
                  (void*)plan->d_ostart, (void*)plan->d_ocol, (void*)plan->d_run_delta,
                  (void*)plan->d_wcols, (void*)plan->d_tent, (void*)plan->d_ldesc, (void*)plan->d_zrow,
                  (void*)plan->d_sw_base, (void*)plan->d_sw_len, (void*)plan->d_sw_ends, (void*)plan->d_sw_slot_row,
                  (void*)plan->d_sw_part_base, (void*)plan->d_sw_split_rows, (void*)plan->d_sw_zrow})
    if (q) (void)hipFree(q);
  delete plan;
  return HPSPMM_OK;
}

HPSPMM_API int hpspmm_plan_bind_values(hpspmm_plan* plan, const float* d_val, void* stream) {
  if (!plan) return fail(HPSPMM_ERR_INVALID_ARG, "plan is NULL");
  plan->bound_val = nullptr;
  if (!d_val || plan->nnz == 0) return HPSPMM_OK;
  if (plan->strategy == HPSPMM_STRATEGY_SWEEP) {
    if (int rc = bind_values_sweep(plan, d_val, (hipStream_t)stream)) return rc;
  } else if (plan->strategy == HPSPMM_STRATEGY_ROUTED) {
    if (int rc = bind_values_routed(plan, d_val, (hipStream_t)stream)) return rc;
  }
  plan->bound_val = d_val;
  return HPSPMM_OK;
}
