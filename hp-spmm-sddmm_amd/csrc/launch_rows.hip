// Whole rows: the launches over the CSR arrays, over the plan's row tiles, and at row lengths given at run time.
#include "host.hpp"

#include "anyk_kernels.hpp"
#include "rowtile_kernels.hpp"

namespace hpspmm_host {

namespace {

// Column-tile width of the rows kernel: the widest tile of B (cols x KT floats)
// that still fits one XCD's L2 next to the streamed arrays, so that a B too big
// for one L2 is split over the XCDs by columns of B instead of thrashing all
// eight.  Measured on the 20k-vertex citation graph at K=128 (B = 10 MB):
// 14.3 us with one 128-wide tile, 11.9 us with two 64-wide, 11.2 us with four
// 32-wide tiles; at K=64 (B = 5 MB) tiling does not pay (6.8 vs 7.2 us).
constexpr int64_t kRowsUntiledBytes = 6 << 20;  // B up to this size is left in one tile
constexpr int64_t kRowsTileBytes = 3 << 20;     // else: the widest tile of B not larger than this

template <int K, int KT>
int launch_rows_tiled(int64_t rows, const int32_t* rp, const int32_t* ci, const float* v, const float* B, float* C,
                      int32_t long_threshold, const int32_t* long_rows, int64_t n_long, hipStream_t st) {
  const int64_t short_blocks = row_blocks(rows, KT);
  const int64_t blocks = (short_blocks + ceil_div(n_long, hpspmm::kWavesPerBlock)) * (K / KT);
  if (blocks > INT32_MAX) return fail(HPSPMM_ERR_INVALID_ARG, "grid too large");
  hipLaunchKernelGGL((hpspmm::spmm_rows_kernel<K, KT>), dim3((unsigned)blocks), dim3(hpspmm::kBlock), 0, st, rows, rp,
                     ci, v, B, C, short_blocks, long_threshold, long_rows, n_long);
  mark_launch(st, "spmm_rows_kernel");
  return HPSPMM_OK;
}

template <int K>
int launch_rows(int64_t rows, int64_t cols, const int32_t* rp, const int32_t* ci, const float* v, const float* B,
                float* C, int32_t long_threshold, const int32_t* long_rows, int64_t n_long, hipStream_t st) {
  if constexpr (K >= 64) {
    // 32-wide tiles only: a 64-wide tile of a B beyond kRowsUntiledBytes can never be within kRowsTileBytes
    if (cols * K * 4 > kRowsUntiledBytes && cols * 32 * 4 <= kRowsTileBytes)
      return launch_rows_tiled<K, 32>(rows, rp, ci, v, B, C, long_threshold, long_rows, n_long, st);
  }
  return launch_rows_tiled<K, K>(rows, rp, ci, v, B, C, long_threshold, long_rows, n_long, st);
}

// The row-tile kernels read val[0] for padding entries (and discard it): a matrix without
// nonzeros may come with val == NULL, so give them some readable address then.
inline const float* readable_values(const hpspmm_plan* p, const float* v) {
  return p->nnz > 0 ? v : reinterpret_cast<const float*>(p->d_tent);
}

// Row tiles at a row length outside the tuned set (K = 0 in the templates below): ldb, ldc = floats
// between the rows of B and of C (= the columns there are); column tiles of 32.
inline int64_t row_tile_column_tiles(int k_template, uint32_t ldc) {
  return k_template ? k_template / 32 : (int64_t)((ldc + 31u) / 32u);
}

// The column tiles of a group of row tiles on one XCD: where the rows of B are not whole 128-byte
// lines, so that neighbouring tiles share lines (citation graph x 16, 1.6 M nonzeros, K = 100: 245 us
// with the tiles dealt round robin, 148 so; R-MAT 3.7 M nonzeros, K = 172: 392 -> 291).
// (hpspmm_plan_options.row_tiles_same_xcd = 0: round robin, for comparisons.)
inline bool row_tiles_same_xcd(const hpspmm_plan* p, int kLd, uint32_t ldb) {
  return kLd != 0 && ldb % 32 != 0 && p->rt_same_xcd;
}

// Chunks of consecutive groups of row tiles per XCD (tuned row lengths): how large, and how many
// workgroups that takes.  `long_groups` = the groups at the front of the layout that hold the long
// rows, which stay dealt one at a time.  chunk_log2 = 0 in the result: no chunks.
hpspmm::TileChunks row_tile_chunks(const hpspmm_plan* p, int kLd, int64_t k_template, int64_t groups, int64_t long_groups,
                                   int64_t* blocks) {
  hpspmm::TileChunks tc{0, 0, (int32_t)groups, 0};
  if (kLd != 0 || k_template <= 0 || p->rt_chunk_log2 == 0) return tc;
  const int64_t ways = hpspmm::kXcds / (k_template / 32);
  long_groups = std::min(long_groups, groups);
  // the plan's own choice (-1): the largest n <= 9 that leaves every XCD 16 chunks - one chunk more
  // or less is then 6 % of its work at most
  int n = p->rt_chunk_log2 > 0 ? p->rt_chunk_log2 : 9;
  if (p->rt_chunk_log2 < 0)
    while (n > 0 && groups - long_groups < (16 * ways << n)) --n;
  if (n <= 0 || groups - long_groups < (2 * ways << n)) return tc;
  tc.chunk_log2 = n;
  tc.long_groups = (int32_t)long_groups;
  tc.long_per = (int32_t)ceil_div(long_groups, ways);
  *blocks = (int64_t)hpspmm::kXcds * (tc.long_per + (ceil_div(groups - long_groups, ways << n) << n));
  return tc;
}

template <int K, int WPB, int kLd, int kSub>
int launch_row_tiles_w(const hpspmm_plan* p, const float* v, const float* B, float* C, hipStream_t st, uint32_t ldb,
                       uint32_t ldc) {
  const bool same_xcd = row_tiles_same_xcd(p, kLd, ldb);
  const int64_t groups = ceil_div(p->rt_waves, WPB);
  int64_t blocks = (same_xcd ? ceil_div(groups, hpspmm::kXcds) * hpspmm::kXcds : groups) * row_tile_column_tiles(K, ldc);
  const hpspmm::TileChunks chunks = row_tile_chunks(p, kLd, K, groups, ceil_div(p->rt_loop, WPB), &blocks);
  if (blocks > INT32_MAX) return fail(HPSPMM_ERR_INVALID_ARG, "grid too large");
  if constexpr (kLd == 0) {
    if (chunks.chunk_log2 > 0) {
      hipLaunchKernelGGL((hpspmm::spmm_rowtiles_kernel<K, WPB, kLd, kSub, true>), dim3((unsigned)blocks), dim3(WPB * 64), 0,
                         st, p->rt_waves, p->rt_loop, p->rt_loop_tiles, p->d_ldesc, p->d_tent, readable_values(p, v), B, C,
                         p->d_zrow + 4, ldb, ldc, same_xcd, chunks);
      mark_launch(st, "spmm_rowtiles_kernel");
      return HPSPMM_OK;
    }
  }
  hipLaunchKernelGGL((hpspmm::spmm_rowtiles_kernel<K, WPB, kLd, kSub>), dim3((unsigned)blocks), dim3(WPB * 64), 0, st,
                     p->rt_waves, p->rt_loop, p->rt_loop_tiles, p->d_ldesc, p->d_tent, readable_values(p, v), B, C,
                     p->d_zrow + 4, ldb, ldc, same_xcd, hpspmm::NoTileChunks{});
  mark_launch(st, "spmm_rowtiles_kernel");
  return HPSPMM_OK;
}

template <int K, int WPB, int kLd, int kSub>
int launch_row_tiles_wg(const hpspmm_plan* p, const float* v, const float* B, float* C, hipStream_t st, uint32_t ldb,
                        uint32_t ldc) {
  const int64_t wave_items = (p->rt_loop - p->rt_wg) + (p->rt_tiles - p->rt_loop_tiles);
  const bool same_xcd = row_tiles_same_xcd(p, kLd, ldb);
  const int64_t groups = p->rt_wg + ceil_div(wave_items, WPB);
  int64_t blocks = (same_xcd ? ceil_div(groups, hpspmm::kXcds) * hpspmm::kXcds : groups) * row_tile_column_tiles(K, ldc);
  const hpspmm::TileChunks chunks =
      row_tile_chunks(p, kLd, K, groups, p->rt_wg + ceil_div(p->rt_loop - p->rt_wg, WPB), &blocks);
  if (blocks > INT32_MAX) return fail(HPSPMM_ERR_INVALID_ARG, "grid too large");
  if constexpr (kLd == 0) {
    if (chunks.chunk_log2 > 0) {
      hipLaunchKernelGGL((hpspmm::spmm_rowtiles_wg_kernel<K, WPB, kLd, kSub, true>), dim3((unsigned)blocks), dim3(WPB * 64),
                         0, st, p->rt_tiles, p->rt_wg, p->rt_loop, p->rt_loop_tiles, p->d_ldesc, p->d_tent,
                         readable_values(p, v), B, C, p->d_zrow + 4, ldb, ldc, same_xcd, chunks);
      mark_launch(st, "spmm_rowtiles_wg_kernel");
      return HPSPMM_OK;
    }
  }
  hipLaunchKernelGGL((hpspmm::spmm_rowtiles_wg_kernel<K, WPB, kLd, kSub>), dim3((unsigned)blocks), dim3(WPB * 64), 0, st,
                     p->rt_tiles, p->rt_wg, p->rt_loop, p->rt_loop_tiles, p->d_ldesc, p->d_tent,
                     readable_values(p, v), B, C, p->d_zrow + 4, ldb, ldc, same_xcd, hpspmm::NoTileChunks{});
  mark_launch(st, "spmm_rowtiles_wg_kernel");
  return HPSPMM_OK;
}

// One wavefront per workgroup while the grid stays small (20k-vertex citation graph, K=32:
// 3.66 us against 3.75 us with four), four beyond that.  A matrix with rows beyond
// kRowTileWorkgroupRows nonzeros gets a workgroup of 8 or 16 wavefronts on each of those rows:
// one wavefront needs about 0.6 us per 64 nonzeros, which a 16k-nonzero row turns into 150 us.
constexpr int64_t kRowTileSmallGrid = 1 << 15;

template <int K, int kLd = 0, int kSub = hpspmm::kSlot>
int launch_row_tiles(const hpspmm_plan* p, const float* v, const float* B, float* C, hipStream_t st,
                     uint32_t ldb = K, uint32_t ldc = K) {
  if (p->rt_wg > 0) {
    if (p->max_row_nnz > 8192) return launch_row_tiles_wg<K, 16, kLd, kSub>(p, v, B, C, st, ldb, ldc);
    return launch_row_tiles_wg<K, 8, kLd, kSub>(p, v, B, C, st, ldb, ldc);
  }
  if ((int64_t)p->rt_waves * row_tile_column_tiles(K, ldc) <= kRowTileSmallGrid)
    return launch_row_tiles_w<K, 1, kLd, kSub>(p, v, B, C, st, ldb, ldc);
  return launch_row_tiles_w<K, hpspmm::kWavesPerBlock, kLd, kSub>(p, v, B, C, st, ldb, ldc);
}

template <int GP, bool kOdd>
int launch_rows_anyk_g(int64_t rows, int64_t k, const int32_t* rp, const int32_t* ci, const float* v, const float* B,
                       float* C, int32_t long_threshold, const int32_t* long_rows, int64_t n_long, hipStream_t st) {
  const int tiles = anyk_tiles(k);
  const int64_t short_blocks = ceil_div(ceil_div(rows, 64 / GP), hpspmm::kWavesPerBlock);
  const int64_t blocks = (short_blocks + ceil_div(n_long, hpspmm::kWavesPerBlock)) * tiles;
  if (blocks > INT32_MAX) return fail(HPSPMM_ERR_INVALID_ARG, "grid too large");
  hipLaunchKernelGGL((hpspmm::spmm_rows_anyk_kernel<GP, kOdd>), dim3((unsigned)blocks), dim3(hpspmm::kBlock), 0, st, rows,
                     (int)k, tiles, rp, ci, v, B, C, short_blocks, long_threshold, long_rows, n_long);
  mark_launch(st, "spmm_rows_anyk_kernel");
  return HPSPMM_OK;
}

int launch_rows_anyk(int64_t rows, int64_t k, const int32_t* rp, const int32_t* ci, const float* v, const float* B,
                     float* C, int32_t long_threshold, const int32_t* long_rows, int64_t n_long, hipStream_t st) {
  return dispatch_anyk_lanes(k, [&](auto GP) {
    constexpr int gp = decltype(GP)::value;
    return odd_k(k) ? launch_rows_anyk_g<gp, true>(rows, k, rp, ci, v, B, C, long_threshold, long_rows, n_long, st)
                    : launch_rows_anyk_g<gp, false>(rows, k, rp, ci, v, B, C, long_threshold, long_rows, n_long, st);
  });
}

}  // namespace

int launch_rows_any(int64_t rows, int64_t cols, int64_t k, const int32_t* rp, const int32_t* ci, const float* v,
                    const float* B, float* C, int32_t long_threshold, const int32_t* long_rows, int64_t n_long,
                    hipStream_t st) {
  if (rows == 0) return HPSPMM_OK;
  if (!fast_k(k)) return launch_rows_anyk(rows, k, rp, ci, v, B, C, long_threshold, long_rows, n_long, st);
  return dispatch_k(k, [&](auto K) {
    return launch_rows<decltype(K)::value>(rows, cols, rp, ci, v, B, C, long_threshold, long_rows, n_long, st);
  });
}

int launch_row_tiles_plan(const hpspmm_plan* p, const float* v, const float* B, float* C, hipStream_t st) {
  if (!p->rt_mode)
    return dispatch_k(p->k, [&](auto K) { return launch_row_tiles<decltype(K)::value>(p, v, B, C, st); });
  // a row length of its own: B as it lies (1: a multiple of 4; 3: any, gathered at 4-byte alignment)
  // or through the plan's padded copy (2), by 8, 4 or 1 lanes per entry
  const uint32_t ldb = p->rt_ldb, ldc = (uint32_t)p->k;
  const int sub = p->rt_sub;
  if (p->rt_mode == 2) {
    if (p->nnz > 0) {  // (without nonzeros B is never read, and may be NULL)
      if (int rc = launch_pad_rows(p->cols, p->k, (int64_t)ldb, B, p->d_bpad, st)) return rc;
    }
    return sub == 1   ? launch_row_tiles<0, 2, 1>(p, v, p->d_bpad, C, st, ldb, ldc)
           : sub == 4 ? launch_row_tiles<0, 2, 4>(p, v, p->d_bpad, C, st, ldb, ldc)
                      : launch_row_tiles<0, 2>(p, v, p->d_bpad, C, st, ldb, ldc);
  }
  if (p->rt_mode == 3)
    return sub == 4 ? launch_row_tiles<0, 3, 4>(p, v, B, C, st, ldb, ldc) : launch_row_tiles<0, 3>(p, v, B, C, st, ldb, ldc);
  return sub == 1   ? launch_row_tiles<0, 1, 1>(p, v, B, C, st, ldb, ldc)
         : sub == 4 ? launch_row_tiles<0, 1, 4>(p, v, B, C, st, ldb, ldc)
                    : launch_row_tiles<0, 1>(p, v, B, C, st, ldb, ldc);
}

int launch_pad_rows(int64_t rows, int64_t k, int64_t kp, const float* src, float* dst, hipStream_t st) {
  hipLaunchKernelGGL(hpspmm::pad_rows_kernel, dim3(grid_for(rows * kp, 1 << 16)), dim3(hpspmm::kBlock), 0, st, rows, k, kp,
                     src, dst);
  mark_launch(st, "pad_rows_kernel");
  return HPSPMM_OK;
}

}  // namespace hpspmm_host
