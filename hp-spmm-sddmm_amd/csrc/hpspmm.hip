// Host side of libhpspmm.so: the C ABI declared in include/hpspmm.h, the plan
// (device-side work assignment) and the kernel launches.
#include "hpspmm.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <climits>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <new>
#include <string>
#include <vector>

#include "anyk_kernels.hpp"
#include "ordered_kernels.hpp"
#include "rank_kernels.hpp"
#include "routed_kernels.hpp"
#include "rowtile_kernels.hpp"
#include "spmm_kernels.hpp"
#include "sweep_kernels.hpp"

namespace {

thread_local std::string g_last_error;

int fail(int code, const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  g_last_error = buf;
  return code;
}

#define HPSPMM_HIP(call)                                                                       \
  do {                                                                                         \
    hipError_t e_ = (call);                                                                    \
    if (e_ != hipSuccess)                                                                      \
      return fail(e_ == hipErrorNoDevice ? HPSPMM_ERR_NO_DEVICE : HPSPMM_ERR_HIP, "%s: %s",    \
                  #call, hipGetErrorString(e_));                                               \
  } while (0)

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Per-launch timing (hpspmm_csr_spmm_timed_launches): while a trace is active on the calling
// thread, every kernel launch of an SpMM is followed by an event record on the launch stream.
constexpr int kMaxTracedLaunches = 8;
struct LaunchTrace {
  hipEvent_t ev[kMaxTracedLaunches];
  const char* name[kMaxTracedLaunches];
  int n = 0;
};
thread_local LaunchTrace* g_trace = nullptr;
inline void mark_launch(hipStream_t st, const char* name) {
  LaunchTrace* t = g_trace;
  if (!t || t->n >= kMaxTracedLaunches) return;
  (void)hipEventRecord(t->ev[t->n], st);
  t->name[t->n++] = name;
}

inline bool fast_k(int64_t k) { return k == 32 || k == 64 || k == 128; }
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
// Every row length that is not a tuned size goes to the run-time-K sub-wave kernels.
// Not a multiple of 4: rows of B and C start at any multiple of 4 bytes, the last lane of a row owns 1 to 3 columns.
inline bool odd_k(int64_t k) { return k % 4 != 0; }
// Lanes per sub-wave for such a K: the power of two that covers a column tile (at most 128 floats).
// Row tiles (32-column tiles of B and C) serve every row length
// (HPSPMM_ROW_TILES_MIN_K in the environment: only from there up, for comparisons).
inline bool row_tiles_serve(int64_t k) {
  if (fast_k(k)) return true;
  if (k >= ((int64_t)1 << 22)) return false;
  const char* e = std::getenv("HPSPMM_ROW_TILES_MIN_K");
  return k >= (e ? (int64_t)std::atoll(e) : (int64_t)1);
}

inline int anyk_lanes(int64_t k) {
  const int64_t g = ((k < hpspmm::kAnyKTile ? k : hpspmm::kAnyKTile) + 3) / 4;
  int gp = 2;
  while (gp < g) gp <<= 1;
  return gp;
}
inline int anyk_tiles(int64_t k) { return (int)((k + hpspmm::kAnyKTile - 1) / hpspmm::kAnyKTile); }

inline bool aligned16(const void* a, const void* b, const void* c) {
  return (((uintptr_t)a | (uintptr_t)b | (uintptr_t)c) & 15u) == 0;
}

int check_dims(int64_t rows, int64_t cols, int64_t nnz, int64_t k) {
  if (rows < 0 || cols < 0 || nnz < 0) return fail(HPSPMM_ERR_INVALID_ARG, "negative dimension (rows=%lld cols=%lld nnz=%lld)",
                                                   (long long)rows, (long long)cols, (long long)nnz);
  if (rows >= INT32_MAX || cols > INT32_MAX || nnz > INT32_MAX)
    return fail(HPSPMM_ERR_INVALID_ARG, "dimension exceeds the int32 index range (rows=%lld cols=%lld nnz=%lld)",
                (long long)rows, (long long)cols, (long long)nnz);
  if (k <= 0 || k > (1 << 20)) return fail(HPSPMM_ERR_INVALID_ARG, "k must be in [1, 2^20], got %lld", (long long)k);
  if (nnz > 0 && cols == 0) return fail(HPSPMM_ERR_INVALID_ARG, "nnz > 0 with cols == 0");
  return HPSPMM_OK;
}

int grid_for(int64_t items, int64_t cap = 1 << 20) {
  int64_t b = ceil_div(items, hpspmm::kBlock);
  if (b < 1) b = 1;
  if (b > cap) b = cap;
  return (int)b;
}

}  // namespace

struct hpspmm_plan {
  int64_t rows = 0, cols = 0, nnz = 0, k = 0;
  // A row length that is a multiple of 4 but not a tuned one (256 = 2 x 128, 40 = one tile of 64 with
  // 10 of its 16 lanes) can be served by a layout built for a tuned length, one column tile after
  // the other: k is then the tile width, k_full the row length of B and C, tiles = ceil(k_full / k).
  // Otherwise k_full = k, tiles = 1.
  int64_t k_full = 0;
  int tiles = 1;
  // The caller's row length when it is not a multiple of 4 and a tuned layout serves it all the same:
  // k_full is then that length rounded up to 4, B is read through a copy with rows padded to k_full
  // (d_bpad, refreshed at the start of every SpMM), C is written in place.  Otherwise k_user = k_full.
  int64_t k_user = 0;
  float* d_bpad = nullptr;
  int strategy = 0;
  int shift = 0;  // log2(segment length)
  int64_t nseg = 0;
  int64_t max_row_nnz = 0, empty_rows = 0;
  bool xcd_remap = true;
  // the arrays the plan was built from: hpspmm_csr_spmm refuses others unless the caller opted out
  const int32_t* src_rowptr = nullptr;
  const int32_t* src_col = nullptr;
  bool allow_moved = false;
  int32_t* d_nnz_row = nullptr;  // [nnz]
  float* d_carry = nullptr;      // [2 * nseg * k]
  // hub cache (segments strategy, optional): the n_hub most referenced rows of B
  int32_t* d_hub_ids = nullptr;  // [n_hub] column index of every cached row
  int32_t* d_hub_col = nullptr;  // [nnz] column indices with cached columns rewritten as ~slot
  float* d_bhot = nullptr;       // [n_hub * k]
  int64_t n_hub = 0;
  // routed strategy
  hpspmm::RoutedLayout lay{};
  int32_t* d_rvptr = nullptr;     // [(n_routed + 1) * nhub] run starts of the routed rows in the hub classes
  int32_t* d_coldptr = nullptr;   // [rows + 1] run starts in the cold class
  int32_t* d_vcol = nullptr;      // [vtotal] column, or ~compact-buffer row
  uint16_t* d_lslot = nullptr;    // [nnz] rank of every stored nonzero within its chunk sorted by class-major position
  int32_t* d_chunk_base = nullptr;  // [nchunks * ncls] first class-major position of the chunk's run in each class
  int32_t* d_chunk_pref = nullptr;  // [nchunks * ncls] nonzeros of the chunk in lower classes
  float* d_vval = nullptr;        // [vtotal] the values in that order, rewritten by every SpMM (not with d_vsrc)
  int32_t* d_vsrc = nullptr;      // [vtotal] column-range slices: index of every position in the caller's arrays
  int32_t* d_vrow = nullptr;      // [vtotal] routed-row number (hub classes) or row (cold class)
  int32_t* d_bhot_src = nullptr;  // [n_bhot] source column of every compact-buffer row (-1 = unused)
  int32_t* d_routed_rows = nullptr;  // [n_routed] row of every routed-row number
  int32_t* d_cross_rows = nullptr;   // short rows whose run crosses a segment boundary
  int32_t* d_zero_rows = nullptr;    // rows without nonzeros
  int64_t n_cross = 0, n_zero = 0;
  float* d_partial = nullptr;     // [n_routed * nhub * k]
  int64_t n_bhot = 0;
  int64_t routed_grid = 0;
  const float* bound_val = nullptr;  // value array whose class-major copy d_vval currently holds (or NULL)
  // ordered strategy
  int32_t* d_ostart = nullptr;  // [rows] first position of every row in processing order
  int32_t* d_ocol = nullptr;    // [nnz] column, or ~slot of the window's LDS copy of B
  int32_t* d_osrc = nullptr;    // [nnz] original index of the nonzero
  int32_t* d_orow = nullptr;    // [nnz] row of the nonzero
  int32_t* d_wcols = nullptr;   // [windows * ocap] columns held in LDS by each window's workgroup
  int ocap = 0;
  int64_t owindows = 0;
  int64_t oserved = 0;          // nonzeros that read B from LDS
  int32_t* d_long_rows = nullptr;  // rows strategy over the CSR arrays: rows longer than long_threshold
  int64_t n_long = 0;
  int32_t long_threshold = INT32_MAX;
  // rows strategy over row tiles
  int2* d_tent = nullptr;     // [rt_tiles * 64] per tile entry: column (-1 = padding), slot / tile data by lane
  int2* d_ldesc = nullptr;    // [rt_loop] per long row: first tile, tile count
  float* d_zrow = nullptr;    // 4 + 32 zeros: what a padding entry gathers instead of a row of B (from d_zrow + 4)
  int32_t rt_tiles = 0, rt_waves = 0, rt_loop = 0, rt_wg = 0, rt_loop_tiles = 0;
  // Row tiles at a row length outside the tuned set: rt_mode = the kernels' kLd (1: k a multiple of
  // 4, B as it lies; 2: B through d_bpad, its rows padded to rt_ldb floats; 3: any k, B as it lies,
  // gathered at 4-byte alignment), 0 = a tuned row length.
  int rt_mode = 0;
  uint32_t rt_ldb = 0;
  // sweep strategy (its stream arrays are d_vcol = entry words, d_vsrc, d_vval when values are bound;
  // partial-result rows of split rows in d_partial; rows without nonzeros in d_zero_rows)
  hpspmm::SweepLayout sw{};
  uint32_t* d_sw_base = nullptr;       // [n_waves + 1] first stream position of every wavefront
  uint32_t* d_sw_len = nullptr;        // [n_waves] length of each of its sub-wave streams
  int32_t* d_sw_ends = nullptr;        // [n_waves * n_windows] end of every window's chunk in those streams
  int32_t* d_sw_slot_row = nullptr;    // [n_waves * slots] where every accumulator slot is stored
  uint32_t* d_sw_part_base = nullptr;  // [rows + 1] first partial-result row of every split row
  int32_t* d_sw_split_rows = nullptr;  // rows cut into several pieces
  float* d_sw_zrow = nullptr;          // 128 zeros: what a padding entry gathers
  int64_t n_split = 0, sw_total = 0;
  int32_t sw_limit = 0;                // nonzeros per piece, at most
  int32_t sw_bands = 0;
  int64_t workspace_bytes = 0;
};

namespace {

// The routed strategy pins column slices to XCDs and xcd_remap deals row ranges to them; both rely on
// workgroup b of a launch running on XCD b % 8.  That holds for the whole device (8 XCDs, 256 CUs);
// a partitioned device (fewer XCDs behind one HIP device) or a future dispatcher would break it
// silently, so it is measured once per device: 512 probe workgroups report the XCD they ran on.
// 0 = not probed yet, 1 = workgroup b runs on XCD b % 8, 2 = it does not (the plan then keeps to the
// strategies that do not depend on it).
constexpr int kMaxDevices = 64;
constexpr int kProbeBlocks = 512;
std::mutex g_xcd_mutex;
int g_xcd_state[kMaxDevices] = {0};

bool xcd_dealing_holds(hipStream_t st) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    (void)hipGetLastError();
    return false;
  }
  if (const char* forced = std::getenv("HPSPMM_XCD_DEALING")) {  // diagnostics: skip the probe
    if (forced[0] == '0' || forced[0] == '1') return forced[0] == '1';
  }
  std::lock_guard<std::mutex> lock(g_xcd_mutex);
  if (g_xcd_state[dev]) return g_xcd_state[dev] == 1;
  int32_t* d_ids = nullptr;
  int32_t ids[kProbeBlocks];
  bool ok = hipMalloc(&d_ids, sizeof ids) == hipSuccess;
  if (ok) {
    hipLaunchKernelGGL(hpspmm::xcc_probe_kernel, dim3(kProbeBlocks), dim3(64), 0, st, d_ids);
    ok = hipMemcpyAsync(ids, d_ids, sizeof ids, hipMemcpyDeviceToHost, st) == hipSuccess &&
         hipStreamSynchronize(st) == hipSuccess;
  }
  if (d_ids) (void)hipFree(d_ids);
  if (!ok) {
    (void)hipGetLastError();
    return false;  // not cached: a transient failure should not decide for the life of the process
  }
  int match = 0;
  for (int b = 0; b < kProbeBlocks; ++b) match += ids[b] == b % hpspmm::kXcds;
  g_xcd_state[dev] = match == kProbeBlocks ? 1 : 2;
  return g_xcd_state[dev] == 1;
}

// Launch geometry of the kernels that run one sub-wave per row.
inline int64_t row_blocks(int64_t rows, int64_t k) {
  const int64_t per_wave = 64 / (k / 4);
  return ceil_div(ceil_div(rows, per_wave), hpspmm::kWavesPerBlock);
}

// Rows longer than this are handled by a whole wavefront in the rows strategy.
constexpr int32_t kLongRowThreshold = 32;

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

// Row tiles (rows strategy): every row cut into slots of 8 nonzeros, 8 slots to a tile, a row's
// slots adjacent in one tile (1 / 2 / 4 / 8 of them for up to 8 / 16 / 32 / 64 nonzeros, tiles
// sorted by that class), longer rows over consecutive tiles, those that get a whole workgroup
// first.  Built on the device (0.2 ms at 100k nonzeros, 0.5 ms at 12 M; on the host it took about
// 3 ms per million nonzeros, after copying the column indices over).  Skipped (the kernel then walks the
// CSR arrays) when padding would blow the layout up, which is what a matrix of mostly empty rows
// does, and beyond kRowTileMaxNnz (rows strategy forced on a very large matrix).
constexpr int64_t kRowTilePadFactor = 8;
constexpr int64_t kRowTileMaxNnz = (int64_t)1 << 28;
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

int build_row_tiles(hpspmm_plan* p, const int32_t* d_rowptr, const int32_t* d_col, hipStream_t st);

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
// HPSPMM_ROW_TILES_XCD = 0 in the environment: round robin, for comparisons.
inline bool row_tiles_same_xcd(int kLd, uint32_t ldb) {
  const char* e = std::getenv("HPSPMM_ROW_TILES_XCD");
  return kLd != 0 && ldb % 32 != 0 && (e ? std::atoi(e) != 0 : true);
}

template <int K, int WPB, int kLd, int kSub>
int launch_row_tiles_w(const hpspmm_plan* p, const float* v, const float* B, float* C, hipStream_t st, uint32_t ldb,
                       uint32_t ldc) {
  const bool same_xcd = row_tiles_same_xcd(kLd, ldb);
  const int64_t groups = ceil_div(p->rt_waves, WPB);
  const int64_t blocks = (same_xcd ? ceil_div(groups, hpspmm::kXcds) * hpspmm::kXcds : groups) * row_tile_column_tiles(K, ldc);
  if (blocks > INT32_MAX) return fail(HPSPMM_ERR_INVALID_ARG, "grid too large");
  hipLaunchKernelGGL((hpspmm::spmm_rowtiles_kernel<K, WPB, kLd, kSub>), dim3((unsigned)blocks), dim3(WPB * 64), 0, st,
                     p->rt_waves, p->rt_loop, p->rt_loop_tiles, p->d_ldesc, p->d_tent, readable_values(p, v), B, C,
                     p->d_zrow + 4, ldb, ldc, same_xcd);
  mark_launch(st, "spmm_rowtiles_kernel");
  return HPSPMM_OK;
}

template <int K, int WPB, int kLd, int kSub>
int launch_row_tiles_wg(const hpspmm_plan* p, const float* v, const float* B, float* C, hipStream_t st, uint32_t ldb,
                        uint32_t ldc) {
  const int64_t wave_items = (p->rt_loop - p->rt_wg) + (p->rt_tiles - p->rt_loop_tiles);
  const bool same_xcd = row_tiles_same_xcd(kLd, ldb);
  const int64_t groups = p->rt_wg + ceil_div(wave_items, WPB);
  const int64_t blocks = (same_xcd ? ceil_div(groups, hpspmm::kXcds) * hpspmm::kXcds : groups) * row_tile_column_tiles(K, ldc);
  if (blocks > INT32_MAX) return fail(HPSPMM_ERR_INVALID_ARG, "grid too large");
  hipLaunchKernelGGL((hpspmm::spmm_rowtiles_wg_kernel<K, WPB, kLd, kSub>), dim3((unsigned)blocks), dim3(WPB * 64), 0, st,
                     p->rt_tiles, p->rt_wg, p->rt_loop, p->rt_loop_tiles, p->d_ldesc, p->d_tent,
                     readable_values(p, v), B, C, p->d_zrow + 4, ldb, ldc, same_xcd);
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

// Lanes per entry of the row-tile kernels at a row length of its own: 8 (32 columns at a time), or 4 / 1
// when there are at most 16 / 4 columns, so that a slot works on 2 / 8 of its entries at a time
// (HPSPMM_ROW_TILES_SUB = 0 in the environment: always 8, for comparisons).
inline int row_tile_sub_lanes(int64_t k) {
  const char* e = std::getenv("HPSPMM_ROW_TILES_SUB");
  if (e && std::atoi(e) == 0) return 8;
  return k <= 4 ? 1 : k <= 16 ? 4 : 8;
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
#define HPSPMM_ROWS_ANYK(GP)                                                                                        \
  return odd_k(k) ? launch_rows_anyk_g<GP, true>(rows, k, rp, ci, v, B, C, long_threshold, long_rows, n_long, st)   \
                  : launch_rows_anyk_g<GP, false>(rows, k, rp, ci, v, B, C, long_threshold, long_rows, n_long, st)
  switch (anyk_lanes(k)) {
    case 2: HPSPMM_ROWS_ANYK(2);
    case 4: HPSPMM_ROWS_ANYK(4);
    case 8: HPSPMM_ROWS_ANYK(8);
    case 16: HPSPMM_ROWS_ANYK(16);
    default: HPSPMM_ROWS_ANYK(32);
  }
#undef HPSPMM_ROWS_ANYK
}

template <int GP, bool kOdd>
int launch_segments_anyk_g(const hpspmm_plan* p, const int32_t* rp, const int32_t* ci, const float* v, const float* B,
                           float* C, hipStream_t st) {
  const int tiles = anyk_tiles(p->k);
  const int64_t blocks = ceil_div(ceil_div(p->nseg, 64 / GP), hpspmm::kWavesPerBlock) * tiles;
  if (blocks > INT32_MAX) return fail(HPSPMM_ERR_INVALID_ARG, "grid too large");
  if (p->nnz > 0) {
    hipLaunchKernelGGL((hpspmm::spmm_segments_anyk_kernel<GP, false, kOdd>), dim3((unsigned)blocks), dim3(hpspmm::kBlock), 0, st, rp,
                       ci, v, p->d_nnz_row, B, C, p->d_carry, p->nnz, p->shift, p->nseg, (int)p->k, tiles,
                       aligned16(ci, v, p->d_nnz_row));
    mark_launch(st, "spmm_segments_anyk_kernel");
  }
  const int64_t fix_blocks = ceil_div(ceil_div(p->rows, 64), hpspmm::kWavesPerBlock);
  hipLaunchKernelGGL((hpspmm::spmm_fixup_anyk_kernel<GP, kOdd>), dim3((unsigned)fix_blocks), dim3(hpspmm::kBlock), 0, st,
                     p->rows, rp, (const float*)p->d_carry, C, p->shift, (int)p->k);
  mark_launch(st, "spmm_fixup_anyk_kernel");
  return HPSPMM_OK;
}

int launch_segments_anyk(const hpspmm_plan* p, const int32_t* rp, const int32_t* ci, const float* v, const float* B,
                         float* C, hipStream_t st) {
#define HPSPMM_SEGMENTS_ANYK(GP)                                                       \
  return odd_k(p->k) ? launch_segments_anyk_g<GP, true>(p, rp, ci, v, B, C, st)        \
                     : launch_segments_anyk_g<GP, false>(p, rp, ci, v, B, C, st)
  switch (anyk_lanes(p->k)) {
    case 2: HPSPMM_SEGMENTS_ANYK(2);
    case 4: HPSPMM_SEGMENTS_ANYK(4);
    case 8: HPSPMM_SEGMENTS_ANYK(8);
    case 16: HPSPMM_SEGMENTS_ANYK(16);
    default: HPSPMM_SEGMENTS_ANYK(32);
  }
#undef HPSPMM_SEGMENTS_ANYK
}

template <int GP, bool kOdd>
int launch_coo_anyk_g(int64_t nnz, int64_t k, const int32_t* ri, const int32_t* ci, const float* v, const float* B,
                      float* C, hipStream_t st) {
  constexpr int P = 64 / GP;
  const int tiles = anyk_tiles(k);
  int shift = 4;  // as launch_coo: 16 nonzeros per sub-wave, doubled while that leaves 4096 wavefronts, up to 512
  while (shift < 9 && (nnz >> (shift + 1)) / P >= 4096) ++shift;
  const int64_t nseg = ceil_div(nnz, (int64_t)1 << shift);
  const int64_t blocks = ceil_div(ceil_div(nseg, P), hpspmm::kWavesPerBlock) * tiles;
  if (blocks > INT32_MAX) return fail(HPSPMM_ERR_INVALID_ARG, "grid too large");
  hipLaunchKernelGGL((hpspmm::spmm_segments_anyk_kernel<GP, true, kOdd>), dim3((unsigned)blocks), dim3(hpspmm::kBlock), 0, st,
                     (const int32_t*)nullptr, ci, v, ri, B, C, (float*)nullptr, nnz, shift, nseg, (int)k, tiles,
                     aligned16(ci, v, ri));
  return HPSPMM_OK;
}

int launch_coo_anyk(int64_t nnz, int64_t k, const int32_t* ri, const int32_t* ci, const float* v, const float* B,
                    float* C, hipStream_t st) {
#define HPSPMM_COO_ANYK(GP)                                                        \
  return odd_k(k) ? launch_coo_anyk_g<GP, true>(nnz, k, ri, ci, v, B, C, st)       \
                  : launch_coo_anyk_g<GP, false>(nnz, k, ri, ci, v, B, C, st)
  switch (anyk_lanes(k)) {
    case 2: HPSPMM_COO_ANYK(2);
    case 4: HPSPMM_COO_ANYK(4);
    case 8: HPSPMM_COO_ANYK(8);
    case 16: HPSPMM_COO_ANYK(16);
    default: HPSPMM_COO_ANYK(32);
  }
#undef HPSPMM_COO_ANYK
}

int launch_rows_any(int64_t rows, int64_t cols, int64_t k, const int32_t* rp, const int32_t* ci, const float* v,
                    const float* B, float* C, int32_t long_threshold, const int32_t* long_rows, int64_t n_long,
                    hipStream_t st) {
  if (rows == 0) return HPSPMM_OK;
  switch (k) {
    case 32: return launch_rows<32>(rows, cols, rp, ci, v, B, C, long_threshold, long_rows, n_long, st);
    case 64: return launch_rows<64>(rows, cols, rp, ci, v, B, C, long_threshold, long_rows, n_long, st);
    case 128: return launch_rows<128>(rows, cols, rp, ci, v, B, C, long_threshold, long_rows, n_long, st);
    default: return launch_rows_anyk(rows, k, rp, ci, v, B, C, long_threshold, long_rows, n_long, st);
  }
}

// Rows scanned by one wavefront of the fix-up kernel: 64, or one per sub-wave while that still
// leaves the grid small.
inline int fixup_rows_per_wave(int64_t rows, int k) { return rows <= (1 << 18) ? 64 / (k / 4) : 64; }

template <int K>
int launch_segments(const hpspmm_plan* p, const int32_t* rp, const int32_t* ci, const float* v,
                    const float* B, float* C, hipStream_t st) {
  constexpr int P = 64 / (K / 4);
  const int64_t nblocks = ceil_div(ceil_div(p->nseg, P), hpspmm::kWavesPerBlock);
  const int64_t grid = p->xcd_remap ? ceil_div(nblocks, hpspmm::kXcds) * hpspmm::kXcds : nblocks;
  if (grid > INT32_MAX) return fail(HPSPMM_ERR_INVALID_ARG, "grid too large");
  if (p->nnz > 0) {
    if (p->n_hub > 0) {
      const int64_t threads = p->n_hub * (K / 4);
      hipLaunchKernelGGL(hpspmm::gather_hub_rows_kernel<K>, dim3((unsigned)ceil_div(threads, hpspmm::kBlock)),
                         dim3(hpspmm::kBlock), 0, st, p->n_hub, p->d_hub_ids, B, p->d_bhot);
      mark_launch(st, "gather_hub_rows_kernel");
      hipLaunchKernelGGL((hpspmm::spmm_segments_kernel<K, false, true>), dim3((unsigned)grid), dim3(hpspmm::kBlock),
                         0, st, rp, p->d_hub_col, v, p->d_nnz_row, B, p->d_bhot, C, p->d_carry, p->nnz, p->shift,
                         p->nseg, nblocks, p->xcd_remap, aligned16(p->d_hub_col, v, p->d_nnz_row));
    } else {
      hipLaunchKernelGGL((hpspmm::spmm_segments_kernel<K, false, false>), dim3((unsigned)grid),
                         dim3(hpspmm::kBlock), 0, st, rp, ci, v, p->d_nnz_row, B, (const float*)nullptr, C,
                         p->d_carry, p->nnz, p->shift, p->nseg, nblocks, p->xcd_remap,
                         aligned16(ci, v, p->d_nnz_row));
    }
    mark_launch(st, "spmm_segments_kernel");
  }
  const int rpw = fixup_rows_per_wave(p->rows, K);
  const int64_t fix_blocks = ceil_div(ceil_div(p->rows, rpw), hpspmm::kWavesPerBlock);
  hipLaunchKernelGGL(hpspmm::spmm_fixup_kernel<K>, dim3((unsigned)fix_blocks), dim3(hpspmm::kBlock), 0, st, p->rows,
                     rp, (const int32_t*)nullptr, p->d_carry, C, p->shift, rpw, (uint32_t)K);
  mark_launch(st, "spmm_fixup_kernel");
  return HPSPMM_OK;
}

// LDS of one workgroup of the ordered strategy, staging tiles included: the most that still lets
// three workgroups share a CU's 160 KB (measured on the co-purchase graph, K = 64: 3.14 ms with
// 32 KB for the rows of B, 2.92 ms with 45 KB, 3.39 ms with 46 KB, where only two fit).
constexpr int kOrderedBlockLdsBytes = 52992;

// kLd: B and C are K columns of wider arrays whose rows are `ld` floats apart (one column tile).
template <int K, int kLd = 0>
int launch_ordered(const hpspmm_plan* p, const int32_t* rp, const float* v, const float* B, float* C,
                   hipStream_t st, uint32_t ld = K) {
  const int64_t nblocks = p->owindows;
  const int64_t grid = p->xcd_remap ? ceil_div(nblocks, hpspmm::kXcds) * hpspmm::kXcds : nblocks;
  if (grid > INT32_MAX) return fail(HPSPMM_ERR_INVALID_ARG, "grid too large");
  if (p->nnz > 0) {
    hipLaunchKernelGGL((hpspmm::spmm_ordered_kernel<K, kLd>), dim3((unsigned)grid), dim3(hpspmm::kBlock),
                       (size_t)p->ocap * K * sizeof(float), st, rp, p->d_ostart, p->d_ocol, p->d_osrc, p->d_orow, v,
                       p->d_wcols, p->ocap, B, C, p->d_carry, p->nnz, p->shift, nblocks, p->xcd_remap, ld);
    mark_launch(st, "spmm_ordered_kernel");
  }
  const int rpw = fixup_rows_per_wave(p->rows, K);
  const int64_t fix_blocks = ceil_div(ceil_div(p->rows, rpw), hpspmm::kWavesPerBlock);
  hipLaunchKernelGGL((hpspmm::spmm_fixup_kernel<K, kLd>), dim3((unsigned)fix_blocks), dim3(hpspmm::kBlock), 0, st,
                     p->rows, rp, p->d_ostart, p->d_carry, C, p->shift, rpw, ld);
  mark_launch(st, "spmm_fixup_kernel");
  return HPSPMM_OK;
}

template <int K>
int launch_coo(int64_t nnz, const int32_t* ri, const int32_t* ci, const float* v, const float* B, float* C,
               hipStream_t st) {
  constexpr int P = 64 / (K / 4);
  // 16 nonzeros per sub-wave, and twice that as long as this leaves 4096 wavefronts, up to 512: the
  // one flush per segment end is the better amortised the longer the segment, and every SIMD still
  // has several wavefronts (social graph, K = 32: 2.16 ms at 64 nonzeros, 1.44 ms at 512; K = 128:
  // 8.33 -> 7.06; R-MAT K = 128: 14.3 -> 13.3; the 20k-vertex citation graph stays at 16)
  int shift = 4;
  while (shift < 9 && (nnz >> (shift + 1)) / P >= 4096) ++shift;
  const int64_t nseg = ceil_div(nnz, (int64_t)1 << shift);
  const int64_t nblocks = ceil_div(ceil_div(nseg, P), hpspmm::kWavesPerBlock);
  if (nblocks > INT32_MAX) return fail(HPSPMM_ERR_INVALID_ARG, "grid too large");
  hipLaunchKernelGGL((hpspmm::spmm_segments_kernel<K, true, false>), dim3((unsigned)nblocks), dim3(hpspmm::kBlock),
                     0, st, (const int32_t*)nullptr, ci, v, ri, B, (const float*)nullptr, C, (float*)nullptr, nnz,
                     shift, nseg, nblocks, false, aligned16(ci, v, ri));
  return HPSPMM_OK;
}

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

// Words of scratch the scan below needs for n values.
inline int64_t scan_scratch_words(int64_t n) { return ceil_div(n, hpspmm::kScanTile) + 1; }

// Device exclusive scan of n uint32 values (three passes, tile sums in between) with the caller's
// scratch (scan_scratch_words(n) words): launches only, no allocation, no synchronisation.  d_out may be d_in.
int exclusive_scan_u32(const uint32_t* d_in, uint32_t* d_out, int64_t n, hipStream_t st, uint32_t* d_tiles) {
  const int64_t ntiles = ceil_div(n, hpspmm::kScanTile);
  if (ntiles > INT32_MAX) return fail(HPSPMM_ERR_INVALID_ARG, "scan too large");
  if (ntiles <= 0) return HPSPMM_OK;
  hipLaunchKernelGGL(hpspmm::scan_tile_sums_kernel, dim3((unsigned)ntiles), dim3(hpspmm::kBlock), 0, st, n, d_in,
                     d_tiles);
  hipLaunchKernelGGL(hpspmm::scan_tile_offsets_kernel, dim3(1), dim3(hpspmm::kBlock), 0, st, ntiles, d_tiles);
  hipLaunchKernelGGL(hpspmm::scan_apply_kernel, dim3((unsigned)ntiles), dim3(hpspmm::kBlock), 0, st, n, d_in, d_tiles,
                     d_out);
  return HPSPMM_OK;
}

// The same with scratch of its own; synchronises the stream.
int exclusive_scan_u32(const uint32_t* d_in, uint32_t* d_out, int64_t n, hipStream_t st) {
  const int64_t ntiles = ceil_div(n, hpspmm::kScanTile);
  if (ntiles > INT32_MAX) return fail(HPSPMM_ERR_INVALID_ARG, "scan too large");
  uint32_t* d_tiles = nullptr;
  HPSPMM_HIP(hipMalloc(&d_tiles, (size_t)ntiles * sizeof(uint32_t)));
  hipLaunchKernelGGL(hpspmm::scan_tile_sums_kernel, dim3((unsigned)ntiles), dim3(hpspmm::kBlock), 0, st, n, d_in,
                     d_tiles);
  hipLaunchKernelGGL(hpspmm::scan_tile_offsets_kernel, dim3(1), dim3(hpspmm::kBlock), 0, st, ntiles, d_tiles);
  hipLaunchKernelGGL(hpspmm::scan_apply_kernel, dim3((unsigned)ntiles), dim3(hpspmm::kBlock), 0, st, n, d_in, d_tiles,
                     d_out);
  hipError_t e = hipStreamSynchronize(st);
  (void)hipFree(d_tiles);
  if (e != hipSuccess) return fail(HPSPMM_ERR_HIP, "scan failed: %s", hipGetErrorString(e));
  return HPSPMM_OK;
}

// Frees what it holds when it goes out of scope (temporaries of a plan-construction step).
struct DeviceTemps {
  std::vector<void*> held;
  ~DeviceTemps() {
    for (void* q : held)
      if (q) (void)hipFree(q);
  }
  template <class T>
  int alloc(T** out, size_t count) {
    *out = nullptr;
    void* q = nullptr;
    if (hipMalloc(&q, std::max<size_t>(count, 1) * sizeof(T)) != hipSuccess) {
      (void)hipGetLastError();
      return fail(HPSPMM_ERR_ALLOC, "device allocation of %zu bytes for the plan failed", count * sizeof(T));
    }
    held.push_back(q);
    *out = (T*)q;
    return HPSPMM_OK;
  }
  // One allocation cut into pieces (an allocation costs 50-200 us, a plan step has a dozen temporaries):
  // room(count) for every piece first, then reserve(), then take() in the same order.
  size_t arena_bytes = 0, arena_used = 0;
  char* arena = nullptr;
  template <class T>
  void room(size_t count) { arena_bytes += (std::max<size_t>(count, 1) * sizeof(T) + 255) & ~(size_t)255; }
  int reserve() {
    if (int rc = alloc(&arena, arena_bytes)) return rc;
    arena_used = 0;
    return HPSPMM_OK;
  }
  template <class T>
  T* take(size_t count) {
    T* out = reinterpret_cast<T*>(arena + arena_used);
    arena_used += (std::max<size_t>(count, 1) * sizeof(T) + 255) & ~(size_t)255;
    return out;
  }
};

// Stable LSD radix sort of n (key, value) pairs over the low `bits` bits of the keys.  d_keys[0] /
// d_vals[0] hold the input, [1] are buffers of the same size, d_hist has 256 * tiles + 1 counters,
// d_scan_scratch scan_scratch_words(256 * tiles) words; returns in *result which of the two value
// buffers holds the sorted values.  Launches only.
int radix_sort_pairs(int64_t n, uint32_t* d_keys[2], int32_t* d_vals[2], uint32_t* d_hist, uint32_t* d_scan_scratch,
                     int bits, hipStream_t st, int* result) {
  const int64_t n_tiles = ceil_div(n, hpspmm::kSortTile);
  int cur = 0;
  for (int shift = 0; shift < bits; shift += 8) {
    hipLaunchKernelGGL(hpspmm::sort_count_kernel, dim3((unsigned)n_tiles), dim3(hpspmm::kBlock), 0, st, n, d_keys[cur],
                       shift, n_tiles, d_hist);
    if (int rc = exclusive_scan_u32(d_hist, d_hist, 256 * n_tiles, st, d_scan_scratch)) return rc;
    hipLaunchKernelGGL(hpspmm::sort_scatter_kernel, dim3((unsigned)n_tiles), dim3(hpspmm::kBlock), 0, st, n,
                       d_keys[cur], d_vals[cur], shift, n_tiles, d_hist, d_keys[cur ^ 1], d_vals[cur ^ 1]);
    cur ^= 1;
  }
  *result = cur;
  return HPSPMM_OK;
}

// The rows sorted by group (one radix pass over the group numbers, stable: rows of a group stay in
// row order), the tile ranges from the group sizes, then one thread per record of the layout.
int build_row_tiles(hpspmm_plan* p, const int32_t* d_rowptr, const int32_t* d_col, hipStream_t st) {
  using hpspmm::kSlotsPerTile;
  constexpr int kTile = hpspmm::kRowTile;
  constexpr int kGroups = hpspmm::kRowTileGroups;
  const int64_t rows = p->rows, nnz = p->nnz;
  if (rows <= 0) return HPSPMM_OK;

  DeviceTemps tmp;
  const int64_t n_tiles = ceil_div(rows, hpspmm::kSortTile);
  const size_t scan_words = (size_t)std::max(scan_scratch_words(256 * n_tiles), scan_scratch_words(rows + 1));
  for (int i = 0; i < 2; ++i) {
    tmp.room<uint32_t>((size_t)rows);
    tmp.room<int32_t>((size_t)rows);
  }
  tmp.room<uint32_t>((size_t)(256 * n_tiles + 1));
  tmp.room<uint32_t>(scan_words);
  tmp.room<uint32_t>(kGroups + 2);
  tmp.room<uint32_t>((size_t)rows + 1);
  if (int rc = tmp.reserve()) return rc;
  uint32_t* d_keys[2];
  int32_t* d_ids[2];
  for (int i = 0; i < 2; ++i) {
    d_keys[i] = tmp.take<uint32_t>((size_t)rows);
    d_ids[i] = tmp.take<int32_t>((size_t)rows);
  }
  uint32_t* d_hist = tmp.take<uint32_t>((size_t)(256 * n_tiles + 1));
  uint32_t* d_scan = tmp.take<uint32_t>(scan_words);
  uint32_t* d_count = tmp.take<uint32_t>(kGroups + 2);
  uint32_t* d_long = tmp.take<uint32_t>((size_t)rows + 1);  // tiles of the rows with tiles of their own, then their scan

  HPSPMM_HIP(hipMemsetAsync(d_count, 0, (kGroups + 2) * sizeof(uint32_t), st));
  hipLaunchKernelGGL(hpspmm::rowtile_classify_kernel, dim3((unsigned)ceil_div(rows, hpspmm::kBlock)), dim3(hpspmm::kBlock),
                     0, st, rows, nnz, d_rowptr, d_keys[0], d_ids[0], d_count);
  int sorted = 0;
  if (int rc = radix_sort_pairs(rows, d_keys, d_ids, d_hist, d_scan, 8, st, &sorted)) return rc;
  const int32_t* d_order = d_ids[sorted];
  uint32_t cnt[kGroups + 2];
  HPSPMM_HIP(hipMemcpyAsync(cnt, d_count, sizeof cnt, hipMemcpyDeviceToHost, st));
  HPSPMM_HIP(hipStreamSynchronize(st));
  // an unchecked rowptr (HPSPMM_PLAN_NO_VALIDATE) that is not monotone or runs past nnz: no tiles,
  // the CSR kernel is left to the caller's arrays as they are
  if (cnt[kGroups + 1] != 0) return HPSPMM_OK;

  hpspmm::RowTileLayout lay{};
  lay.count[4] = (int64_t)cnt[0] + cnt[1];
  lay.count[3] = cnt[2];
  lay.count[2] = cnt[3];
  lay.count[1] = cnt[4];
  lay.count[0] = 0;
  for (int g = 5; g < kGroups; ++g) lay.count[0] += cnt[g];
  lay.loop_tiles = cnt[kGroups];
  lay.start[4] = 0;
  lay.start[3] = lay.count[4];
  lay.start[2] = lay.start[3] + lay.count[3];
  lay.start[1] = lay.start[2] + lay.count[2];
  lay.start[0] = lay.start[1] + lay.count[1];
  // tile ranges: long rows, then the classes from 8 slots a row down to 1
  const int64_t t3 = lay.count[3], t2 = ceil_div(lay.count[2], 2), t1 = ceil_div(lay.count[1], 4),
                t0 = ceil_div(lay.count[0], 8);
  lay.first[3] = lay.loop_tiles;
  lay.first[2] = lay.loop_tiles + t3;
  lay.first[1] = lay.loop_tiles + t3 + t2;
  lay.first[0] = lay.loop_tiles + t3 + t2 + t1;
  lay.tiles = lay.loop_tiles + t3 + t2 + t1 + t0;
  const int64_t tiles = lay.tiles;
  if (tiles * kTile > kRowTilePadFactor * nnz + (1 << 20) || tiles >= (1 << 24)) return HPSPMM_OK;  // not worth it

  const int64_t n_loop = lay.count[4];
  const size_t bytes_ent = (size_t)tiles * kTile * sizeof(int2);
  const size_t bytes_loop = (size_t)std::max<int64_t>(n_loop, 1) * sizeof(int2);
  if (hipMalloc(&p->d_tent, bytes_ent) != hipSuccess || hipMalloc(&p->d_ldesc, bytes_loop) != hipSuccess ||
      hipMalloc(&p->d_zrow, 36 * sizeof(float)) != hipSuccess) {
    (void)hipGetLastError();
    return fail(HPSPMM_ERR_ALLOC, "device allocation of %zu bytes for the row tiles failed", bytes_ent + bytes_loop);
  }
  p->workspace_bytes += (int64_t)(bytes_ent + bytes_loop + 36 * sizeof(float));
  if (n_loop > 0) {
    hipLaunchKernelGGL(hpspmm::rowtile_long_tiles_kernel, dim3((unsigned)ceil_div(n_loop + 1, hpspmm::kBlock)),
                       dim3(hpspmm::kBlock), 0, st, n_loop, d_order, d_rowptr, d_long);
    if (int rc = exclusive_scan_u32(d_long, d_long, n_loop + 1, st, d_scan)) return rc;
    hipLaunchKernelGGL(hpspmm::rowtile_ldesc_kernel, dim3((unsigned)ceil_div(n_loop, hpspmm::kBlock)), dim3(hpspmm::kBlock),
                       0, st, n_loop, d_long, p->d_ldesc);
  }
  if (tiles > 0)
    hipLaunchKernelGGL(hpspmm::rowtile_fill_kernel, dim3((unsigned)ceil_div(tiles * kTile, hpspmm::kBlock)),
                       dim3(hpspmm::kBlock), 0, st, lay, d_order, p->d_ldesc, d_rowptr, d_col, p->d_tent);
  HPSPMM_HIP(hipMemsetAsync(p->d_zrow, 0, 36 * sizeof(float), st));
  hipError_t e = hipStreamSynchronize(st);  // the temporaries go out of scope
  if (e == hipSuccess) e = hipGetLastError();
  if (e != hipSuccess) return fail(HPSPMM_ERR_HIP, "row tiles: %s", hipGetErrorString(e));
  p->rt_tiles = (int32_t)tiles;
  p->rt_loop = (int32_t)n_loop;
  p->rt_wg = (int32_t)cnt[0];
  p->rt_loop_tiles = (int32_t)lay.loop_tiles;
  p->rt_waves = (int32_t)(n_loop + (tiles - lay.loop_tiles));
  return HPSPMM_OK;
}

// Column popularity, on the device: d_count[c] = nonzeros in column c, and d_ids = the `want` most
// referenced columns in order of decreasing count (ties by lower index, so the choice is
// reproducible); columns referenced fewer than twice are dropped.  One object per plan construction:
// the routed and the hub-cache decisions share the histogram, and the ranking too when they ask for
// the same `want`.
struct ColumnRanking {
  int32_t* d_count = nullptr;  // [cols] occurrences among the sampled nonzeros
  int32_t* d_ids = nullptr;    // [n_ids]
  int64_t stride = 1;          // every stride-th nonzero was counted
  int64_t sampled = 0;         // how many that is
  int64_t want = 0, n_ids = 0, served = 0;  // served = nonzeros in the ranked columns (sample count x stride)
  ~ColumnRanking() {
    if (d_count) (void)hipFree(d_count);
    if (d_ids) (void)hipFree(d_ids);
  }
};


// Histogram of every `stride`-th column index into a fresh d_count_out (caller frees).
int count_columns(const hpspmm_plan* p, const int32_t* d_col, int64_t stride, hipStream_t st, int32_t** d_count_out) {
  int32_t* d_count = nullptr;
  HPSPMM_HIP(hipMalloc(&d_count, (size_t)std::max<int64_t>(1, p->cols) * sizeof(int32_t)));
  hipError_t e = hipMemsetAsync(d_count, 0, (size_t)std::max<int64_t>(1, p->cols) * sizeof(int32_t), st);
  if (e != hipSuccess) {
    (void)hipFree(d_count);
    return fail(HPSPMM_ERR_HIP, "hipMemsetAsync: %s", hipGetErrorString(e));
  }
  const int64_t chunks = ceil_div(ceil_div(p->nnz, stride), hpspmm::kCountChunk);
  if (chunks > 0)
    hipLaunchKernelGGL(hpspmm::count_columns_strided_kernel, dim3((unsigned)chunks), dim3(hpspmm::kBlock), 0, st,
                       p->nnz, stride, d_col, d_count);
  *d_count_out = d_count;
  return HPSPMM_OK;
}

// The `want` largest of the n counters at d_count (ties at the threshold by lower index, counters
// below 2 never): *d_keys_out = their keys (~count << 32 | index) in index order (caller frees),
// *m_out how many.
int select_top_columns(const int32_t* d_count, int64_t n, int64_t want, hipStream_t st,
                       unsigned long long** d_keys_out, int64_t* m_out) {
  *d_keys_out = nullptr;
  *m_out = 0;
  want = std::min(want, n);
  if (want <= 0 || n <= 0) return HPSPMM_OK;
  uint32_t *d_hist = nullptr, *d_above = nullptr, *d_equal = nullptr;
  struct Guard {
    void** q[3];
    ~Guard() {
      for (void** x : q)
        if (*x) (void)hipFree(*x);
    }
  } guard{{(void**)&d_hist, (void**)&d_above, (void**)&d_equal}};
  HPSPMM_HIP(hipMalloc(&d_hist, 256 * sizeof(uint32_t)));
  // radix select of the want-th largest counter, most significant byte first
  uint32_t prefix = 0;
  int64_t remaining = want;  // how many of the counters matching the prefix so far are wanted
  for (int shift = 24; shift >= 0; shift -= 8) {
    uint32_t hist[256];
    HPSPMM_HIP(hipMemsetAsync(d_hist, 0, sizeof hist, st));
    hipLaunchKernelGGL(hpspmm::select_histogram_kernel, dim3(grid_for(n, 2048)), dim3(hpspmm::kBlock), 0, st, n,
                       d_count, prefix, shift, d_hist);
    HPSPMM_HIP(hipMemcpyAsync(hist, d_hist, sizeof hist, hipMemcpyDeviceToHost, st));
    HPSPMM_HIP(hipStreamSynchronize(st));
    int b = 255;
    for (; b > 0 && remaining > (int64_t)hist[b]; --b) remaining -= hist[b];
    prefix |= (uint32_t)b << shift;
  }
  // counters above max(threshold, 1), then as many at the threshold as are still wanted
  const int32_t found = (int32_t)prefix;
  const int32_t threshold = found < 2 ? 1 : found;
  HPSPMM_HIP(hipMalloc(&d_above, (size_t)(n + 1) * sizeof(uint32_t)));
  HPSPMM_HIP(hipMalloc(&d_equal, (size_t)(n + 1) * sizeof(uint32_t)));
  hipLaunchKernelGGL(hpspmm::select_flags_kernel, dim3((unsigned)ceil_div(n + 1, hpspmm::kBlock)),
                     dim3(hpspmm::kBlock), 0, st, n, d_count, threshold, d_above, d_equal);
  if (int rc = exclusive_scan_u32(d_above, d_above, n + 1, st)) return rc;
  if (int rc = exclusive_scan_u32(d_equal, d_equal, n + 1, st)) return rc;
  uint32_t n_above = 0, n_equal = 0;
  HPSPMM_HIP(hipMemcpyAsync(&n_above, d_above + n, sizeof n_above, hipMemcpyDeviceToHost, st));
  HPSPMM_HIP(hipMemcpyAsync(&n_equal, d_equal + n, sizeof n_equal, hipMemcpyDeviceToHost, st));
  HPSPMM_HIP(hipStreamSynchronize(st));
  const int64_t ties = found < 2 ? 0 : std::min<int64_t>(n_equal, want - (int64_t)n_above);
  const int64_t m = (int64_t)n_above + std::max<int64_t>(ties, 0);
  if (m <= 0) return HPSPMM_OK;
  unsigned long long* d_keys = nullptr;
  HPSPMM_HIP(hipMalloc(&d_keys, (size_t)m * sizeof(unsigned long long)));
  hipLaunchKernelGGL(hpspmm::select_compact_kernel, dim3((unsigned)ceil_div(n, hpspmm::kBlock)), dim3(hpspmm::kBlock), 0,
                     st, n, d_count, threshold, d_above, d_equal, n_above, (uint32_t)std::max<int64_t>(ties, 0), d_keys);
  hipError_t e = hipStreamSynchronize(st);  // the scans go out of scope
  if (e != hipSuccess) {
    (void)hipFree(d_keys);
    return fail(HPSPMM_ERR_HIP, "column selection failed: %s", hipGetErrorString(e));
  }
  *d_keys_out = d_keys;
  *m_out = m;
  return HPSPMM_OK;
}

int rank_columns(const hpspmm_plan* p, const int32_t* d_col, int64_t want, hipStream_t st, ColumnRanking& rk) {
  if (rk.d_ids && rk.want == want) return HPSPMM_OK;
  if (rk.d_ids) {
    (void)hipFree(rk.d_ids);
    rk.d_ids = nullptr;
  }
  rk.want = want;
  rk.n_ids = 0;
  rk.served = 0;
  if (!rk.d_count) {
    // A large matrix is ranked from a sample of its nonzeros: which columns are hot, and roughly how
    // hot, shows in every 4th nonzero as well as in all of them, and the histogram is the most
    // expensive step of the plan (random read-modify-writes: 12 ms for the 128 M nonzeros of R-MAT
    // scale 22).  Strided, hence the same sample every time.
    rk.stride = p->nnz >= ((int64_t)1 << 26) ? 8 : p->nnz >= ((int64_t)1 << 25) ? 4 : p->nnz >= ((int64_t)1 << 23) ? 2 : 1;
    rk.sampled = ceil_div(p->nnz, rk.stride);
    if (int rc = count_columns(p, d_col, rk.stride, st, &rk.d_count)) return rc;
  }
  unsigned long long* d_keys = nullptr;
  int64_t m = 0;
  if (int rc = select_top_columns(rk.d_count, p->cols, want, st, &d_keys, &m)) return rc;
  struct Guard {
    unsigned long long* q;
    ~Guard() {
      if (q) (void)hipFree(q);
    }
  } guard{d_keys};
  HPSPMM_HIP(hipMalloc(&rk.d_ids, (size_t)std::max<int64_t>(1, m) * sizeof(int32_t)));
  if (m == 0) return HPSPMM_OK;
  unsigned long long served = 0;
  {
    // The keys arrive in column order within "above the threshold" and then "at the threshold": a
    // stable sort by inverted count alone leaves ties in column order, as a sort of the whole keys would.
    DeviceTemps tmp;
    const int64_t n_tiles = ceil_div(m, hpspmm::kSortTile);
    for (int i = 0; i < 2; ++i) {
      tmp.room<uint32_t>((size_t)m);
      tmp.room<int32_t>((size_t)m);
    }
    tmp.room<uint32_t>((size_t)(256 * n_tiles + 1));
    tmp.room<uint32_t>((size_t)scan_scratch_words(256 * n_tiles));
    tmp.room<unsigned long long>(1);
    if (int rc = tmp.reserve()) return rc;
    uint32_t* d_sort_keys[2];
    int32_t* d_sort_ids[2];
    for (int i = 0; i < 2; ++i) {
      d_sort_keys[i] = tmp.take<uint32_t>((size_t)m);
      d_sort_ids[i] = tmp.take<int32_t>((size_t)m);
    }
    uint32_t* d_hist = tmp.take<uint32_t>((size_t)(256 * n_tiles + 1));
    uint32_t* d_scan = tmp.take<uint32_t>((size_t)scan_scratch_words(256 * n_tiles));
    unsigned long long* d_served = tmp.take<unsigned long long>(1);
    HPSPMM_HIP(hipMemsetAsync(d_served, 0, sizeof(unsigned long long), st));
    hipLaunchKernelGGL(hpspmm::rank_split_kernel, dim3((unsigned)ceil_div(m, hpspmm::kBlock)), dim3(hpspmm::kBlock), 0, st,
                       (int32_t)m, d_keys, d_sort_keys[0], d_sort_ids[0], d_served);
    int sorted = 0;
    if (int rc = radix_sort_pairs(m, d_sort_keys, d_sort_ids, d_hist, d_scan, 32, st, &sorted)) return rc;
    HPSPMM_HIP(hipMemcpyAsync(rk.d_ids, d_sort_ids[sorted], (size_t)m * sizeof(int32_t), hipMemcpyDeviceToDevice, st));
    HPSPMM_HIP(hipMemcpyAsync(&served, d_served, sizeof served, hipMemcpyDeviceToHost, st));
    hipError_t e = hipStreamSynchronize(st);
    if (e == hipSuccess) e = hipGetLastError();
    if (e != hipSuccess) return fail(HPSPMM_ERR_HIP, "column ranking failed: %s", hipGetErrorString(e));
  }
  rk.n_ids = m;
  rk.served = (int64_t)served * rk.stride;
  return HPSPMM_OK;
}

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
// Phases: a slice of B larger than this is worked through in two phases, which halves the
// set of hot rows an L2 has to hold at a time.  Every phase adds a partial-result row per
// routed row, and more than two never paid: 233k-vertex social graph, K = 128 (15 MB a
// slice) 4.11 / 4.01 / 4.34 ms with 1 / 2 / 3 phases, K = 64 (7.5 MB a slice) 2.14 / 2.28 /
// 2.51 ms; R-MAT scale 22, K = 128 (268 MB a slice) 6.63 / 6.23 / 6.32 ms.
constexpr int64_t kRoutedPhaseBytes = (int64_t)8 << 20;

// p->d_nnz_row = the row of every nonzero, built the first time a step of the construction needs it
// (the segments kernels, the sortedness check, the routed and sweep layouts do; a plan that ends up
// with the ordered strategy or with row tiles never does).
int ensure_row_expansion(hpspmm_plan* p, const int32_t* d_rowptr, hipStream_t st) {
  if (p->d_nnz_row) return HPSPMM_OK;
  const size_t row_bytes = (size_t)std::max<int64_t>(p->nnz, 1) * sizeof(int32_t);
  if (hipMalloc(&p->d_nnz_row, row_bytes) != hipSuccess) {
    (void)hipGetLastError();
    p->d_nnz_row = nullptr;
    return fail(HPSPMM_ERR_ALLOC, "device allocation of %zu bytes for the plan failed", row_bytes);
  }
  p->workspace_bytes += (int64_t)row_bytes;
  if (p->nnz > 0)
    hipLaunchKernelGGL(hpspmm::expand_rows_kernel, dim3((unsigned)ceil_div(p->nnz, hpspmm::kExpandPerBlock)),
                       dim3(hpspmm::kBlock), 0, st, p->rows, p->nnz, d_rowptr, p->d_nnz_row);
  HPSPMM_HIP(hipGetLastError());
  return HPSPMM_OK;
}

// True if the column indices of every row are in non-decreasing order.  Errors count as "no".
bool columns_sorted(hpspmm_plan* p, const int32_t* d_rowptr, const int32_t* d_col, hipStream_t st) {
  if (ensure_row_expansion(p, d_rowptr, st) != HPSPMM_OK) return false;
  int32_t* d_flag = nullptr;
  if (hipMalloc(&d_flag, sizeof(int32_t)) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  int32_t unsorted = 1;
  hipError_t e = hipMemsetAsync(d_flag, 0, sizeof(int32_t), st);
  if (e == hipSuccess) {
    hipLaunchKernelGGL(hpspmm::columns_unsorted_kernel, dim3(grid_for(p->nnz, 1 << 16)), dim3(hpspmm::kBlock), 0, st,
                       p->nnz, p->d_nnz_row, d_col, d_flag);
    e = hipMemcpyAsync(&unsorted, d_flag, sizeof(int32_t), hipMemcpyDeviceToHost, st);
  }
  if (e == hipSuccess) e = hipStreamSynchronize(st);
  (void)hipFree(d_flag);
  return e == hipSuccess && unsorted == 0;
}

// Builds the routed layout.  Returns HPSPMM_OK with p->strategy left at
// SEGMENTS when the graph does not qualify (and `forced` is false).
int build_routed(hpspmm_plan* p, const int32_t* d_rowptr, const int32_t* d_col, bool forced, int log2_hubs,
                 int log2_row_threshold, int want_sub, bool sort_values, ColumnRanking& rk, hipStream_t st) {
  const int64_t rows = p->rows, nnz = p->nnz, k = p->k;
  if (!forced && (nnz < kRoutedMinNnz || p->cols * k * 4 < kRoutedMinBBytes)) return HPSPMM_OK;
  const int64_t nonempty = std::max<int64_t>(1, rows - p->empty_rows);
  if (!forced && (double)nnz / (double)nonempty < kRoutedMinRowNnz) return HPSPMM_OK;
  if (nnz > INT32_MAX - ((int64_t)1 << 24)) return HPSPMM_OK;  // virtual indices stay int32
  // cached rows per class
  const int64_t h =
      std::max<int64_t>(1, ((int64_t)1 << (log2_hubs ? log2_hubs : kRoutedLog2Cached)) / hpspmm::kSlices);
  if (int rc = rank_columns(p, d_col, h * hpspmm::kSlices, st, rk)) return rc;
  if (!forced && (double)rk.served < kRoutedMinShare * (double)nnz) return HPSPMM_OK;
  const int32_t n_ids = (int32_t)rk.n_ids;

  const int64_t slice_bytes = p->cols * k * 4 / hpspmm::kSlices;
  int nsub = slice_bytes > kRoutedPhaseBytes ? 2 : 1;
  if (want_sub) nsub = std::min(want_sub, hpspmm::kMaxSub);

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
  if (!sort_values && nsub == 1 && nnz > 0 && p->cols * p->k_full * 4 < ((int64_t)1 << 32) &&
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
  if (!forced && (double)origin[nhub] < kRoutedMinRoutedShare * (double)nnz) return HPSPMM_OK;

  hpspmm::RoutedLayout& lay = p->lay;
  lay = hpspmm::RoutedLayout{};
  lay.rows = rows;
  lay.n_routed = n_routed;
  lay.shift = p->shift;
  lay.nsub = nsub;
  lay.nhub = nhub;
  const int64_t subwaves = 64 / (k / 4);
  const int64_t quantum = ((int64_t)1 << p->shift) * subwaves * hpspmm::kWavesPerBlock;  // nonzeros per workgroup
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
  const size_t total_bytes = rvptr_bytes + coldptr_bytes + 3 * v_bytes +
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
  const unsigned cgrid = (unsigned)ceil_div(rows, hpspmm::kBlock);
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
  (void)hipFree(p->d_nnz_row);  // the row of every nonzero served the fill; the class-major arrays replace it
  p->d_nnz_row = nullptr;
  p->n_bhot = inplace ? 0 : n_bhot;
  p->n_hub = inplace ? 0 : (int64_t)n_ids;
  p->nseg = nseg;
  p->strategy = HPSPMM_STRATEGY_ROUTED;
  return HPSPMM_OK;
}

// kLd: B and C are K columns of wider arrays whose rows are `ld` floats apart (one column tile);
// values_ready: an earlier tile of the same product has already brought the values into the plan's order.
template <int K, int kLd = 0>
int launch_routed(const hpspmm_plan* p, const float* v, const float* B, float* C, hipStream_t st, uint32_t ld = K,
                  bool values_ready = false) {
  // values bound to the plan are already in class-major order: only the hub rows of B are refreshed
  const bool bound = p->bound_val && p->bound_val == v;
  const bool inplace = p->d_vsrc && !(bound && p->d_vval);
  const int64_t permute_nnz = (p->d_vsrc || bound || values_ready) ? 0 : p->nnz;
  const int64_t gather_blocks = ceil_div(p->n_bhot * (K / 4), hpspmm::kBlock);
  const int64_t prep_blocks = gather_blocks + ceil_div(permute_nnz, hpspmm::kPermChunk);
  if (prep_blocks > INT32_MAX) return fail(HPSPMM_ERR_INVALID_ARG, "grid too large");
  if (prep_blocks > 0) {
    hipLaunchKernelGGL((hpspmm::routed_prepare_kernel<K, kLd>), dim3((unsigned)prep_blocks), dim3(hpspmm::kBlock), 0, st,
                       p->n_bhot, gather_blocks, p->d_bhot_src, B, p->d_bhot, p->nnz, p->lay.nhub + 1, v, p->d_lslot,
                       p->d_chunk_base, p->d_chunk_pref, p->d_vval, ld);
    mark_launch(st, "routed_prepare_kernel");
  }
  if (p->routed_grid > 0) {
    // One launch; with HPSPMM_ROUTED_SPLIT_LAUNCH=1 (diagnostics: per-class times and counters) one per
    // phase of the hub classes and one for the cold class, each from its first workgroup on.
    const char* split_env = std::getenv("HPSPMM_ROUTED_SPLIT_LAUNCH");
    const bool split = split_env && split_env[0] == '1';
    const int parts = split ? p->lay.nsub + 1 : 1;
    for (int part = 0; part < parts; ++part) {
      const int64_t first = split ? p->lay.phase_begin[part] : 0;
      const int64_t last = split ? (part < p->lay.nsub ? p->lay.phase_begin[part + 1] : p->routed_grid) : p->routed_grid;
      if (last <= first) continue;
      const dim3 grid((unsigned)(last - first));
      if (inplace)
        hipLaunchKernelGGL((hpspmm::spmm_routed_kernel<K, true, false, kLd>), grid, dim3(hpspmm::kBlock), 0, st, p->lay,
                           p->d_rvptr, p->d_coldptr, p->d_vcol, v, p->d_vsrc, p->d_vrow, B, p->d_bhot, p->d_partial,
                           p->d_carry, C, first, ld);
      else if (p->d_vsrc)  // column-range slices, values bound: the plan's own copy of them, still no compact buffer
        hipLaunchKernelGGL((hpspmm::spmm_routed_kernel<K, false, false, kLd>), grid, dim3(hpspmm::kBlock), 0, st, p->lay,
                           p->d_rvptr, p->d_coldptr, p->d_vcol, p->d_vval, (const int32_t*)nullptr, p->d_vrow, B,
                           p->d_bhot, p->d_partial, p->d_carry, C, first, ld);
      else
        hipLaunchKernelGGL((hpspmm::spmm_routed_kernel<K, false, true, kLd>), grid, dim3(hpspmm::kBlock), 0, st, p->lay,
                           p->d_rvptr, p->d_coldptr, p->d_vcol, p->d_vval, (const int32_t*)nullptr, p->d_vrow, B,
                           p->d_bhot, p->d_partial, p->d_carry, C, first, ld);
      mark_launch(st, !split ? "spmm_routed_kernel" : part < p->lay.nsub ? "spmm_routed_kernel(hub phase)"
                                                                          : "spmm_routed_kernel(cold class)");
    }
  }
  const int64_t routed_blocks = row_blocks(p->lay.n_routed, K);
  const int64_t cross_blocks = row_blocks(p->n_cross, K);
  const int64_t fin_blocks = routed_blocks + cross_blocks + row_blocks(p->n_zero, K);
  if (fin_blocks > 0) {
    hipLaunchKernelGGL((hpspmm::spmm_routed_final_kernel<K, kLd>), dim3((unsigned)fin_blocks), dim3(hpspmm::kBlock), 0, st,
                       p->lay, p->d_rvptr, p->d_coldptr, p->d_routed_rows, routed_blocks, p->d_cross_rows, p->n_cross,
                       cross_blocks, p->d_zero_rows, p->n_zero, p->d_partial, p->d_carry, C, ld);
    mark_launch(st, "spmm_routed_final_kernel");
  }
  return HPSPMM_OK;
}

// Builds the ordered layout for the processing order d_order (a permutation of
// the row numbers, in device memory).  p->shift is chosen here.
// With min_served > 0 the layout is kept only if at least that share of the nonzeros reads B from
// LDS; otherwise everything built here is freed again and the plan is left as it was.
int build_ordered(hpspmm_plan* p, const int32_t* d_rowptr, const int32_t* d_col, const int32_t* d_order,
                  double min_served, hipStream_t st) {
  const int64_t rows = p->rows, nnz = p->nnz, k = p->k;
  const int64_t subwaves = 64 / (k / 4);
  // window = one workgroup's segments, at most kOrderedMaxWindow nonzeros
  int shift = 9;
  while (((int64_t)hpspmm::kWavesPerBlock * subwaves << shift) > hpspmm::kOrderedMaxWindow) --shift;
  const int window = (int)((int64_t)hpspmm::kWavesPerBlock * subwaves << shift);
  const int64_t staging_bytes = 3 * hpspmm::kWavesPerBlock * subwaves * hpspmm::kTileStride * 4;
  const int cap = (int)((kOrderedBlockLdsBytes - staging_bytes) / (k * 4));
  const int64_t windows = ceil_div(nnz, window);
  const int64_t nseg = ceil_div(nnz, (int64_t)1 << shift);

  uint32_t* d_len = nullptr;   // [rows + 1] row lengths in processing order, then their scan
  int32_t* d_seen = nullptr;   // [rows] + [1]: permutation check
  unsigned long long* d_served = nullptr;
  struct Guard {
    void** q[3];
    ~Guard() {
      for (void** x : q)
        if (*x) (void)hipFree(*x);
    }
  } guard{{(void**)&d_len, (void**)&d_seen, (void**)&d_served}};
  HPSPMM_HIP(hipMalloc(&d_len, (size_t)(rows + 1) * sizeof(uint32_t)));
  HPSPMM_HIP(hipMalloc(&d_seen, (size_t)(rows + 1) * sizeof(int32_t)));
  HPSPMM_HIP(hipMalloc(&d_served, sizeof(unsigned long long)));
  HPSPMM_HIP(hipMemsetAsync(d_seen, 0, (size_t)(rows + 1) * sizeof(int32_t), st));
  HPSPMM_HIP(hipMemsetAsync(d_served, 0, sizeof(unsigned long long), st));
  const unsigned rgrid = (unsigned)ceil_div(rows + 1, hpspmm::kBlock);
  hipLaunchKernelGGL(hpspmm::ordered_mark_kernel, dim3(rgrid), dim3(hpspmm::kBlock), 0, st, rows, d_order, d_seen,
                     d_seen + rows);
  int32_t bad = 0;
  HPSPMM_HIP(hipMemcpyAsync(&bad, d_seen + rows, sizeof bad, hipMemcpyDeviceToHost, st));
  HPSPMM_HIP(hipStreamSynchronize(st));
  if (bad) return fail(HPSPMM_ERR_INVALID_ARG, "row order is not a permutation of [0, rows)");
  hipLaunchKernelGGL(hpspmm::ordered_len_kernel, dim3(rgrid), dim3(hpspmm::kBlock), 0, st, rows, d_rowptr, d_order,
                     d_len);
  if (int rc = exclusive_scan_u32(d_len, d_len, rows + 1, st)) return rc;

  const size_t n_bytes = (size_t)std::max<int64_t>(nnz, 1) * sizeof(int32_t);
  const size_t start_bytes = (size_t)std::max<int64_t>(rows, 1) * sizeof(int32_t);
  const size_t wcols_bytes = (size_t)std::max<int64_t>(windows, 1) * (size_t)cap * sizeof(int32_t);
  const size_t carry_bytes = (size_t)std::max<int64_t>(nseg, 1) * 2 * (size_t)k * sizeof(float);
  float* d_new_carry = nullptr;
  auto drop = [&]() {
    for (void** q : {(void**)&p->d_ostart, (void**)&p->d_ocol, (void**)&p->d_osrc, (void**)&p->d_orow,
                     (void**)&p->d_wcols, (void**)&d_new_carry}) {
      if (*q) (void)hipFree(*q);
      *q = nullptr;
    }
  };
  if (hipMalloc(&p->d_ostart, start_bytes) != hipSuccess || hipMalloc(&p->d_ocol, n_bytes) != hipSuccess ||
      hipMalloc(&p->d_osrc, n_bytes) != hipSuccess || hipMalloc(&p->d_orow, n_bytes) != hipSuccess ||
      hipMalloc(&p->d_wcols, wcols_bytes) != hipSuccess || hipMalloc(&d_new_carry, carry_bytes) != hipSuccess) {
    (void)hipGetLastError();
    drop();
    return fail(HPSPMM_ERR_ALLOC, "device allocation for the ordered plan failed");
  }
  hipLaunchKernelGGL(hpspmm::ordered_fill_kernel, dim3((unsigned)ceil_div(rows, hpspmm::kWavesPerBlock)),
                     dim3(hpspmm::kBlock), 0, st, rows, d_rowptr, d_col, d_order, d_len, p->d_ostart, p->d_ocol,
                     p->d_osrc, p->d_orow);
  if (windows > INT32_MAX) {
    drop();
    return fail(HPSPMM_ERR_INVALID_ARG, "grid too large");
  }
  if (nnz > 0)
    hipLaunchKernelGGL(hpspmm::ordered_hot_kernel, dim3((unsigned)windows), dim3(hpspmm::kBlock), 0, st, nnz, window,
                       cap, p->d_ocol, p->d_wcols, d_served);
  hipLaunchKernelGGL(hpspmm::ordered_partition_kernel, dim3((unsigned)ceil_div(rows, hpspmm::kWavesPerBlock)),
                     dim3(hpspmm::kBlock), 0, st, rows, d_rowptr, p->d_ostart, window, p->d_ocol, p->d_osrc);
  unsigned long long served = 0;
  hipError_t e = hipMemcpyAsync(&served, d_served, sizeof served, hipMemcpyDeviceToHost, st);
  if (e == hipSuccess) e = hipStreamSynchronize(st);
  if (e == hipSuccess) e = hipGetLastError();
  if (e != hipSuccess) {
    drop();
    return fail(HPSPMM_ERR_HIP, "construction of the ordered plan failed: %s", hipGetErrorString(e));
  }
  if ((double)served < min_served * (double)nnz) {
    drop();
    return HPSPMM_OK;
  }
  // accepted: the segments strategy's buffers are not needed any more
  if (p->d_nnz_row) { (void)hipFree(p->d_nnz_row); p->d_nnz_row = nullptr; }
  if (p->d_carry) (void)hipFree(p->d_carry);
  p->d_carry = d_new_carry;
  p->workspace_bytes = (int64_t)(start_bytes + 3 * n_bytes + wcols_bytes + carry_bytes);
  p->shift = shift;
  p->nseg = nseg;
  p->ocap = cap;
  p->owindows = windows;
  p->oserved = (int64_t)served;
  p->strategy = HPSPMM_STRATEGY_ORDERED;
  return HPSPMM_OK;
}

// Automatic clustering is tried for graphs of at least this size ...
constexpr int64_t kClusterMinNnz = (int64_t)1 << 22;
constexpr int64_t kClusterMinBBytes = (int64_t)24 << 20;
constexpr int32_t kClusterMaxSize = 4096;   // rows of a cluster that still counts as one a window can profit from
constexpr double kClusterMinIntra = 0.15;   // share of the nonzeros inside such clusters for the order to be used
constexpr int64_t kClusterMinMeanNnz = 8;
// ... and its order is kept if this share of the nonzeros then reads B from LDS.
constexpr double kClusterMinServed = 0.15;

// Integer from the environment (diagnostic overrides of the plan's defaults).
int env_int(const char* name, int fallback) {
  const char* v = std::getenv(name);
  return v && *v ? std::atoi(v) : fallback;
}

// Finds a processing order for a square matrix by label propagation on its graph: rows of one
// label next to each other, labels in increasing order, rows of a label in increasing order.
// d_order_out receives a device array of `rows` entries (caller frees).
constexpr int kClusterMaxSweeps = 16;

// *d_order_out = the row numbers sorted by label[row], rows of one label in increasing order (a new
// device array of `rows` entries, caller frees).  Stable radix sort, 8 bits a pass, over as many
// bits as the largest possible label (rows - 1) has.
int sort_rows_by_label(int64_t rows, const int32_t* d_label, hipStream_t st, int32_t** d_order_out) {
  *d_order_out = nullptr;
  const int64_t n_tiles = ceil_div(rows, hpspmm::kSortTile);
  uint32_t *d_keys[2] = {nullptr, nullptr}, *d_hist = nullptr;
  int32_t* d_vals[2] = {nullptr, nullptr};
  struct Guard {
    void** q[5];
    ~Guard() {
      for (void** x : q)
        if (*x) (void)hipFree(*x);
    }
  } guard{{(void**)&d_keys[0], (void**)&d_keys[1], (void**)&d_vals[0], (void**)&d_vals[1], (void**)&d_hist}};
  for (int i = 0; i < 2; ++i) {
    HPSPMM_HIP(hipMalloc(&d_keys[i], (size_t)rows * sizeof(uint32_t)));
    HPSPMM_HIP(hipMalloc(&d_vals[i], (size_t)rows * sizeof(int32_t)));
  }
  HPSPMM_HIP(hipMalloc(&d_hist, (size_t)(256 * n_tiles + 1) * sizeof(uint32_t)));
  hipLaunchKernelGGL(hpspmm::label_pairs_kernel, dim3((unsigned)ceil_div(rows, hpspmm::kBlock)), dim3(hpspmm::kBlock), 0,
                     st, rows, d_label, d_keys[0], d_vals[0]);
  int bits = 1;
  while (bits < 32 && ((int64_t)1 << bits) < rows) ++bits;
  int cur = 0;
  for (int shift = 0; shift < bits; shift += 8) {
    hipLaunchKernelGGL(hpspmm::sort_count_kernel, dim3((unsigned)n_tiles), dim3(hpspmm::kBlock), 0, st, rows,
                       d_keys[cur], shift, n_tiles, d_hist);
    if (int rc = exclusive_scan_u32(d_hist, d_hist, 256 * n_tiles, st)) return rc;
    hipLaunchKernelGGL(hpspmm::sort_scatter_kernel, dim3((unsigned)n_tiles), dim3(hpspmm::kBlock), 0, st, rows,
                       d_keys[cur], d_vals[cur], shift, n_tiles, d_hist, d_keys[cur ^ 1], d_vals[cur ^ 1]);
    cur ^= 1;
  }
  HPSPMM_HIP(hipStreamSynchronize(st));
  HPSPMM_HIP(hipGetLastError());
  *d_order_out = d_vals[cur];
  d_vals[cur] = nullptr;  // handed to the caller
  return HPSPMM_OK;
}

int cluster_rows(const hpspmm_plan* p, const int32_t* d_rowptr, const int32_t* d_col, hipStream_t st,
                 int32_t** d_order_out, double* intra_share_out) {
  const int64_t rows = p->rows;
  *d_order_out = nullptr;
  *intra_share_out = 0.0;
  int32_t* d_label = nullptr;
  int32_t* d_label_next = nullptr;
  uint32_t* d_changed = nullptr;
  struct Guard {
    void** q[3];
    ~Guard() {
      for (void** x : q)
        if (*x) (void)hipFree(*x);
    }
  } guard{{(void**)&d_label, (void**)&d_label_next, (void**)&d_changed}};
  HPSPMM_HIP(hipMalloc(&d_label, (size_t)rows * sizeof(int32_t)));
  HPSPMM_HIP(hipMalloc(&d_label_next, (size_t)rows * sizeof(int32_t)));
  HPSPMM_HIP(hipMalloc(&d_changed, hpspmm::kClusterCounters * sizeof(uint32_t)));
  std::vector<uint32_t> counters((size_t)hpspmm::kClusterCounters);
  hipLaunchKernelGGL(hpspmm::cluster_init_kernel, dim3((unsigned)ceil_div(rows, hpspmm::kBlock)), dim3(hpspmm::kBlock),
                     0, st, rows, d_label);
  const int max_sweeps = std::max(1, env_int("HPSPMM_CLUSTER_SWEEPS", kClusterMaxSweeps));  // diagnostics
  const bool debug = std::getenv("HPSPMM_CLUSTER_DEBUG") != nullptr;
  for (int sweep = 0; sweep < max_sweeps; ++sweep) {
    HPSPMM_HIP(hipMemsetAsync(d_changed, 0, counters.size() * sizeof(uint32_t), st));
    hipLaunchKernelGGL(hpspmm::cluster_sweep_kernel,
                       dim3((unsigned)ceil_div(ceil_div(rows, 2), hpspmm::kWavesPerBlock * 2 * hpspmm::kClusterRowsPerHalf)),
                       dim3(hpspmm::kBlock), 0, st, rows, d_rowptr, d_col, d_label, d_label_next, (uint32_t)sweep,
                       d_changed);
    std::swap(d_label, d_label_next);
    HPSPMM_HIP(hipMemcpyAsync(counters.data(), d_changed, counters.size() * sizeof(uint32_t), hipMemcpyDeviceToHost,
                              st));
    HPSPMM_HIP(hipStreamSynchronize(st));
    int64_t changed = 0;
    for (uint32_t c : counters) changed += c;
    if (debug) fprintf(stderr, "cluster sweep %d: %lld of %lld rows changed their label\n", sweep, (long long)changed, (long long)rows);
    if (changed * 200 < rows) break;
  }
  // share of the nonzeros that stay inside a cluster small enough for a workgroup's window, from
  // every 4th row when there are a million of them (a threshold decision: 1.4 -> 0.4 ms at 2.4 M rows)
  const int64_t score_stride = rows >= ((int64_t)1 << 20) ? 4 : 1;
  {
    int32_t* d_size = nullptr;
    hipError_t e = hipMalloc(&d_size, (size_t)rows * sizeof(int32_t));
    if (e == hipSuccess) e = hipMemsetAsync(d_size, 0, (size_t)rows * sizeof(int32_t), st);
    if (e == hipSuccess) e = hipMemsetAsync(d_changed, 0, counters.size() * sizeof(uint32_t), st);
    if (e == hipSuccess) {
      hipLaunchKernelGGL(hpspmm::label_sizes_kernel, dim3((unsigned)ceil_div(rows, hpspmm::kBlock)), dim3(hpspmm::kBlock),
                         0, st, rows, d_label, d_size);
      hipLaunchKernelGGL(hpspmm::cluster_intra_kernel,
                         dim3((unsigned)ceil_div(ceil_div(rows, score_stride), hpspmm::kWavesPerBlock)),
                         dim3(hpspmm::kBlock), 0, st, rows, score_stride, d_rowptr, d_col, d_label, d_size,
                         kClusterMaxSize, d_changed);
      e = hipMemcpyAsync(counters.data(), d_changed, counters.size() * sizeof(uint32_t), hipMemcpyDeviceToHost, st);
    }
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    if (d_size) (void)hipFree(d_size);
    if (e != hipSuccess) return fail(HPSPMM_ERR_HIP, "cluster scoring failed: %s", hipGetErrorString(e));
    int64_t intra = 0;
    for (uint32_t c : counters) intra += c;
    intra *= score_stride;
    *intra_share_out = p->nnz > 0 ? (double)intra / (double)p->nnz : 0.0;
    if (debug) fprintf(stderr, "cluster: %.4f of the nonzeros inside clusters of at most %d rows\n", *intra_share_out, kClusterMaxSize);
  }
  // rows ordered by label, the rows of a label in increasing order: a stable sort, hence the same
  // order on every run
  int32_t* d_order = nullptr;
  if (int rc = sort_rows_by_label(rows, d_label, st, &d_order)) return rc;
  *d_order_out = d_order;
  return HPSPMM_OK;
}

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

// ---------------------------------------------------------------------------------------------
// Sweep strategy: plan construction and launch.
// ---------------------------------------------------------------------------------------------

constexpr int kSweepMaxBands = 64;
constexpr int32_t kSweepMaxWindows = 8192;
constexpr int32_t kSweepMaxLimit = 32768;  // piece lengths are sorted as 16-bit keys
constexpr int kSweepWindowLog2 = 19;       // bytes of B per window
constexpr int kSweepSpinLimit = 400;
// Windows a wavefront may be ahead of the slowest of its CU.  Social graph, 233k vertices, ms at
// K = 32 / 64 / 128: windows of 512 KB with lead 2: 1.09 / 1.68 / 3.17, lead 3: 1.11 / 1.70 / 2.86;
// 1 MB with lead 2: 1.09 / 1.70 / 2.92, lead 4: 1.12 / 1.71 / 3.07; 256 KB with lead 4: 1.09 / 1.67 / 3.15.
inline int sweep_lead(int64_t k) { return k >= 128 ? 3 : 2; }
// Automatic choice: B beyond what the L2s hold between them without help, enough work to fill the device.
constexpr double kSweepMinSpan = 0.5;  // mean distance from a row's first to its last column, as a share of the columns
constexpr int64_t kSweepMinNnz = (int64_t)1 << 22;
constexpr int64_t kSweepMinBBytes = (int64_t)5 << 20;  // social graph: 6 MB of B, sweep 103 / 127 us against 123 / 141; 3 MB: 90 / 65 against 87 / 63

// Lets the sweep kernels have their LDS; *out = workgroups of them that one CU holds (1 is what the
// layout is made for).
template <int K>
int sweep_prepare_kernels(int* out) {
  const size_t lds = hpspmm::sweep_lds_bytes<K>();
  HPSPMM_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&hpspmm::spmm_sweep_kernel<K, true>),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  HPSPMM_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&hpspmm::spmm_sweep_kernel<K, false>),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  HPSPMM_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&hpspmm::spmm_sweep_kernel<K, true, 1>),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  HPSPMM_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&hpspmm::spmm_sweep_kernel<K, false, 1>),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  HPSPMM_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&hpspmm::spmm_sweep_kernel<K, true, 2>),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  HPSPMM_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&hpspmm::spmm_sweep_kernel<K, false, 2>),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  HPSPMM_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(out, hpspmm::spmm_sweep_kernel<K, true>,
                                                          hpspmm::sweep_waves<K>() * 64, lds));
  return HPSPMM_OK;
}

// Gives back what an abandoned attempt at the sweep layout has allocated in the plan so far.
void drop_sweep_buffers(hpspmm_plan* p) {
  for (void** q : {(void**)&p->d_sw_part_base, (void**)&p->d_sw_base, (void**)&p->d_sw_len, (void**)&p->d_sw_ends,
                   (void**)&p->d_sw_slot_row}) {
    if (*q) (void)hipFree(*q);
    *q = nullptr;
  }
}

// Builds the sweep layout on top of a segments plan.  Returns HPSPMM_OK
// with p->strategy left at SEGMENTS when the matrix does not qualify.  Diagnostics: the environment
// variables HPSPMM_SWEEP_WINDOW_LOG2 (bytes of B per window), HPSPMM_SWEEP_LEAD, HPSPMM_SWEEP_SPIN,
// HPSPMM_SWEEP_LIMIT (nonzeros per piece) and HPSPMM_SWEEP_PRIORITIES override the defaults.
int build_sweep(hpspmm_plan* p, const int32_t* d_rowptr, const int32_t* d_col, bool forced, hipStream_t st) {
  const int64_t rows = p->rows, nnz = p->nnz, k = p->k;
  if (nnz <= 0) return HPSPMM_OK;
  // gather offsets are 32-bit, stream entries keep the column in 24 bits
  if (p->cols * p->k_full * 4 >= ((int64_t)1 << 32) || p->cols > ((int64_t)1 << hpspmm::kSweepColBits)) return HPSPMM_OK;
  if (!forced && (nnz < kSweepMinNnz || p->cols * k * 4 < kSweepMinBBytes)) return HPSPMM_OK;
  const int P = (int)(64 / (k / 4));
  const int WS = P * hpspmm::kSweepSlots;
  const int wpb = k == 32 ? hpspmm::sweep_waves<32>() : k == 64 ? hpspmm::sweep_waves<64>() : hpspmm::sweep_waves<128>();

  // one workgroup fills a CU, and a band fills the device exactly: every CU then runs the same
  // load (a CU with less runs its wavefronts faster, and they leave the others behind)
  int per_cu = 0;
  if (int rc = k == 32 ? sweep_prepare_kernels<32>(&per_cu) : k == 64 ? sweep_prepare_kernels<64>(&per_cu)
                                                                     : sweep_prepare_kernels<128>(&per_cu))
    return rc;
  if (per_cu < 1) return HPSPMM_OK;
  int dev = 0;
  hipDeviceProp_t prop;
  HPSPMM_HIP(hipGetDevice(&dev));
  HPSPMM_HIP(hipGetDeviceProperties(&prop, dev));
  const int64_t band_blocks = prop.multiProcessorCount;
  const int64_t band_waves = band_blocks * wpb;

  // piece limit: a good half of what a sub-wave gets in all, so that the slots of a wavefront even out
  const int64_t nonempty = std::max<int64_t>(1, rows - p->empty_rows);
  const int64_t bands_guess = ceil_div(nonempty + nonempty / 8, band_waves * WS);
  int64_t limit64 = nnz / (bands_guess * band_waves * P) * 6 / 10;
  limit64 = std::max<int64_t>(64, std::min<int64_t>(limit64, kSweepMaxLimit));
  const int32_t limit = std::max(1, std::min<int>(env_int("HPSPMM_SWEEP_LIMIT", (int)limit64), kSweepMaxLimit));

  const int wlog2 = env_int("HPSPMM_SWEEP_WINDOW_LOG2", kSweepWindowLog2);
  int wshift = 0;  // log2 of the columns per window
  while (wshift < 30 && (((int64_t)1 << (wshift + 1)) * k * 4) <= ((int64_t)1 << wlog2)) ++wshift;
  const int64_t n_windows = ceil_div(p->cols, (int64_t)1 << wshift);
  if (n_windows > kSweepMaxWindows) return HPSPMM_OK;
  // every non-empty row is at least one piece: what the two criteria below come to at the very least
  // (rules the layout out for a matrix of many short rows before any kernel has run)
  if (!forced && (ceil_div(nonempty, band_waves * WS) * hpspmm::kXcds * p->cols > nnz / 4 || nonempty * n_windows * 3 > nnz * 2))
    return HPSPMM_OK;
  if (!columns_sorted(p, d_rowptr, d_col, st)) return HPSPMM_OK;  // a row must meet the windows in stored order
  if (!forced) {
    // rows that reach across most of the columns (a banded matrix is better off with whole rows or segments)
    unsigned long long* d_span = nullptr;
    unsigned long long span = 0;
    HPSPMM_HIP(hipMalloc(&d_span, sizeof span));
    hipError_t e = hipMemsetAsync(d_span, 0, sizeof span, st);
    if (e == hipSuccess) {
      hipLaunchKernelGGL(hpspmm::sweep_row_span_kernel, dim3(grid_for(rows, 4096)), dim3(hpspmm::kBlock), 0, st, rows,
                         d_rowptr, d_col, d_span);
      e = hipMemcpyAsync(&span, d_span, sizeof span, hipMemcpyDeviceToHost, st);
    }
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    (void)hipFree(d_span);
    if (e != hipSuccess) return fail(HPSPMM_ERR_HIP, "row span: %s", hipGetErrorString(e));
    if ((double)span < kSweepMinSpan * (double)p->cols * (double)std::max<int64_t>(1, rows - p->empty_rows)) return HPSPMM_OK;
  }

  DeviceTemps tmp;
  // pieces per row, their scans
  uint32_t *d_pbase = nullptr, *d_part = nullptr, *d_scan0 = nullptr;
  if (int rc = tmp.alloc(&d_pbase, (size_t)rows + 1 + (size_t)scan_scratch_words(rows + 1))) return rc;
  d_scan0 = d_pbase + rows + 1;
  if (hipMalloc(&p->d_sw_part_base, (size_t)(rows + 1) * sizeof(uint32_t)) != hipSuccess) {
    (void)hipGetLastError();
    return fail(HPSPMM_ERR_ALLOC, "device allocation for the plan failed");
  }
  d_part = p->d_sw_part_base;
  hipLaunchKernelGGL(hpspmm::sweep_row_pieces_kernel, dim3((unsigned)ceil_div(rows + 1, hpspmm::kBlock)),
                     dim3(hpspmm::kBlock), 0, st, rows, d_rowptr, limit, d_pbase, d_part);
  if (int rc = exclusive_scan_u32(d_pbase, d_pbase, rows + 1, st, d_scan0)) return rc;
  if (int rc = exclusive_scan_u32(d_part, d_part, rows + 1, st, d_scan0)) return rc;
  uint32_t n_pieces = 0, n_parts = 0;
  HPSPMM_HIP(hipMemcpyAsync(&n_pieces, d_pbase + rows, sizeof n_pieces, hipMemcpyDeviceToHost, st));
  HPSPMM_HIP(hipMemcpyAsync(&n_parts, d_part + rows, sizeof n_parts, hipMemcpyDeviceToHost, st));
  HPSPMM_HIP(hipStreamSynchronize(st));
  if (n_pieces == 0) {
    drop_sweep_buffers(p);
    return HPSPMM_OK;
  }

  const int64_t n_bands = ceil_div((int64_t)n_pieces, band_waves * WS);
  // every band re-reads B once on every XCD: worth it while that stays well below the gather volume,
  // and while a piece still finds one or two nonzeros in a window (the co-purchase graph at 6 M
  // nonzeros has 0.85 on average and takes 251 us against 134 with the ordered strategy)
  if (n_bands > kSweepMaxBands ||
      (!forced && (n_bands * hpspmm::kXcds * p->cols > nnz / 4 || (int64_t)n_pieces * n_windows * 3 > nnz * 2))) {
    drop_sweep_buffers(p);
    return HPSPMM_OK;
  }
  const int64_t n_waves = n_bands * band_waves;
  const int64_t n_slots = n_waves * WS;

  // the other temporaries, one allocation
  const int64_t n_tiles = ceil_div((int64_t)n_pieces, hpspmm::kSortTile);
  const size_t scan_words = (size_t)std::max(scan_scratch_words(256 * n_tiles), scan_scratch_words(n_waves + 1));
  for (int i = 0; i < 2; ++i) {
    tmp.room<uint32_t>(n_pieces);
    tmp.room<int32_t>(n_pieces);
  }
  tmp.room<uint32_t>((size_t)(256 * n_tiles + 1));
  tmp.room<uint32_t>(scan_words);
  tmp.room<int32_t>(n_pieces);
  tmp.room<int32_t>((size_t)n_slots);
  tmp.room<int32_t>((size_t)rows * (size_t)(n_windows + 1));
  tmp.room<int32_t>((size_t)n_slots * (size_t)n_windows);
  tmp.room<uint32_t>((size_t)n_waves + 1);
  tmp.room<int32_t>(2);
  if (int rc = tmp.reserve()) return rc;
  uint32_t* d_keys[2];
  int32_t* d_vals[2];
  for (int i = 0; i < 2; ++i) {
    d_keys[i] = tmp.take<uint32_t>(n_pieces);
    d_vals[i] = tmp.take<int32_t>(n_pieces);
  }
  uint32_t* d_hist = tmp.take<uint32_t>((size_t)(256 * n_tiles + 1));
  uint32_t* d_scan = tmp.take<uint32_t>(scan_words);
  int32_t* d_piece_row = tmp.take<int32_t>(n_pieces);
  int32_t* d_piece_of = tmp.take<int32_t>((size_t)n_slots);
  int32_t* d_wstart = tmp.take<int32_t>((size_t)rows * (size_t)(n_windows + 1));
  int32_t* d_run_at = tmp.take<int32_t>((size_t)n_slots * (size_t)n_windows);
  uint32_t* d_stream_len = tmp.take<uint32_t>((size_t)n_waves + 1);
  int32_t* d_counts = tmp.take<int32_t>(2);

  // pieces by decreasing length, dealt to the wavefronts
  hipLaunchKernelGGL(hpspmm::sweep_piece_keys_kernel, dim3((unsigned)ceil_div(rows, hpspmm::kBlock)),
                     dim3(hpspmm::kBlock), 0, st, rows, d_rowptr, limit, d_pbase, d_keys[0], d_vals[0], d_piece_row);
  int sorted = 0;
  if (int rc = radix_sort_pairs(n_pieces, d_keys, d_vals, d_hist, d_scan, 16, st, &sorted)) return rc;
  HPSPMM_HIP(hipMemsetAsync(d_piece_of, 0xFF, (size_t)n_slots * sizeof(int32_t), st));
  hipLaunchKernelGGL(hpspmm::sweep_assign_kernel, dim3((unsigned)ceil_div((int64_t)n_pieces, hpspmm::kBlock)),
                     dim3(hpspmm::kBlock), 0, st, (int64_t)n_pieces, d_vals[sorted], (int32_t)n_bands, (int32_t)band_waves,
                     (int32_t)WS, d_piece_of);

  // where every row enters every window
  hipLaunchKernelGGL(hpspmm::sweep_row_windows_kernel, dim3((unsigned)ceil_div(nnz, hpspmm::kBlock)),
                     dim3(hpspmm::kBlock), 0, st, nnz, p->d_nnz_row, d_rowptr, d_col, wshift, (int32_t)n_windows, d_wstart);

  // chunk lengths, stream lengths, stream origins
  if (hipMalloc(&p->d_sw_base, (size_t)(n_waves + 1) * sizeof(uint32_t)) != hipSuccess ||
      hipMalloc(&p->d_sw_len, (size_t)n_waves * sizeof(uint32_t)) != hipSuccess ||
      hipMalloc(&p->d_sw_ends, (size_t)n_waves * (size_t)n_windows * sizeof(int32_t)) != hipSuccess ||
      hipMalloc(&p->d_sw_slot_row, (size_t)n_slots * sizeof(int32_t)) != hipSuccess) {
    (void)hipGetLastError();
    return fail(HPSPMM_ERR_ALLOC, "device allocation for the plan failed");
  }
  const dim3 wave_grid((unsigned)n_waves);
  switch (P) {
    case 8:
      hipLaunchKernelGGL(hpspmm::sweep_chunks_kernel<8>, wave_grid, dim3(hpspmm::kBlock), 0, st, (int32_t)n_windows, limit,
                         d_piece_of, d_piece_row, d_pbase, d_rowptr, d_wstart, d_run_at, p->d_sw_ends, p->d_sw_len);
      break;
    case 4:
      hipLaunchKernelGGL(hpspmm::sweep_chunks_kernel<4>, wave_grid, dim3(hpspmm::kBlock), 0, st, (int32_t)n_windows, limit,
                         d_piece_of, d_piece_row, d_pbase, d_rowptr, d_wstart, d_run_at, p->d_sw_ends, p->d_sw_len);
      break;
    default:
      hipLaunchKernelGGL(hpspmm::sweep_chunks_kernel<2>, wave_grid, dim3(hpspmm::kBlock), 0, st, (int32_t)n_windows, limit,
                         d_piece_of, d_piece_row, d_pbase, d_rowptr, d_wstart, d_run_at, p->d_sw_ends, p->d_sw_len);
      break;
  }
  hipLaunchKernelGGL(hpspmm::sweep_stream_lengths_kernel, dim3((unsigned)ceil_div(n_waves + 1, hpspmm::kBlock)),
                     dim3(hpspmm::kBlock), 0, st, n_waves, P, p->d_sw_len, d_stream_len);
  // the total must stay an int32 position: checked on the 64-bit sum of the lengths before the 32-bit scan
  {
    std::vector<uint32_t> lens((size_t)n_waves);
    HPSPMM_HIP(hipMemcpyAsync(lens.data(), p->d_sw_len, (size_t)n_waves * sizeof(uint32_t), hipMemcpyDeviceToHost, st));
    HPSPMM_HIP(hipStreamSynchronize(st));
    int64_t total = 0;
    uint32_t longest = 0;
    for (uint32_t v : lens) {
      total += (int64_t)v * P;
      longest = std::max(longest, v);
    }
    // (positions within a window's chunk are kept in 28 bits while the streams are laid out)
    if (total >= INT32_MAX - 64 || longest >= (1u << 28)) {
      drop_sweep_buffers(p);
      return HPSPMM_OK;
    }
    p->sw_total = total;
  }
  if (int rc = exclusive_scan_u32(d_stream_len, p->d_sw_base, n_waves + 1, st, d_scan)) return rc;

  // the streams
  const int64_t total = p->sw_total;
  if (hipMalloc(&p->d_vcol, (size_t)std::max<int64_t>(total, 1) * sizeof(int32_t)) != hipSuccess ||
      hipMalloc(&p->d_vsrc, (size_t)std::max<int64_t>(total, 1) * sizeof(int32_t)) != hipSuccess ||
      hipMalloc(&p->d_partial, (size_t)std::max<int64_t>(n_parts, 1) * (size_t)k * sizeof(float)) != hipSuccess ||
      hipMalloc(&p->d_sw_split_rows, (size_t)std::max<int64_t>(n_parts / 2, 1) * sizeof(int32_t)) != hipSuccess ||
      hipMalloc(&p->d_zero_rows, (size_t)std::max<int64_t>(p->empty_rows, 1) * sizeof(int32_t)) != hipSuccess ||
      hipMalloc(&p->d_sw_zrow, 128 * sizeof(float)) != hipSuccess) {
    (void)hipGetLastError();
    return fail(HPSPMM_ERR_ALLOC, "device allocation for the plan failed");
  }
  hipLaunchKernelGGL(hpspmm::sweep_clear_stream_kernel, dim3(grid_for(total, 1 << 16)), dim3(hpspmm::kBlock), 0, st, total,
                     p->d_vcol, p->d_vsrc);
  hipLaunchKernelGGL(hpspmm::sweep_fill_kernel, wave_grid, dim3(hpspmm::kBlock), 0, st, (int32_t)n_windows, wshift, limit,
                     (int32_t)WS, (int32_t)(k / 4), d_piece_of, d_piece_row, d_pbase, d_rowptr, d_col, d_wstart, d_run_at,
                     p->d_sw_ends, p->d_sw_base, p->d_sw_len, p->d_vcol, p->d_vsrc);
  hipLaunchKernelGGL(hpspmm::sweep_slot_rows_kernel, dim3((unsigned)ceil_div(n_slots, hpspmm::kBlock)), dim3(hpspmm::kBlock),
                     0, st, n_slots, d_piece_of, d_piece_row, d_pbase, d_part, d_rowptr, limit, p->d_sw_slot_row);

  // rows cut into pieces, rows without nonzeros
  HPSPMM_HIP(hipMemsetAsync(d_counts, 0, 2 * sizeof(int32_t), st));
  HPSPMM_HIP(hipMemsetAsync(p->d_sw_zrow, 0, 128 * sizeof(float), st));
  const dim3 row_grid((unsigned)ceil_div(rows, hpspmm::kBlock));
  hipLaunchKernelGGL(hpspmm::sweep_collect_rows_kernel, row_grid, dim3(hpspmm::kBlock), 0, st, rows, d_rowptr, limit, 1,
                     p->d_sw_split_rows, d_counts);
  hipLaunchKernelGGL(hpspmm::sweep_collect_rows_kernel, row_grid, dim3(hpspmm::kBlock), 0, st, rows, d_rowptr, limit, 0,
                     p->d_zero_rows, d_counts + 1);
  int32_t counts[2] = {0, 0};
  HPSPMM_HIP(hipMemcpyAsync(counts, d_counts, sizeof counts, hipMemcpyDeviceToHost, st));
  hipError_t e = hipStreamSynchronize(st);
  if (e == hipSuccess) e = hipGetLastError();
  if (e != hipSuccess) return fail(HPSPMM_ERR_HIP, "sweep layout failed: %s", hipGetErrorString(e));
  if (counts[0] < 0 || counts[0] > (int32_t)(n_parts / 2) || counts[1] != p->empty_rows)
    return fail(HPSPMM_ERR_HIP, "sweep layout: inconsistent row lists");
  p->n_split = counts[0];
  p->n_zero = counts[1];
  p->sw_limit = limit;
  p->sw_bands = (int32_t)n_bands;
  p->sw.n_waves = n_waves;
  p->sw.n_windows = (int32_t)n_windows;
  p->sw.lead = std::max(1, env_int("HPSPMM_SWEEP_LEAD", sweep_lead(k)));
  p->sw.spin_limit = std::max(0, env_int("HPSPMM_SWEEP_SPIN", kSweepSpinLimit));
  p->sw.priorities = env_int("HPSPMM_SWEEP_PRIORITIES", 1);
  if (std::getenv("HPSPMM_SWEEP_DEBUG"))
    fprintf(stderr, "sweep plan: bands=%lld waves=%lld windows=%lld limit=%d pieces=%u split_rows=%d nnz=%lld stream=%lld (%.3f)\n",
            (long long)n_bands, (long long)n_waves, (long long)n_windows, limit, n_pieces, counts[0], (long long)nnz,
            (long long)total, (double)total / (double)nnz);
  // the segments plan underneath is no longer needed
  if (p->d_nnz_row) (void)hipFree(p->d_nnz_row);
  if (p->d_carry) (void)hipFree(p->d_carry);
  p->d_nnz_row = nullptr;
  p->d_carry = nullptr;
  p->workspace_bytes = 2 * total * 4 + (int64_t)std::max<int64_t>(n_parts, 1) * k * 4 + (n_waves + 1) * 4 + n_waves * 4 +
                       n_waves * n_windows * 4 + n_slots * 4 + (rows + 1) * 4 + std::max<int64_t>(n_parts / 2, 1) * 4 +
                       std::max<int64_t>(p->empty_rows, 1) * 4 + 512;
  p->nseg = 0;
  p->shift = 0;
  p->strategy = HPSPMM_STRATEGY_SWEEP;
  return HPSPMM_OK;
}

// kLd: B and C are K columns of wider arrays whose rows are `ld` floats apart (one column tile).
template <int K, int kLd = 0>
int launch_sweep(const hpspmm_plan* p, const int32_t* rp, const float* v, const float* B, float* C, hipStream_t st,
                 uint32_t ld = K) {
  const bool bound = p->bound_val && p->bound_val == v && p->d_vval;
  constexpr int wpb = hpspmm::sweep_waves<K>();
  const dim3 grid((unsigned)(p->sw.n_waves / wpb));
  const size_t lds = hpspmm::sweep_lds_bytes<K>();
  if (bound)
    hipLaunchKernelGGL((hpspmm::spmm_sweep_kernel<K, false, kLd>), grid, dim3(wpb * 64), lds, st, p->sw, p->d_sw_base,
                       p->d_sw_len, p->d_sw_ends, p->d_vcol, p->d_vval, (const int32_t*)nullptr, p->d_sw_slot_row, B,
                       p->d_sw_zrow, p->d_partial, C, ld);
  else
    hipLaunchKernelGGL((hpspmm::spmm_sweep_kernel<K, true, kLd>), grid, dim3(wpb * 64), lds, st, p->sw, p->d_sw_base,
                       p->d_sw_len, p->d_sw_ends, p->d_vcol, v, p->d_vsrc, p->d_sw_slot_row, B, p->d_sw_zrow,
                       p->d_partial, C, ld);
  mark_launch(st, "spmm_sweep_kernel");
  const int64_t split_blocks = row_blocks(p->n_split, K);
  const int64_t fin_blocks = split_blocks + row_blocks(p->n_zero, K);
  if (fin_blocks > 0) {
    hipLaunchKernelGGL((hpspmm::spmm_sweep_final_kernel<K, kLd>), dim3((unsigned)fin_blocks), dim3(hpspmm::kBlock), 0, st,
                       rp, p->sw_limit, p->d_sw_split_rows, p->n_split, split_blocks, p->d_sw_part_base, p->d_zero_rows,
                       p->n_zero, p->d_partial, C, ld);
    mark_launch(st, "spmm_sweep_final_kernel");
  }
  return HPSPMM_OK;
}

}  // namespace

extern "C" {

int hpspmm_version(void) { return 100; }

const char* hpspmm_last_error(void) { return g_last_error.c_str(); }

// Column tiles are tried for matrices of at least this many nonzeros (below, whole rows or plain
// segments at the full row length are as good), or when the caller forces one of the layouts.
constexpr int64_t kTiledMinNnz = (int64_t)1 << 22;

// k_full = 0: the plan is for row length k.  Otherwise: a plan of tile width k for B and C of row
// length k_full (see hpspmm_plan::k_full).
static int plan_create_impl(int64_t rows, int64_t cols, int64_t nnz, const int32_t* d_rowptr, const int32_t* d_col,
                            int64_t k, uint32_t flags, const int32_t* d_order, void* stream,
                            hpspmm_plan** plan_out, int64_t k_full = 0) {
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
  // (HPSPMM_NO_COLUMN_TILES in the environment switches this off, for comparisons)
  const int64_t kp = (k + 3) & ~(int64_t)3;
  const int64_t kw = fast_k(kp) ? kp : tile_width(kp);
  if (k_full == 0 && !fast_k(k) && kw > 0 && (k % 4 == 0 || k >= 16) && nnz > 0 &&
      !std::getenv("HPSPMM_NO_COLUMN_TILES") &&
      (nnz >= kTiledMinNnz || d_order ||
       (flags & (HPSPMM_PLAN_FORCE_ROUTED | HPSPMM_PLAN_FORCE_SWEEP | HPSPMM_PLAN_CLUSTER)))) {
    hpspmm_plan* tiled = nullptr;
    int rc = plan_create_impl(rows, cols, nnz, d_rowptr, d_col, kw, flags, d_order, stream, &tiled, kp);
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
  const bool xcd_ok = xcd_dealing_holds(st);
  p->xcd_remap = !(flags & HPSPMM_PLAN_NO_XCD_REMAP) && xcd_ok;

  // Automatic choice, in this order: tiny matrix -> rows; a matrix in the rows strategy's range
  // (`rows_range`) -> ordered if it has communities, else rows; beyond that range -> routed if a
  // few columns take most of the nonzeros, else ordered if it has communities, else segments.
  ColumnRanking ranking;         // column popularity, shared by the routed and the hub-cache decisions
  bool rows_need_tiles = false;  // rows strategy chosen on the strength of the row tiles
  bool rows_range = false;       // provisional segments; rows unless the ordered strategy qualifies
  bool want_row_tiles = true;    // rows strategy: over row tiles if they can be built
  if (!row_tiles_serve(k)) {
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
    const bool mid = in_range && p->max_row_nnz <= longest_ok && !(flags & HPSPMM_PLAN_NO_ROW_TILES);
    if (nnz == 0 || tiny || (mid && nnz < kClusterMinNnz)) {
      p->strategy = HPSPMM_STRATEGY_ROWS;
      rows_need_tiles = !(nnz == 0 || tiny);
      want_row_tiles = mid;
    } else {
      p->strategy = HPSPMM_STRATEGY_SEGMENTS;
      rows_range = mid;
    }
  }

  if (p->strategy == HPSPMM_STRATEGY_ROWS && want_row_tiles && row_tiles_serve(k) && rows > 0 && nnz < kRowTileMaxNnz &&
      !(flags & HPSPMM_PLAN_NO_ROW_TILES)) {
    if (int rc = build_row_tiles(p, d_rowptr, d_col, st)) {
      return rc;
    }
  }
  if (p->strategy == HPSPMM_STRATEGY_ROWS && rows_need_tiles && !p->d_tent) p->strategy = HPSPMM_STRATEGY_SEGMENTS;

  if (p->strategy == HPSPMM_STRATEGY_SEGMENTS) {
    int forced = (int)((flags >> 8) & 0xFu);
    if (forced && (forced < 3 || forced > 15)) {
      return fail(HPSPMM_ERR_INVALID_ARG, "forced segment shift %d outside [3, 15]", forced);
    }
    p->shift = forced ? forced : choose_shift(nnz, k, p->max_row_nnz);
    p->nseg = ceil_div(nnz, (int64_t)1 << p->shift);
    // what the segments kernels need (the row of every nonzero, the carry slots) is allocated at the
    // end, if the plan is still a segments plan then: the layouts tried below mostly replace both
  }
  // Long rows over a B that is small against the gather volume: every wavefront walks B window by
  // window (tried first: where it qualifies it beats the routed strategy - social graph, 233k
  // vertices, K = 32 / 64 / 128: 1.09 / 1.68 / 2.86 ms against 1.11 / 1.92 / 3.72).  When the matrix
  // does not qualify, or cannot be laid out that way (unsorted columns, more than 2^24 columns),
  // the plan stays what it was.
  if (p->strategy == HPSPMM_STRATEGY_SEGMENTS && fast_k(k) && nnz > 0 && !(flags & HPSPMM_PLAN_NO_SWEEP) &&
      ((flags & HPSPMM_PLAN_FORCE_SWEEP) ||
       (!rows_range && !(flags & (HPSPMM_PLAN_FORCE_SEGMENTS | HPSPMM_PLAN_FORCE_ROUTED | HPSPMM_PLAN_CLUSTER))))) {
    if (int rc = build_sweep(p, d_rowptr, d_col, (flags & HPSPMM_PLAN_FORCE_SWEEP) != 0, st)) return rc;
  }
  if (p->strategy == HPSPMM_STRATEGY_SEGMENTS && fast_k(k) && !(flags & HPSPMM_PLAN_NO_ROUTED) && nnz > 0 &&
      !rows_range &&
      (xcd_ok || (flags & HPSPMM_PLAN_FORCE_ROUTED)) &&
      !(flags & HPSPMM_PLAN_FORCE_SEGMENTS && !(flags & HPSPMM_PLAN_FORCE_ROUTED))) {
    if (int rc = build_routed(p, d_rowptr, d_col, (flags & HPSPMM_PLAN_FORCE_ROUTED) != 0,
                              (flags & HPSPMM_PLAN_FORCE_ROUTED) ? (int)((flags >> 16) & 0x1Fu) : 0,
                              (flags & HPSPMM_PLAN_FORCE_ROUTED) ? (int)((flags >> 24) & 0x1Fu) : 0,
                              (flags & HPSPMM_PLAN_FORCE_ROUTED) ? (int)((flags >> 29) & 0x7u) : 0,
                              (flags & HPSPMM_PLAN_ROUTED_SORT_VALUES) != 0, ranking, st)) {
      return rc;
    }
  }
  // Community structure: not routed, the matrix is a graph (square) and B does not fit the L2s -
  // look for clusters of rows that share columns.  Tried before the hub cache: a graph can have
  // both popular columns and communities (the co-purchase graph at a quarter of its size: the 64k
  // most referenced columns take a quarter of the nonzeros there), and the ordered strategy is then
  // the faster of the two (0.73 ms against 1.15 ms for segments with the hub cache).
  const bool want_cluster = (flags & HPSPMM_PLAN_CLUSTER) != 0;
  if (p->strategy == HPSPMM_STRATEGY_SEGMENTS && fast_k(k) && rows == cols && nnz > 0 &&
      !(flags & HPSPMM_PLAN_NO_CLUSTER) &&
      (want_cluster || (!(flags & HPSPMM_PLAN_FORCE_SEGMENTS) && nnz >= kClusterMinNnz &&
                        cols * k * 4 >= kClusterMinBBytes && nnz >= rows * kClusterMinMeanNnz))) {
    int32_t* d_order = nullptr;
    double intra_share = 0.0;
    int rc = cluster_rows(p, d_rowptr, d_col, st, &d_order, &intra_share);
    if (rc == HPSPMM_OK && (want_cluster || intra_share >= kClusterMinIntra))
      rc = build_ordered(p, d_rowptr, d_col, d_order, want_cluster ? 0.0 : kClusterMinServed, st);
    if (d_order) (void)hipFree(d_order);
    if (rc) {
      return rc;
    }
  }
  if (p->strategy == HPSPMM_STRATEGY_SEGMENTS && rows_range && row_tiles_serve(k)) {
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
  if (p->d_tent && !fast_k(k)) {
    // Row tiles at a row length of its own.  The gathers are fastest when every 32-column tile of a
    // row of B is one aligned 128-byte line (R-MAT graph, 3.7 M nonzeros: K = 96 131 us, K = 100
    // 186 us as it lies).  A B whose rows do not even start at multiples of 32 bytes is therefore
    // read through a copy with rows padded to a multiple of 32 floats, refreshed at the start of
    // every SpMM, where that copy is cheap against the gathers - 40 nonzeros for every row of B,
    // 2^20 in all (co-purchase graph, 2.5 M nonzeros, K = 100: 140 -> 118 us, K = 41: 77 -> 66;
    // but K = 200: 267 -> 319, K = 48: 58 -> 64; R-MAT, 28 nonzeros a row, K = 172: 291 -> 342;
    // co-purchase graph at 0.6 M nonzeros, K = 41: 16.5 -> 20.2).  HPSPMM_ROW_TILES_PAD = 0 / 1 in
    // the environment: never / whenever the length is not a multiple of 32, for comparisons.
    // Otherwise the rows stay as they lie; a length that is not a multiple of 4 is then gathered
    // with 16-byte loads at 4-byte alignment - except below 4 columns, where a row is shorter than
    // one such load: the copy then has rows of 4 floats.
    const char* pad_env = std::getenv("HPSPMM_ROW_TILES_PAD");
    const bool pad = k < 4 || (k % 32 != 0 && (pad_env ? std::atoi(pad_env) != 0
                                                       : (k > 32 && k % 8 != 0 && nnz >= 2 * kRowTilePadMinNnz &&
                                                          nnz >= 40 * cols)));
    p->rt_ldb = (uint32_t)(k < 4 ? 4 : pad ? (k + 31) & ~(int64_t)31 : k);
    p->rt_mode = pad ? 2 : k % 4 ? 3 : 1;
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
    if (int rc = build_hub_cache(p, d_col, (int)((flags >> 16) & 0x1Fu), (flags & HPSPMM_PLAN_HUB_CACHE) != 0, ranking, st)) {
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
static int plan_create_guarded(int64_t rows, int64_t cols, int64_t nnz, const int32_t* d_rowptr,
                               const int32_t* d_col, int64_t k, uint32_t flags, const int32_t* d_order, void* stream,
                               hpspmm_plan** plan_out) {
  int rc;
  try {
    rc = plan_create_impl(rows, cols, nnz, d_rowptr, d_col, k, flags, d_order, stream, plan_out);
  } catch (const std::bad_alloc&) {
    if (plan_out) *plan_out = nullptr;
    rc = fail(HPSPMM_ERR_ALLOC, "out of host memory while building the plan");
  } catch (const std::exception& e) {
    if (plan_out) *plan_out = nullptr;
    rc = fail(HPSPMM_ERR_ALLOC, "plan construction failed: %s", e.what());
  }
  return rc;
}

int hpspmm_plan_create(int64_t rows, int64_t cols, int64_t nnz, const int32_t* d_rowptr, const int32_t* d_col,
                       int64_t k, uint32_t flags, void* stream, hpspmm_plan** plan_out) {
  return plan_create_guarded(rows, cols, nnz, d_rowptr, d_col, k, flags, nullptr, stream, plan_out);
}

int hpspmm_plan_create_ordered(int64_t rows, int64_t cols, int64_t nnz, const int32_t* d_rowptr,
                               const int32_t* d_col, int64_t k, uint32_t flags, const int32_t* d_row_order,
                               void* stream, hpspmm_plan** plan_out) {
  if (rows > 0 && !d_row_order) return fail(HPSPMM_ERR_INVALID_ARG, "d_row_order is NULL");
  return plan_create_guarded(rows, cols, nnz, d_rowptr, d_col, k, flags, d_row_order, stream, plan_out);
}

int hpspmm_plan_get_info(const hpspmm_plan* plan, hpspmm_plan_info* out) {
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
  return HPSPMM_OK;
}

int hpspmm_plan_destroy(hpspmm_plan* plan) {
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
                  (void*)plan->d_vval, (void*)plan->d_vsrc, (void*)plan->d_vrow, (void*)plan->d_bhot_src, (void*)plan->d_partial,
                  (void*)plan->d_routed_rows, (void*)plan->d_cross_rows, (void*)plan->d_zero_rows,
                  (void*)plan->d_ostart, (void*)plan->d_ocol, (void*)plan->d_osrc, (void*)plan->d_orow,
                  (void*)plan->d_wcols, (void*)plan->d_tent, (void*)plan->d_ldesc, (void*)plan->d_zrow,
                  (void*)plan->d_sw_base, (void*)plan->d_sw_len, (void*)plan->d_sw_ends, (void*)plan->d_sw_slot_row,
                  (void*)plan->d_sw_part_base, (void*)plan->d_sw_split_rows, (void*)plan->d_sw_zrow})
    if (q) (void)hipFree(q);
  delete plan;
  return HPSPMM_OK;
}

int hpspmm_plan_bind_values(hpspmm_plan* plan, const float* d_val, void* stream) {
  if (!plan) return fail(HPSPMM_ERR_INVALID_ARG, "plan is NULL");
  plan->bound_val = nullptr;
  if (!d_val || plan->nnz == 0) return HPSPMM_OK;
  if (plan->strategy == HPSPMM_STRATEGY_SWEEP) {
    hipStream_t st = (hipStream_t)stream;
    if (!plan->d_vval) {
      if (hipMalloc(&plan->d_vval, (size_t)std::max<int64_t>(plan->sw_total, 1) * sizeof(float)) != hipSuccess) {
        (void)hipGetLastError();
        plan->d_vval = nullptr;
        return fail(HPSPMM_ERR_ALLOC, "device allocation for the bound values failed");
      }
      plan->workspace_bytes += plan->sw_total * (int64_t)sizeof(float);
    }
    hipLaunchKernelGGL(hpspmm::sweep_gather_values_kernel, dim3(grid_for(plan->sw_total, 1 << 16)), dim3(hpspmm::kBlock),
                       0, st, plan->sw_total, plan->d_vsrc, d_val, plan->d_vval);
    HPSPMM_HIP(hipGetLastError());
  } else if (plan->strategy == HPSPMM_STRATEGY_ROUTED && plan->d_vsrc) {
    // column-range slices: constant values are worth a copy in the plan's order after all (reading them
    // in place costs the main kernel what a bound plan no longer pays in re-ordering)
    hipStream_t st = (hipStream_t)stream;
    const int64_t vtotal = plan->lay.cls_end[plan->lay.nhub];
    if (!plan->d_vval) {
      if (hipMalloc(&plan->d_vval, (size_t)std::max<int64_t>(vtotal, 1) * sizeof(float)) != hipSuccess) {
        (void)hipGetLastError();
        plan->d_vval = nullptr;
        return fail(HPSPMM_ERR_ALLOC, "device allocation for the bound values failed");
      }
      plan->workspace_bytes += vtotal * (int64_t)sizeof(float);
    }
    hipLaunchKernelGGL(hpspmm::routed_gather_values_kernel, dim3(grid_for(vtotal, 1 << 16)), dim3(hpspmm::kBlock), 0,
                       st, vtotal, plan->d_vsrc, d_val, plan->d_vval);
    HPSPMM_HIP(hipGetLastError());
  } else if (plan->strategy == HPSPMM_STRATEGY_ROUTED) {
    hipStream_t st = (hipStream_t)stream;
    // the value half of routed_prepare_kernel alone (its template argument only shapes the other half)
    const int64_t blocks = ceil_div(plan->nnz, hpspmm::kPermChunk);
    if (blocks > INT32_MAX) return fail(HPSPMM_ERR_INVALID_ARG, "grid too large");
    hipLaunchKernelGGL(hpspmm::routed_prepare_kernel<32>, dim3((unsigned)blocks), dim3(hpspmm::kBlock), 0, st,
                       (int64_t)0, (int64_t)0, (const int32_t*)nullptr, (const float*)nullptr, (float*)nullptr,
                       plan->nnz, plan->lay.nhub + 1, d_val, plan->d_lslot, plan->d_chunk_base, plan->d_chunk_pref,
                       plan->d_vval, 32u);
    HPSPMM_HIP(hipGetLastError());
  }
  plan->bound_val = d_val;
  return HPSPMM_OK;
}

int hpspmm_csr_spmm(hpspmm_plan* plan, const int32_t* d_rowptr, const int32_t* d_col, const float* d_val,
                    const float* d_B, float* d_C, void* stream) {
  if (!plan) return fail(HPSPMM_ERR_INVALID_ARG, "plan is NULL");
  if (plan->rows == 0) return HPSPMM_OK;
  if (!d_rowptr || !d_C) return fail(HPSPMM_ERR_INVALID_ARG, "d_rowptr or d_C is NULL");
  if (plan->nnz > 0 && (!d_col || !d_val || !d_B))
    return fail(HPSPMM_ERR_INVALID_ARG, "d_col, d_val or d_B is NULL with nnz > 0");
  // The plan holds the structure of the arrays it was built from (some strategies run entirely
  // from its own copy): other addresses most likely mean another matrix, whose product would
  // silently be that of the old one.
  if (!plan->allow_moved && (d_rowptr != plan->src_rowptr || (plan->nnz > 0 && d_col != plan->src_col)))
    return fail(HPSPMM_ERR_INVALID_ARG,
                "d_rowptr / d_col are not the arrays this plan was built from (build a new plan for another "
                "structure, or create the plan with HPSPMM_PLAN_ALLOW_MOVED_CSR if the same structure has moved)");
  hipStream_t st = (hipStream_t)stream;
  int rc;
  // another value array overwrites the plan's copy of the bound one
  if (plan->bound_val && plan->bound_val != d_val) plan->bound_val = nullptr;
  if (plan->k_full != plan->k || plan->k_user != plan->k_full) {
    // one column tile after the other through the layout built for the tile width; the operands of
    // tile t are columns [t * k, (t + 1) * k) of B and C.  The rows of B are k_full floats apart -
    // the caller's B, or its padded copy when the caller's row length is not a multiple of 4 -,
    // those of C k_user floats.
    rc = HPSPMM_OK;
    const float* Bsrc = d_B;
    if (plan->k_user != plan->k_full) {
      hipLaunchKernelGGL(hpspmm::pad_rows_kernel, dim3(grid_for(plan->cols * plan->k_full, 1 << 16)), dim3(hpspmm::kBlock),
                         0, st, plan->cols, plan->k_user, plan->k_full, d_B, plan->d_bpad);
      mark_launch(st, "pad_rows_kernel");
      Bsrc = plan->d_bpad;
    }
    const uint32_t shorter = (uint32_t)(plan->k_full - plan->k_user);  // 0 ... 3
    for (int t = 0; t < plan->tiles && rc == HPSPMM_OK; ++t) {
      const float* Bt = Bsrc + (int64_t)t * plan->k;
      float* Ct = d_C + (int64_t)t * plan->k;
      // the row length of B; how much shorter C's rows are; the columns of the tile that exist when
      // the last one is narrower than the layout
      const int64_t left = plan->k_user - (int64_t)t * plan->k;
      const uint32_t ld = (uint32_t)plan->k_full | shorter << 22 | (left < plan->k ? (uint32_t)left << 24 : 0u);
      if (plan->strategy != HPSPMM_STRATEGY_ORDERED && plan->strategy != HPSPMM_STRATEGY_SWEEP &&
          plan->strategy != HPSPMM_STRATEGY_ROUTED) {
        rc = fail(HPSPMM_ERR_INVALID_ARG, "plan of column tiles without a tiled strategy");
      } else if (shorter == 0) {
        if (plan->strategy == HPSPMM_STRATEGY_ORDERED) {
          switch (plan->k) {
            case 32: rc = launch_ordered<32, 1>(plan, d_rowptr, d_val, Bt, Ct, st, ld); break;
            case 64: rc = launch_ordered<64, 1>(plan, d_rowptr, d_val, Bt, Ct, st, ld); break;
            default: rc = launch_ordered<128, 1>(plan, d_rowptr, d_val, Bt, Ct, st, ld); break;
          }
        } else if (plan->strategy == HPSPMM_STRATEGY_SWEEP) {
          switch (plan->k) {
            case 32: rc = launch_sweep<32, 1>(plan, d_rowptr, d_val, Bt, Ct, st, ld); break;
            case 64: rc = launch_sweep<64, 1>(plan, d_rowptr, d_val, Bt, Ct, st, ld); break;
            default: rc = launch_sweep<128, 1>(plan, d_rowptr, d_val, Bt, Ct, st, ld); break;
          }
        } else {
          switch (plan->k) {
            case 32: rc = launch_routed<32, 1>(plan, d_val, Bt, Ct, st, ld, t > 0); break;
            case 64: rc = launch_routed<64, 1>(plan, d_val, Bt, Ct, st, ld, t > 0); break;
            default: rc = launch_routed<128, 1>(plan, d_val, Bt, Ct, st, ld, t > 0); break;
          }
        }
      } else {  // rows of C shorter than those of B, at any 4-byte alignment
        if (plan->strategy == HPSPMM_STRATEGY_ORDERED) {
          switch (plan->k) {
            case 32: rc = launch_ordered<32, 2>(plan, d_rowptr, d_val, Bt, Ct, st, ld); break;
            case 64: rc = launch_ordered<64, 2>(plan, d_rowptr, d_val, Bt, Ct, st, ld); break;
            default: rc = launch_ordered<128, 2>(plan, d_rowptr, d_val, Bt, Ct, st, ld); break;
          }
        } else if (plan->strategy == HPSPMM_STRATEGY_SWEEP) {
          switch (plan->k) {
            case 32: rc = launch_sweep<32, 2>(plan, d_rowptr, d_val, Bt, Ct, st, ld); break;
            case 64: rc = launch_sweep<64, 2>(plan, d_rowptr, d_val, Bt, Ct, st, ld); break;
            default: rc = launch_sweep<128, 2>(plan, d_rowptr, d_val, Bt, Ct, st, ld); break;
          }
        } else {
          switch (plan->k) {
            case 32: rc = launch_routed<32, 2>(plan, d_val, Bt, Ct, st, ld, t > 0); break;
            case 64: rc = launch_routed<64, 2>(plan, d_val, Bt, Ct, st, ld, t > 0); break;
            default: rc = launch_routed<128, 2>(plan, d_val, Bt, Ct, st, ld, t > 0); break;
          }
        }
      }
    }
  } else if (plan->strategy == HPSPMM_STRATEGY_ORDERED) {
    switch (plan->k) {
      case 32: rc = launch_ordered<32>(plan, d_rowptr, d_val, d_B, d_C, st); break;
      case 64: rc = launch_ordered<64>(plan, d_rowptr, d_val, d_B, d_C, st); break;
      default: rc = launch_ordered<128>(plan, d_rowptr, d_val, d_B, d_C, st); break;
    }
  } else if (plan->strategy == HPSPMM_STRATEGY_SWEEP) {
    switch (plan->k) {
      case 32: rc = launch_sweep<32>(plan, d_rowptr, d_val, d_B, d_C, st); break;
      case 64: rc = launch_sweep<64>(plan, d_rowptr, d_val, d_B, d_C, st); break;
      default: rc = launch_sweep<128>(plan, d_rowptr, d_val, d_B, d_C, st); break;
    }
  } else if (plan->strategy == HPSPMM_STRATEGY_ROUTED) {
    switch (plan->k) {
      case 32: rc = launch_routed<32>(plan, d_val, d_B, d_C, st); break;
      case 64: rc = launch_routed<64>(plan, d_val, d_B, d_C, st); break;
      default: rc = launch_routed<128>(plan, d_val, d_B, d_C, st); break;
    }
  } else if (plan->strategy == HPSPMM_STRATEGY_SEGMENTS && !fast_k(plan->k)) {
    rc = launch_segments_anyk(plan, d_rowptr, d_col, d_val, d_B, d_C, st);
  } else if (plan->strategy == HPSPMM_STRATEGY_SEGMENTS) {
    switch (plan->k) {
      case 32: rc = launch_segments<32>(plan, d_rowptr, d_col, d_val, d_B, d_C, st); break;
      case 64: rc = launch_segments<64>(plan, d_rowptr, d_col, d_val, d_B, d_C, st); break;
      default: rc = launch_segments<128>(plan, d_rowptr, d_col, d_val, d_B, d_C, st); break;
    }
  } else if (plan->d_tent && plan->rt_mode) {
    const uint32_t ldb = plan->rt_ldb, ldc = (uint32_t)plan->k;
    const int sub = row_tile_sub_lanes(plan->k);
    if (plan->rt_mode == 2) {
      if (plan->nnz > 0) {  // (without nonzeros B is never read, and may be NULL)
        hipLaunchKernelGGL(hpspmm::pad_rows_kernel, dim3(grid_for(plan->cols * (int64_t)ldb, 1 << 16)),
                           dim3(hpspmm::kBlock), 0, st, plan->cols, plan->k, (int64_t)ldb, d_B, plan->d_bpad);
        mark_launch(st, "pad_rows_kernel");
      }
      rc = sub == 1   ? launch_row_tiles<0, 2, 1>(plan, d_val, plan->d_bpad, d_C, st, ldb, ldc)
           : sub == 4 ? launch_row_tiles<0, 2, 4>(plan, d_val, plan->d_bpad, d_C, st, ldb, ldc)
                      : launch_row_tiles<0, 2>(plan, d_val, plan->d_bpad, d_C, st, ldb, ldc);
    } else if (plan->rt_mode == 3) {
      rc = sub == 4 ? launch_row_tiles<0, 3, 4>(plan, d_val, d_B, d_C, st, ldb, ldc)
                    : launch_row_tiles<0, 3>(plan, d_val, d_B, d_C, st, ldb, ldc);
    } else {
      rc = sub == 1   ? launch_row_tiles<0, 1, 1>(plan, d_val, d_B, d_C, st, ldb, ldc)
           : sub == 4 ? launch_row_tiles<0, 1, 4>(plan, d_val, d_B, d_C, st, ldb, ldc)
                      : launch_row_tiles<0, 1>(plan, d_val, d_B, d_C, st, ldb, ldc);
    }
  } else if (plan->d_tent) {
    switch (plan->k) {
      case 32: rc = launch_row_tiles<32>(plan, d_val, d_B, d_C, st); break;
      case 64: rc = launch_row_tiles<64>(plan, d_val, d_B, d_C, st); break;
      default: rc = launch_row_tiles<128>(plan, d_val, d_B, d_C, st); break;
    }
  } else {
    rc = launch_rows_any(plan->rows, plan->cols, plan->k, d_rowptr, d_col, d_val, d_B, d_C, plan->long_threshold,
                         plan->d_long_rows, plan->n_long, st);
  }
  if (rc) return rc;
  HPSPMM_HIP(hipGetLastError());
  return HPSPMM_OK;
}

int hpspmm_csr_spmm_noplan(int64_t rows, int64_t cols, int64_t nnz, const int32_t* d_rowptr,
                           const int32_t* d_col, const float* d_val, const float* d_B, int64_t k, float* d_C,
                           void* stream) {
  if (int rc = check_dims(rows, cols, nnz, k)) return rc;
  if (rows == 0) return HPSPMM_OK;
  if (!d_rowptr || !d_C) return fail(HPSPMM_ERR_INVALID_ARG, "d_rowptr or d_C is NULL");
  if (nnz > 0 && (!d_col || !d_val || !d_B))
    return fail(HPSPMM_ERR_INVALID_ARG, "d_col, d_val or d_B is NULL with nnz > 0");
  if (int rc = launch_rows_any(rows, cols, k, d_rowptr, d_col, d_val, d_B, d_C, INT32_MAX, nullptr, 0,
                               (hipStream_t)stream))
    return rc;
  HPSPMM_HIP(hipGetLastError());
  return HPSPMM_OK;
}

// ---------------------------------------------------------------------------------------------
// hpspmm_csr_spmm_static: the segments strategy without a plan and without any allocation.  What a
// plan would hold in its workspace lives in one file-scope device array: the row of every nonzero
// (kStaticMaxNnz int32) followed by the carry slots (kStaticCarryFloats floats).  Every device the
// library is loaded on holds its own copy of the array; its address there is looked up once per
// device (hipGetSymbolAddress) and only that pointer is ever handed to kernels.
// ---------------------------------------------------------------------------------------------
}  // extern "C"

namespace {
constexpr int64_t kStaticMaxNnz = (int64_t)1 << 22;
constexpr int64_t kStaticCarryFloats = (int64_t)1 << 22;
constexpr size_t kStaticScratchBytes = (size_t)kStaticMaxNnz * sizeof(int32_t) + (size_t)kStaticCarryFloats * sizeof(float);
}  // namespace
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
namespace {
std::mutex g_static_mutex;
void* g_static_ptr[kMaxDevices] = {nullptr};

// Device address of `scratch` on the current device (looked up on the first call per device).
int static_scratch(void** out) {
  int dev = 0;
  HPSPMM_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return fail(HPSPMM_ERR_INVALID_ARG, "device index %d not supported", dev);
  std::lock_guard<std::mutex> lock(g_static_mutex);
  if (!g_static_ptr[dev]) {
    void* ptr = nullptr;
    HPSPMM_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (!ptr) return fail(HPSPMM_ERR_HIP, "hipGetSymbolAddress returned a null address for the static workspace");
    g_static_ptr[dev] = ptr;
  }
  *out = g_static_ptr[dev];
  return HPSPMM_OK;
}

template <int K>
int launch_static(int64_t rows, int64_t nnz, const int32_t* rp, const int32_t* ci, const float* v, const float* B,
                  float* C, int32_t* nnz_row, float* carry, hipStream_t st) {
  constexpr int P = 64 / (K / 4);
  // segment length as a plan would choose it, then doubled until the carry slots fit the static array
  int shift = 5;
  const int64_t target_waves = 256 * 4 * 16;
  while (shift < 9 && (nnz >> (shift + 1)) / P >= target_waves) ++shift;
  while (2 * ceil_div(nnz, (int64_t)1 << shift) * K > kStaticCarryFloats) ++shift;
  const int64_t nseg = ceil_div(nnz, (int64_t)1 << shift);
  if (nnz > 0) {
    hipLaunchKernelGGL(hpspmm::expand_rows_kernel, dim3((unsigned)ceil_div(nnz, hpspmm::kExpandPerBlock)), dim3(hpspmm::kBlock),
                       0, st, rows, nnz, rp, nnz_row);
    const int64_t nblocks = ceil_div(ceil_div(nseg, P), hpspmm::kWavesPerBlock);
    hipLaunchKernelGGL((hpspmm::spmm_segments_kernel<K, false, false>), dim3((unsigned)nblocks), dim3(hpspmm::kBlock),
                       0, st, rp, ci, v, (const int32_t*)nnz_row, B, (const float*)nullptr, C, carry, nnz, shift, nseg,
                       nblocks, false, aligned16(ci, v, nnz_row));
  }
  const int rpw = fixup_rows_per_wave(rows, K);
  const int64_t fix_blocks = ceil_div(ceil_div(rows, rpw), hpspmm::kWavesPerBlock);
  hipLaunchKernelGGL(hpspmm::spmm_fixup_kernel<K>, dim3((unsigned)fix_blocks), dim3(hpspmm::kBlock), 0, st, rows, rp,
                     (const int32_t*)nullptr, (const float*)carry, C, shift, rpw, (uint32_t)K);
  return HPSPMM_OK;
}
}  // namespace

extern "C" {

int hpspmm_csr_spmm_static(int64_t rows, int64_t cols, int64_t nnz, const int32_t* d_rowptr, const int32_t* d_col,
                           const float* d_val, const float* d_B, int64_t k, float* d_C, void* stream) {
  if (int rc = check_dims(rows, cols, nnz, k)) return rc;
  if (!fast_k(k)) return fail(HPSPMM_ERR_INVALID_ARG, "hpspmm_csr_spmm_static: k must be 32, 64 or 128, got %lld", (long long)k);
  if (nnz > kStaticMaxNnz)
    return fail(HPSPMM_ERR_INVALID_ARG,
                "hpspmm_csr_spmm_static: nnz = %lld exceeds the static workspace (at most %lld nonzeros); use a plan",
                (long long)nnz, (long long)kStaticMaxNnz);
  if (rows == 0) return HPSPMM_OK;
  if (!d_rowptr || !d_C) return fail(HPSPMM_ERR_INVALID_ARG, "d_rowptr or d_C is NULL");
  if (nnz > 0 && (!d_col || !d_val || !d_B))
    return fail(HPSPMM_ERR_INVALID_ARG, "d_col, d_val or d_B is NULL with nnz > 0");
  void* base = nullptr;
  if (int rc = static_scratch(&base)) return rc;
  int32_t* nnz_row = static_cast<int32_t*>(base);
  float* carry = reinterpret_cast<float*>(static_cast<unsigned char*>(base) + (size_t)kStaticMaxNnz * sizeof(int32_t));
  hipStream_t st = (hipStream_t)stream;
  int rc;
  switch (k) {
    case 32: rc = launch_static<32>(rows, nnz, d_rowptr, d_col, d_val, d_B, d_C, nnz_row, carry, st); break;
    case 64: rc = launch_static<64>(rows, nnz, d_rowptr, d_col, d_val, d_B, d_C, nnz_row, carry, st); break;
    default: rc = launch_static<128>(rows, nnz, d_rowptr, d_col, d_val, d_B, d_C, nnz_row, carry, st); break;
  }
  if (rc) return rc;
  HPSPMM_HIP(hipGetLastError());
  return HPSPMM_OK;
}

int hpspmm_coo_spmm_accumulate(int64_t rows, int64_t cols, int64_t nnz, const int32_t* d_row,
                               const int32_t* d_col, const float* d_val, const float* d_B, int64_t k, float* d_C,
                               void* stream) {
  if (int rc = check_dims(rows, cols, nnz, k)) return rc;
  if (nnz == 0) return HPSPMM_OK;
  if (rows == 0) return fail(HPSPMM_ERR_INVALID_ARG, "nnz > 0 with rows == 0");
  if (!d_row || !d_col || !d_val || !d_B || !d_C) return fail(HPSPMM_ERR_INVALID_ARG, "NULL device pointer");
  hipStream_t st = (hipStream_t)stream;
  int rc = HPSPMM_OK;
  switch (k) {
    case 32: rc = launch_coo<32>(nnz, d_row, d_col, d_val, d_B, d_C, st); break;
    case 64: rc = launch_coo<64>(nnz, d_row, d_col, d_val, d_B, d_C, st); break;
    case 128: rc = launch_coo<128>(nnz, d_row, d_col, d_val, d_B, d_C, st); break;
    default: rc = launch_coo_anyk(nnz, k, d_row, d_col, d_val, d_B, d_C, st);  // segments reduced in registers, one atomic per flush
  }
  if (rc) return rc;
  HPSPMM_HIP(hipGetLastError());
  return HPSPMM_OK;
}

int hpspmm_fill_f32(float* d_x, int64_t n, float value, void* stream) {
  if (n < 0) return fail(HPSPMM_ERR_INVALID_ARG, "negative length");
  if (n == 0) return HPSPMM_OK;
  if (!d_x) return fail(HPSPMM_ERR_INVALID_ARG, "d_x is NULL");
  hipLaunchKernelGGL(hpspmm::fill_f32_kernel, dim3(grid_for(n, 1 << 16)), dim3(hpspmm::kBlock), 0,
                     (hipStream_t)stream, d_x, n, value);
  HPSPMM_HIP(hipGetLastError());
  return HPSPMM_OK;
}

int hpspmm_csr_spmm_timed(hpspmm_plan* plan, const int32_t* d_rowptr, const int32_t* d_col, const float* d_val,
                          const float* d_B, float* d_C, void* stream, int warmup, int iters, float* mean_ms_out) {
  if (!mean_ms_out || iters <= 0 || warmup < 0) return fail(HPSPMM_ERR_INVALID_ARG, "bad timing arguments");
  hipStream_t st = (hipStream_t)stream;
  for (int i = 0; i < warmup; ++i)
    if (int rc = hpspmm_csr_spmm(plan, d_rowptr, d_col, d_val, d_B, d_C, stream)) return rc;
  hipEvent_t t0, t1;
  HPSPMM_HIP(hipEventCreate(&t0));
  HPSPMM_HIP(hipEventCreate(&t1));
  int rc = HPSPMM_OK;
  hipError_t e = hipEventRecord(t0, st);
  for (int i = 0; i < iters && rc == HPSPMM_OK && e == hipSuccess; ++i)
    rc = hpspmm_csr_spmm(plan, d_rowptr, d_col, d_val, d_B, d_C, stream);
  if (e == hipSuccess) e = hipEventRecord(t1, st);
  if (e == hipSuccess) e = hipEventSynchronize(t1);
  float ms = 0.f;
  if (e == hipSuccess && rc == HPSPMM_OK) e = hipEventElapsedTime(&ms, t0, t1);
  (void)hipEventDestroy(t0);
  (void)hipEventDestroy(t1);
  if (rc) return rc;
  if (e != hipSuccess) return fail(HPSPMM_ERR_HIP, "timing failed: %s", hipGetErrorString(e));
  *mean_ms_out = ms / (float)iters;
  return HPSPMM_OK;
}

int hpspmm_csr_spmm_timed_launches(hpspmm_plan* plan, const int32_t* d_rowptr, const int32_t* d_col,
                                   const float* d_val, const float* d_B, float* d_C, void* stream, int warmup,
                                   int iters, int max_launches, float* mean_ms_out, const char** names_out,
                                   int* n_launches_out) {
  if (!mean_ms_out || !names_out || !n_launches_out || iters <= 0 || warmup < 0 || max_launches <= 0)
    return fail(HPSPMM_ERR_INVALID_ARG, "bad timing arguments");
  *n_launches_out = 0;
  hipStream_t st = (hipStream_t)stream;
  for (int i = 0; i < warmup; ++i)
    if (int rc = hpspmm_csr_spmm(plan, d_rowptr, d_col, d_val, d_B, d_C, stream)) return rc;
  LaunchTrace trace;
  hipEvent_t begin;
  HPSPMM_HIP(hipEventCreate(&begin));
  int created = 0;
  hipError_t e = hipSuccess;
  for (; created < kMaxTracedLaunches && e == hipSuccess; ++created) e = hipEventCreate(&trace.ev[created]);
  if (e != hipSuccess) {
    for (int q = 0; q < created - 1; ++q) (void)hipEventDestroy(trace.ev[q]);
    (void)hipEventDestroy(begin);
    return fail(HPSPMM_ERR_HIP, "hipEventCreate: %s", hipGetErrorString(e));
  }
  double sum[kMaxTracedLaunches] = {0};
  int rc = HPSPMM_OK, n = 0;
  for (int i = 0; i < iters && rc == HPSPMM_OK && e == hipSuccess; ++i) {
    trace.n = 0;
    e = hipEventRecord(begin, st);
    g_trace = &trace;
    rc = hpspmm_csr_spmm(plan, d_rowptr, d_col, d_val, d_B, d_C, stream);
    g_trace = nullptr;
    if (rc != HPSPMM_OK || e != hipSuccess) break;
    n = trace.n;
    if (n == 0) break;
    e = hipEventSynchronize(trace.ev[n - 1]);
    for (int q = 0; q < n && e == hipSuccess; ++q) {
      float ms = 0.f;
      e = hipEventElapsedTime(&ms, q == 0 ? begin : trace.ev[q - 1], trace.ev[q]);
      sum[q] += ms;
    }
  }
  (void)hipEventDestroy(begin);
  for (int q = 0; q < created; ++q) (void)hipEventDestroy(trace.ev[q]);
  if (rc) return rc;
  if (e != hipSuccess) return fail(HPSPMM_ERR_HIP, "timing failed: %s", hipGetErrorString(e));
  const int out = n < max_launches ? n : max_launches;
  for (int q = 0; q < out; ++q) {
    mean_ms_out[q] = (float)(sum[q] / iters);
    names_out[q] = trace.name[q];
  }
  *n_launches_out = out;
  return HPSPMM_OK;
}

}  // extern "C"
