// Host side of libhpspmm.so, shared by its translation units: error reporting, the plan, the
// helpers of plan construction (scan, sort, column ranking) and the launch functions of every
// strategy.  Nothing here is part of the C ABI (include/hpspmm.h).
//
//   abi.hip            entry points that are not about plans: SpMM dispatch, timing, fill, COO,
//                      the plan-less and the allocation-free SpMM
//   plan.hip           hpspmm_plan_create*: validation, the choice of strategy, plan info,
//                      value binding, destruction
//   plan_util.hip      device scan / radix sort / column ranking / row expansion / XCD probe
//   plan_rows.hip      row tiles (rows strategy)
//   plan_routed.hip    routed layout            launch_routed.hip   its kernels' launches
//   plan_ordered.hip   clustering, ordered layout
//   plan_sweep.hip     sweep layout             launch_sweep.hip    its kernels' launches
//   launch_rows.hip    whole rows: CSR arrays, row tiles, run-time row lengths
//   launch_segments.hip  segments (+ hub cache), ordered, COO accumulate, static workspace
#pragma once

#include "hpspmm.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <climits>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <type_traits>
#include <vector>

#include "anyk_kernels.hpp"
#include "routed_kernels.hpp"
#include "spmm_kernels.hpp"
#include "sweep_kernels.hpp"

// Entry points of the C ABI are the only symbols the library exports.
#define HPSPMM_API extern "C" __attribute__((visibility("default")))

namespace hpspmm_host {

// Sets the calling thread's error message (hpspmm_last_error) and returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
const char* last_error_message();

#define HPSPMM_HIP(call)                                                                                \
  do {                                                                                                  \
    hipError_t e_ = (call);                                                                             \
    if (e_ != hipSuccess)                                                                               \
      return ::hpspmm_host::fail(e_ == hipErrorNoDevice ? HPSPMM_ERR_NO_DEVICE : HPSPMM_ERR_HIP, "%s: %s", \
                                 #call, hipGetErrorString(e_));                                         \
  } while (0)

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Per-launch timing (hpspmm_csr_spmm_timed_launches): while a trace is active on the calling
// thread, every kernel launch of an SpMM is followed by an event record on the launch stream.
// Launches beyond the trace's capacity are counted, not recorded.
constexpr int kMaxTracedLaunches = 32;
struct LaunchTrace {
  hipEvent_t ev[kMaxTracedLaunches];
  const char* name[kMaxTracedLaunches];
  int n = 0;        // events recorded
  int launches = 0;  // launches seen
};
void set_launch_trace(LaunchTrace* t);  // NULL ends the trace
void mark_launch(hipStream_t st, const char* name);

inline bool fast_k(int64_t k) { return k == 32 || k == 64 || k == 128; }
// Not a multiple of 4: rows of B and C start at any multiple of 4 bytes, the last lane of a row owns 1 to 3 columns.
inline bool odd_k(int64_t k) { return k % 4 != 0; }

// Lanes per sub-wave of the run-time-K kernels for row length k: the power of two that covers a
// column tile (at most 128 floats); and how many such tiles a row has.
inline int anyk_lanes(int64_t k) {
  const int64_t g = ((k < hpspmm::kAnyKTile ? k : hpspmm::kAnyKTile) + 3) / 4;
  int gp = 2;
  while (gp < g) gp <<= 1;
  return gp;
}
inline int anyk_tiles(int64_t k) { return (int)((k + hpspmm::kAnyKTile - 1) / hpspmm::kAnyKTile); }
// f(std::integral_constant<int, GP>) for GP = anyk_lanes(k).
template <class F>
int dispatch_anyk_lanes(int64_t k, F&& f) {
  switch (anyk_lanes(k)) {
    case 2: return f(std::integral_constant<int, 2>{});
    case 4: return f(std::integral_constant<int, 4>{});
    case 8: return f(std::integral_constant<int, 8>{});
    case 16: return f(std::integral_constant<int, 16>{});
    default: return f(std::integral_constant<int, 32>{});
  }
}

// Rows longer than this are handled by a whole wavefront in the rows strategy over the CSR arrays.
constexpr int32_t kLongRowThreshold = 32;

// Launch geometry of the kernels that run one sub-wave per row.
inline int64_t row_blocks(int64_t rows, int64_t k) {
  const int64_t per_wave = 64 / (k / 4);
  return (((rows + per_wave - 1) / per_wave) + hpspmm::kWavesPerBlock - 1) / hpspmm::kWavesPerBlock;
}

inline bool aligned16(const void* a, const void* b, const void* c) {
  return (((uintptr_t)a | (uintptr_t)b | (uintptr_t)c) & 15u) == 0;
}

int check_dims(int64_t rows, int64_t cols, int64_t nnz, int64_t k);

inline int grid_for(int64_t items, int64_t cap = 1 << 20) {
  int64_t b = ceil_div(items, hpspmm::kBlock);
  if (b < 1) b = 1;
  if (b > cap) b = cap;
  return (int)b;
}

// f(std::integral_constant<int, K>) for the tuned row length k (32, 64, anything else = 128).
template <class F>
int dispatch_k(int64_t k, F&& f) {
  switch (k) {
    case 32: return f(std::integral_constant<int, 32>{});
    case 64: return f(std::integral_constant<int, 64>{});
    default: return f(std::integral_constant<int, 128>{});
  }
}
// f(K, kLd) for the tuned row length k and the operand form ld_mode of the tiled kernels (0: rows of
// B and C are K floats; 1: row lengths at run time; 2: rows of C shorter than those of B).
template <class F>
int dispatch_k_ld(int64_t k, int ld_mode, F&& f) {
  return dispatch_k(k, [&](auto K) {
    switch (ld_mode) {
      case 0: return f(K, std::integral_constant<int, 0>{});
      case 1: return f(K, std::integral_constant<int, 1>{});
      default: return f(K, std::integral_constant<int, 2>{});
    }
  });
}

// What hpspmm_plan_options carries (see include/hpspmm.h), sizes packed into the flag word unpacked.
struct PlanOptions {
  uint32_t flags = 0;
  const int32_t* d_row_order = nullptr;
  int segment_shift = 0;      // 0 = automatic
  int hub_log2 = 0;           // 0 = default
  int routed_row_log2 = 0, routed_phases = 0;
  int routed_tile_width = 0;  // 0 = automatic, -1 = never, 32 / 64
  bool routed_split_launch = false;
  int routed_lds_rows = 0;    // column-tile phases: rows of B a workgroup keeps in LDS (0 = what fits, -1 = none)
  int xcd_dealing = -1;       // -1 probe, 0 / 1 assume
  bool column_tiles = true;   // a row length outside the tuned set may get the tiled layouts
  int64_t row_tiles_min_k = 1;
  int row_tiles_pad = -1;     // -1 auto, 0 never, 1 whenever the length is not a multiple of 32
  bool row_tiles_narrow = true;    // 4 / 1 lanes per entry at <= 16 / <= 4 columns
  bool row_tiles_same_xcd = true;
  int row_tiles_chunk_log2 = 0;  // tuned row lengths: 2^n consecutive groups of row tiles to an XCD at a time (0: the plan decides, -1: one)
  int sweep_window_log2 = 0, sweep_lead = 0, sweep_limit = 0;  // 0 = default
  int sweep_spin = -1;        // -1 = default, else the limit (0 = never wait)
  int sweep_priorities = -1;  // -1 = default (on), 0 = off
  int cluster_sweeps = 0;
  bool report = false;        // plan-time reports on stderr
};

}  // namespace hpspmm_host

struct hpspmm_plan {
  int64_t rows = 0, cols = 0, nnz = 0, k = 0;
  double stored_miss = -1.0;  // stored_order_miss_share() of the matrix, if the choice of strategy measured it
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
  // (column-tile phases keep the rows run by run instead: d_vcol then holds entry words, see kRunStart)
  int32_t* d_run_row = nullptr;   // [n_runs] routed-row number or row of every run, in class-major order
  int32_t* d_seg_run = nullptr;   // [nseg] run of every segment's first entry
  int64_t n_runs = 0;
  int32_t* d_bhot_src = nullptr;  // [n_bhot] source column of every compact-buffer row (-1 = unused)
  int32_t* d_routed_rows = nullptr;  // [n_routed] row of every routed-row number
  int32_t* d_cross_rows = nullptr;   // routed: short rows whose run crosses a segment boundary
  int32_t* d_zero_rows = nullptr;    // rows without nonzeros
  int64_t n_cross = 0, n_zero = 0;
  float* d_partial = nullptr;     // [n_routed * nhub * k]
  int64_t n_bhot = 0;
  int64_t routed_grid = 0;
  bool routed_split_launch = false;  // diagnostics: hub phases and cold class as launches of their own
  const float* bound_val = nullptr;  // value array whose class-major copy d_vval currently holds (or NULL)
  // ordered strategy
  int32_t* d_ostart = nullptr;  // [rows] first position of every row in processing order
  int32_t* d_ocol = nullptr;    // [nnz] entry words: column, or slot of the window's LDS copy of B; first-of-row flag
  int32_t* d_run_delta = nullptr;  // [n_runs] index of a row's first value in the caller's array - its position in the order
  // (d_run_row: the non-empty rows in processing order; d_seg_run, d_zero_rows as above; d_cross_rows: the rows
  // that cross a window boundary)
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
  int rt_sub = 8;            // lanes per entry of the row-tile kernels at such a row length: 8, 4 or 1
  bool rt_same_xcd = true;   // the column tiles of a group of row tiles on one XCD where rows of B share lines
  int rt_chunk_log2 = 0;     // tuned row lengths: 2^n consecutive groups of row tiles to an XCD at a time (0: one, -1: by the size)
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

namespace hpspmm_host {

// ---- plan_util.hip -------------------------------------------------------------------------

// Whether workgroup b of a launch runs on XCD b % 8 on the current device (probed once per device
// and process; `assume` = 0 / 1 skips the probe).
bool xcd_dealing_holds(hipStream_t st, int assume);

// Words of scratch the scan below needs for n values.
inline int64_t scan_scratch_words(int64_t n) { return ceil_div(n, hpspmm::kScanTile) + 1; }
// Device exclusive scan of n uint32 values (three passes, tile sums in between) with the caller's
// scratch (scan_scratch_words(n) words): launches only, no allocation, no synchronisation.  d_out may be d_in.
int exclusive_scan_u32(const uint32_t* d_in, uint32_t* d_out, int64_t n, hipStream_t st, uint32_t* d_tiles);
// The same with scratch of its own; synchronises the stream.
int exclusive_scan_u32(const uint32_t* d_in, uint32_t* d_out, int64_t n, hipStream_t st);

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
// d_vals[0] hold the input, [1] are buffers of the same size, d_hist has 256 * tiles + 1 counters
// (tiles = ceil(n / sort_tile())), d_scan_scratch scan_scratch_words(256 * tiles) words; returns in
// *result which of the two value buffers holds the sorted values.  Launches only.
int64_t sort_tile();
int radix_sort_pairs(int64_t n, uint32_t* d_keys[2], int32_t* d_vals[2], uint32_t* d_hist, uint32_t* d_scan_scratch,
                     int bits, hipStream_t st, int* result);
// *d_order_out = the row numbers sorted by label[row], rows of one label in increasing order (a new
// device array of `rows` entries, caller frees).  Labels lie in [0, label_range).
int sort_rows_by_label(int64_t rows, const int32_t* d_label, int64_t label_range, hipStream_t st,
                       int32_t** d_order_out);

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
int rank_columns(const hpspmm_plan* p, const int32_t* d_col, int64_t want, hipStream_t st, ColumnRanking& rk);

// p->d_nnz_row = the row of every nonzero, built the first time a step of the construction needs it
// (the segments kernels, the sortedness check, the routed and sweep layouts do; a plan that ends up
// with the ordered strategy or with row tiles never does).
int ensure_row_expansion(hpspmm_plan* p, const int32_t* d_rowptr, hipStream_t st);
// True if the column indices of every row are in non-decreasing order.  Errors count as "no".
bool columns_sorted(hpspmm_plan* p, const int32_t* d_rowptr, const int32_t* d_col, hipStream_t st);

// Share of the gathers of rows of B that miss a cache of about 30k rows of B (one 32-column tile of
// them: 4 MB, an L2) when the matrix is walked in stored order, every XCD taking one piece in eight:
// 32 samples of the column stream, each walked until it has met 40k distinct columns (or 16 times as
// many nonzeros).  Near 1 for columns without any order, 1 / (references per column within reach)
// for a banded or block-structured matrix.  1.0 when the matrix is too small to sample or there is
// no room for the bit tables.
constexpr int kLocalitySamples = 32;
constexpr int64_t kLocalityCapacity = 40960;
constexpr int64_t kLocalityMaxWalk = 16;
int stored_order_miss_share(const hpspmm_plan* p, const int32_t* d_col, hipStream_t st, double* share);

// ---- layouts (plan_*.hip): each leaves p->strategy alone when the matrix does not qualify ----

int build_row_tiles(hpspmm_plan* p, const int32_t* d_rowptr, const int32_t* d_col, hipStream_t st);
int build_routed(hpspmm_plan* p, const int32_t* d_rowptr, const int32_t* d_col, bool forced, const PlanOptions& opt,
                 ColumnRanking& rk, hipStream_t st);
int build_ordered(hpspmm_plan* p, const int32_t* d_rowptr, const int32_t* d_col, const int32_t* d_order,
                  double min_served, hipStream_t st);
int cluster_rows(hpspmm_plan* p, const int32_t* d_rowptr, const int32_t* d_col, const PlanOptions& opt,
                 hipStream_t st, int32_t** d_order_out, double* intra_share_out);
int build_sweep(hpspmm_plan* p, const int32_t* d_rowptr, const int32_t* d_col, bool forced, double other_us,
                const PlanOptions& opt, hipStream_t st);

// ---- launches (launch_*.hip) ---------------------------------------------------------------

// Row tiles serve row length k (every tuned length; any other up to 2^22 from opt.row_tiles_min_k).
constexpr int64_t kRowTileMaxNnz = (int64_t)1 << 28;

int launch_rows_any(int64_t rows, int64_t cols, int64_t k, const int32_t* rp, const int32_t* ci, const float* v,
                    const float* B, float* C, int32_t long_threshold, const int32_t* long_rows, int64_t n_long,
                    hipStream_t st);
// Whole rows over the plan's row tiles (plan->d_tent), at a tuned or any other row length.
int launch_row_tiles_plan(const hpspmm_plan* p, const float* v, const float* B, float* C, hipStream_t st);
int launch_segments_plan(const hpspmm_plan* p, const int32_t* rp, const int32_t* ci, const float* v, const float* B,
                         float* C, hipStream_t st);
// ld_mode / ld: see dispatch_k_ld and row_length() in spmm_kernels.hpp.
int launch_ordered_plan(const hpspmm_plan* p, const int32_t* rp, const float* v, const float* B, float* C,
                        hipStream_t st, int ld_mode, uint32_t ld);
int launch_routed_plan(const hpspmm_plan* p, const float* v, const float* B, float* C, hipStream_t st, int ld_mode,
                       uint32_t ld, bool values_ready);
int launch_sweep_plan(const hpspmm_plan* p, const int32_t* rp, const float* v, const float* B, float* C,
                      hipStream_t st, int ld_mode, uint32_t ld);
int launch_coo_any(int64_t nnz, int64_t k, const int32_t* ri, const int32_t* ci, const float* v, const float* B,
                   float* C, hipStream_t st);
// The segments strategy from a workspace of the caller's: row of every nonzero (nnz int32) and carry slots.
int launch_segments_workspace(int64_t rows, int64_t nnz, int64_t k, const int32_t* rp, const int32_t* ci,
                              const float* v, const float* B, float* C, int32_t* nnz_row, float* carry,
                              int64_t carry_floats, hipStream_t st);
// Lets the routed strategy's column-tile kernel of that tile width have its LDS; *lds_rows = rows of B
// that fit a workgroup's LDS next to its staging tiles.
int routed_tiles_prepare(int tile_width, int* lds_rows);
// Lets the sweep kernels for row length k have their LDS; *per_cu = workgroups of them one CU holds.
int sweep_prepare_kernels(int64_t k, int* per_cu);
// Wavefronts per workgroup of the sweep kernel for row length k.
int sweep_waves_for(int64_t k);
// The caller's values in the plan's own order, for hpspmm_plan_bind_values.
int bind_values_sweep(hpspmm_plan* p, const float* d_val, hipStream_t st);
int bind_values_routed(hpspmm_plan* p, const float* d_val, hipStream_t st);
// dst[r, 0:kp) = src[r, 0:k) followed by zeros.
int launch_pad_rows(int64_t rows, int64_t k, int64_t kp, const float* src, float* dst, hipStream_t st);

}  // namespace hpspmm_host
