// Shared helpers of plan construction: error messages, launch tracing, device scan and radix sort,
// column ranking, the row of every nonzero, the probe of how workgroups are dealt to the XCDs.
#include "host.hpp"

#include <cstdarg>
#include <mutex>
#include <string>

#include "rank_kernels.hpp"
#include "routed_plan_kernels.hpp"

namespace hpspmm_host {

namespace {
thread_local std::string g_last_error;
thread_local LaunchTrace* g_trace = nullptr;
}  // namespace

int fail(int code, const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  g_last_error = buf;
  return code;
}

const char* last_error_message() { return g_last_error.c_str(); }

void set_launch_trace(LaunchTrace* t) { g_trace = t; }

void mark_launch(hipStream_t st, const char* name) {
  LaunchTrace* t = g_trace;
  if (!t) return;
  ++t->launches;
  if (t->n >= kMaxTracedLaunches) return;
  (void)hipEventRecord(t->ev[t->n], st);
  t->name[t->n++] = name;
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

// The routed strategy pins column slices to XCDs and xcd_remap deals row ranges to them; both rely on
// workgroup b of a launch running on XCD b % 8.  That holds for the whole device (8 XCDs, 256 CUs);
// a partitioned device (fewer XCDs behind one HIP device) or a future dispatcher would break it
// silently, so it is measured once per device: 512 probe workgroups report the XCD they ran on.
// 0 = not probed yet, 1 = workgroup b runs on XCD b % 8, 2 = it does not (the plan then keeps to the
// strategies that do not depend on it).
namespace {
constexpr int kMaxDevices = 64;
constexpr int kProbeBlocks = 512;
std::mutex g_xcd_mutex;
int g_xcd_state[kMaxDevices] = {0};
}  // namespace

bool xcd_dealing_holds(hipStream_t st, int assume) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    (void)hipGetLastError();
    return false;
  }
  if (assume == 0 || assume == 1) return assume == 1;  // the caller's word instead of the probe
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

int64_t sort_tile() { return hpspmm::kSortTile; }

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

int sort_rows_by_label(int64_t rows, const int32_t* d_label, int64_t label_range, hipStream_t st,
                       int32_t** d_order_out) {
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
  while (bits < 32 && ((int64_t)1 << bits) < label_range) ++bits;
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

// Histogram of every `stride`-th column index into a fresh d_count_out (caller frees).
static int count_columns(const hpspmm_plan* p, const int32_t* d_col, int64_t stride, hipStream_t st, int32_t** d_count_out) {
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
static int select_top_columns(const int32_t* d_count, int64_t n, int64_t want, hipStream_t st,
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

int stored_order_miss_share(const hpspmm_plan* p, const int32_t* d_col, hipStream_t st, double* share) {
  *share = 1.0;
  const int64_t nnz = p->nnz;
  if (nnz < (int64_t)kLocalitySamples * hpspmm::kLocalityBlock) return HPSPMM_OK;
  DeviceTemps tmp;
  uint32_t* d_tables = nullptr;
  const size_t table_words = (size_t)1 << (hpspmm::kLocalityBits - 5);
  const size_t words = kLocalitySamples * table_words + 4 * kLocalitySamples;
  if (tmp.alloc(&d_tables, words) != HPSPMM_OK) return HPSPMM_OK;  // no room: no estimate
  uint32_t* d_out = d_tables + kLocalitySamples * table_words;
  HPSPMM_HIP(hipMemsetAsync(d_tables, 0, words * sizeof(uint32_t), st));
  hipLaunchKernelGGL(hpspmm::locality_walk_kernel, dim3(kLocalitySamples), dim3(hpspmm::kLocalityBlock), 0, st, nnz, d_col,
                     nnz / kLocalitySamples, p->cols > ((int64_t)1 << hpspmm::kLocalityBits) ? 1 : 0,
                     (uint32_t)kLocalityCapacity, (uint32_t)(kLocalityMaxWalk * kLocalityCapacity), d_tables, d_out);
  uint32_t out[4 * kLocalitySamples];
  HPSPMM_HIP(hipMemcpyAsync(out, d_out, sizeof out, hipMemcpyDeviceToHost, st));
  HPSPMM_HIP(hipStreamSynchronize(st));
  double fresh = 0, walked = 0;
  for (int s = 0; s < kLocalitySamples; ++s) {
    fresh += (double)out[4 * s + 3] - (double)out[4 * s + 1];
    walked += (double)out[4 * s + 2] - (double)out[4 * s + 0];
  }
  if (walked > 0) *share = std::min(1.0, fresh / walked);
  return HPSPMM_OK;
}

}  // namespace hpspmm_host
