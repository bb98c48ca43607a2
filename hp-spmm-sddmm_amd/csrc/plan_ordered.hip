// Ordered strategy: clustering of the rows (label propagation) and the layout over a row order.
#include "host.hpp"

#include "ordered_kernels.hpp"
#include "rank_kernels.hpp"
#include "routed_plan_kernels.hpp"

namespace hpspmm_host {

namespace {
// LDS of one workgroup of the ordered strategy, staging tiles included: the most that still lets
// three workgroups share a CU's 160 KB (measured on the co-purchase graph, K = 64: 3.14 ms with
// 32 KB for the rows of B, 2.92 ms with 45 KB, 3.39 ms with 46 KB, where only two fit).
constexpr int kOrderedBlockLdsBytes = 52992;
}  // namespace

// Builds the ordered layout for the processing order d_order (a permutation of
// the row numbers, in device memory).  p->shift is chosen here.
// With min_served > 0 the layout is kept only if at least that share of the nonzeros reads B from
// LDS; otherwise everything built here is freed again and the plan is left as it was.
int build_ordered(hpspmm_plan* p, const int32_t* d_rowptr, const int32_t* d_col, const int32_t* d_order,
                  double min_served, hipStream_t st) {
  const int64_t rows = p->rows, nnz = p->nnz, k = p->k;
  if (p->cols > (int64_t)hpspmm::kEntryPayload) return HPSPMM_OK;  // an entry word keeps the column in 29 bits
  const int64_t subwaves = 64 / (k / 4);
  // window = one workgroup's segments, at most kOrderedMaxWindow nonzeros
  int shift = 9;
  while (((int64_t)hpspmm::kWavesPerBlock * subwaves << shift) > hpspmm::kOrderedMaxWindow) --shift;
  const int window = (int)((int64_t)hpspmm::kWavesPerBlock * subwaves << shift);
  const int64_t staging_bytes = 3 * hpspmm::kWavesPerBlock * subwaves * hpspmm::kTileStride * 4;
  const int cap = (int)((kOrderedBlockLdsBytes - staging_bytes) / (k * 4));
  // (at the end of a window the same LDS takes one row of K floats per segment, spmm_ordered_kernel)
  if (cap < hpspmm::kWavesPerBlock * subwaves) return HPSPMM_OK;
  const int64_t windows = ceil_div(nnz, window);
  const int64_t nseg = ceil_div(nnz, (int64_t)1 << shift);

  uint32_t* d_len = nullptr;   // [rows + 1] row lengths in processing order, then their scan
  uint32_t* d_some = nullptr;  // [rows + 1] 1 for a row with nonzeros, then the scan: its run number
  int32_t* d_seen = nullptr;   // [rows] + [1]: permutation check
  unsigned long long* d_served = nullptr;
  struct Guard {
    void** q[4];
    ~Guard() {
      for (void** x : q)
        if (*x) (void)hipFree(*x);
    }
  } guard{{(void**)&d_len, (void**)&d_seen, (void**)&d_served, (void**)&d_some}};
  HPSPMM_HIP(hipMalloc(&d_len, (size_t)(rows + 1) * sizeof(uint32_t)));
  HPSPMM_HIP(hipMalloc(&d_some, (size_t)(rows + 1) * sizeof(uint32_t)));
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
                     d_len, d_some);
  if (int rc = exclusive_scan_u32(d_len, d_len, rows + 1, st)) return rc;
  if (int rc = exclusive_scan_u32(d_some, d_some, rows + 1, st)) return rc;
  uint32_t runs = 0;
  HPSPMM_HIP(hipMemcpyAsync(&runs, d_some + rows, sizeof runs, hipMemcpyDeviceToHost, st));
  HPSPMM_HIP(hipStreamSynchronize(st));
  const int64_t n_runs = runs;

  const size_t n_bytes = (size_t)std::max<int64_t>(nnz, 1) * sizeof(int32_t);
  const size_t start_bytes = (size_t)std::max<int64_t>(rows, 1) * sizeof(int32_t);
  const size_t wcols_bytes = (size_t)std::max<int64_t>(windows, 1) * (size_t)cap * sizeof(int32_t);
  const size_t carry_bytes = (size_t)std::max<int64_t>(nseg, 1) * 2 * (size_t)k * sizeof(float);
  float* d_new_carry = nullptr;
  auto drop = [&]() {
    for (void** q : {(void**)&p->d_ostart, (void**)&p->d_ocol, (void**)&p->d_wcols,
                     (void**)&d_new_carry, (void**)&p->d_run_row, (void**)&p->d_run_delta, (void**)&p->d_seg_run,
                     (void**)&p->d_cross_rows, (void**)&p->d_zero_rows}) {
      if (*q) (void)hipFree(*q);
      *q = nullptr;
    }
  };
  const size_t run_bytes = (size_t)std::max<int64_t>(n_runs, 1) * sizeof(int32_t);
  const size_t seg_bytes = (size_t)std::max<int64_t>(nseg, 1) * sizeof(int32_t);
  if (hipMalloc(&p->d_ostart, start_bytes) != hipSuccess || hipMalloc(&p->d_ocol, n_bytes) != hipSuccess ||
      hipMalloc(&p->d_run_row, run_bytes) != hipSuccess || hipMalloc(&p->d_run_delta, run_bytes) != hipSuccess ||
      hipMalloc(&p->d_seg_run, seg_bytes) != hipSuccess ||
      hipMalloc(&p->d_wcols, wcols_bytes) != hipSuccess || hipMalloc(&d_new_carry, carry_bytes) != hipSuccess) {
    (void)hipGetLastError();
    drop();
    return fail(HPSPMM_ERR_ALLOC, "device allocation for the ordered plan failed");
  }
  hipLaunchKernelGGL(hpspmm::ordered_fill_kernel, dim3((unsigned)ceil_div(rows, hpspmm::kWavesPerBlock)),
                     dim3(hpspmm::kBlock), 0, st, rows, d_rowptr, d_col, d_order, d_len, d_some, shift, p->d_ostart,
                     p->d_ocol, p->d_run_row, p->d_run_delta, p->d_seg_run);
  if (windows > INT32_MAX) {
    drop();
    return fail(HPSPMM_ERR_INVALID_ARG, "grid too large");
  }
  if (nnz > 0)
    hipLaunchKernelGGL(hpspmm::ordered_hot_kernel, dim3((unsigned)windows), dim3(hpspmm::kBlock), 0, st, nnz, window,
                       cap, p->d_ocol, p->d_wcols, d_served);
  // (A row's nonzeros stay in stored order.  Moving those that read B from LDS behind the others within
  // every row - a batch of gathers is as slow as its slowest load - bought nothing: co-purchase graph,
  // K = 64, 2.93 ms with that order, 2.92 without, and it cost an index per nonzero to find the values.)
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
  // the lists of the rows the fix-up kernel has to visit: those without nonzeros and those that cross
  // a window boundary (the main kernel adds up the rows cut inside a window)
  {
    int window_shift = shift;
    while (((int64_t)1 << window_shift) < window) ++window_shift;
    DeviceTemps tmp;
    uint8_t* d_action = nullptr;
    int32_t* d_counts = nullptr;
    int rc = tmp.alloc(&d_action, (size_t)std::max<int64_t>(rows, 1));
    if (!rc) rc = tmp.alloc(&d_counts, 2);
    if (rc || hipMalloc(&p->d_cross_rows, start_bytes) != hipSuccess || hipMalloc(&p->d_zero_rows, start_bytes) != hipSuccess) {
      (void)hipGetLastError();
      drop();
      return rc ? rc : fail(HPSPMM_ERR_ALLOC, "device allocation for the ordered plan failed");
    }
    const unsigned row_grid = (unsigned)ceil_div(std::max<int64_t>(rows, 1), hpspmm::kBlock);
    hipLaunchKernelGGL(hpspmm::ordered_action_kernel, dim3(row_grid), dim3(hpspmm::kBlock), 0, st, rows, d_rowptr,
                       p->d_ostart, window_shift, d_action);
    hipError_t e2 = hipMemsetAsync(d_counts, 0, 2 * sizeof(int32_t), st);
    const unsigned collect_grid = (unsigned)ceil_div(std::max<int64_t>(rows, 1), hpspmm::kCollectRows);
    hipLaunchKernelGGL(hpspmm::routed_collect_rows_kernel, dim3(collect_grid), dim3(hpspmm::kBlock), 0, st, rows, d_action,
                       hpspmm::kActionCross, p->d_cross_rows, d_counts);
    hipLaunchKernelGGL(hpspmm::routed_collect_rows_kernel, dim3(collect_grid), dim3(hpspmm::kBlock), 0, st, rows, d_action,
                       hpspmm::kActionZero, p->d_zero_rows, d_counts + 1);
    int32_t counts[2] = {0, 0};
    if (e2 == hipSuccess) e2 = hipMemcpyAsync(counts, d_counts, sizeof counts, hipMemcpyDeviceToHost, st);
    if (e2 == hipSuccess) e2 = hipStreamSynchronize(st);
    if (e2 == hipSuccess) e2 = hipGetLastError();
    if (e2 != hipSuccess) {
      drop();
      return fail(HPSPMM_ERR_HIP, "construction of the ordered plan failed: %s", hipGetErrorString(e2));
    }
    p->n_cross = counts[0];
    p->n_zero = counts[1];
    p->n_runs = n_runs;
  }
  // accepted: the segments strategy's buffers are not needed any more
  if (p->d_nnz_row) { (void)hipFree(p->d_nnz_row); p->d_nnz_row = nullptr; }
  if (p->d_carry) (void)hipFree(p->d_carry);
  p->d_carry = d_new_carry;
  p->workspace_bytes = (int64_t)(3 * start_bytes + n_bytes + wcols_bytes + carry_bytes + 2 * run_bytes + seg_bytes);
  p->shift = shift;
  p->nseg = nseg;
  p->ocap = cap;
  p->owindows = windows;
  p->oserved = (int64_t)served;
  p->strategy = HPSPMM_STRATEGY_ORDERED;
  return HPSPMM_OK;
}

// Label propagation over a graph of n vertices given as CSR adjacency (nnz entries): *d_label_out
// receives the label of every vertex (a new device array, caller frees; NULL with status OK when the
// device has no room for the labels), *intra_share_out the share of the entries whose two ends carry
// one label of at most kClusterMaxSize vertices.
constexpr int kClusterMaxSweeps = 16;
constexpr int32_t kClusterMaxSize = 4096;  // vertices of a cluster that still counts as one a window can profit from
constexpr int kClusterLookSweeps = 4;           // after this many sweeps the clusters found so far are scored once
// ... and the propagation ends if their share of the entries is below this (graphs with communities: 0.12-0.18 by then,
// on their way to 0.46-0.83; preferential attachment, R-MAT, users x items, uniform rows: 0.003-0.026, never beyond 0.03)
constexpr double kClusterLookMinIntra = 0.05;

static int cluster_graph(int64_t n, int64_t nnz, const int32_t* d_rowptr, const int32_t* d_col, const PlanOptions& opt,
                         hipStream_t st, int32_t** d_label_out, double* intra_share_out) {
  *d_label_out = nullptr;
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
  int32_t* d_size = nullptr;
  struct SizeGuard {
    int32_t** q;
    ~SizeGuard() {
      if (*q) (void)hipFree(*q);
    }
  } size_guard{&d_size};
  if (hipMalloc(&d_label, (size_t)n * sizeof(int32_t)) != hipSuccess ||
      hipMalloc(&d_label_next, (size_t)n * sizeof(int32_t)) != hipSuccess ||
      hipMalloc(&d_size, (size_t)n * sizeof(int32_t)) != hipSuccess ||
      hipMalloc(&d_changed, hpspmm::kClusterCounters * sizeof(uint32_t)) != hipSuccess) {
    (void)hipGetLastError();
    return HPSPMM_OK;  // no room: no labels, the plan stays what it was
  }
  std::vector<uint32_t> counters((size_t)hpspmm::kClusterCounters);
  hipLaunchKernelGGL(hpspmm::cluster_init_kernel, dim3((unsigned)ceil_div(n, hpspmm::kBlock)), dim3(hpspmm::kBlock),
                     0, st, n, d_label);
  const int max_sweeps = opt.cluster_sweeps > 0 ? opt.cluster_sweeps : kClusterMaxSweeps;
  const bool debug = opt.report;
  // share of the entries that stay inside a cluster small enough for a workgroup's window, from
  // every 4th vertex when there are a million of them (a threshold decision: 1.4 -> 0.4 ms at 2.4 M rows)
  const int64_t score_stride = n >= ((int64_t)1 << 20) ? 4 : 1;
  auto intra_share = [&](double* share) -> int {
    hipError_t e = hipMemsetAsync(d_size, 0, (size_t)n * sizeof(int32_t), st);
    if (e == hipSuccess) e = hipMemsetAsync(d_changed, 0, counters.size() * sizeof(uint32_t), st);
    if (e == hipSuccess) {
      hipLaunchKernelGGL(hpspmm::label_sizes_kernel, dim3((unsigned)ceil_div(n, hpspmm::kBlock)), dim3(hpspmm::kBlock),
                         0, st, n, d_label, d_size);
      hipLaunchKernelGGL(hpspmm::cluster_intra_kernel,
                         dim3((unsigned)ceil_div(ceil_div(n, score_stride), hpspmm::kWavesPerBlock)),
                         dim3(hpspmm::kBlock), 0, st, n, score_stride, d_rowptr, d_col, d_label, d_size,
                         kClusterMaxSize, d_changed);
      e = hipMemcpyAsync(counters.data(), d_changed, counters.size() * sizeof(uint32_t), hipMemcpyDeviceToHost, st);
    }
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    if (e != hipSuccess) return fail(HPSPMM_ERR_HIP, "cluster scoring failed: %s", hipGetErrorString(e));
    int64_t intra = 0;
    for (uint32_t c : counters) intra += c;
    intra *= score_stride;
    *share = nnz > 0 ? (double)intra / (double)nnz : 0.0;
    return HPSPMM_OK;
  };
  for (int sweep = 0; sweep < max_sweeps; ++sweep) {
    HPSPMM_HIP(hipMemsetAsync(d_changed, 0, counters.size() * sizeof(uint32_t), st));
    hipLaunchKernelGGL(hpspmm::cluster_sweep_kernel,
                       dim3((unsigned)ceil_div(ceil_div(n, 2), hpspmm::kWavesPerBlock * 2 * hpspmm::kClusterRowsPerHalf)),
                       dim3(hpspmm::kBlock), 0, st, n, d_rowptr, d_col, d_label, d_label_next, (uint32_t)sweep,
                       d_changed);
    std::swap(d_label, d_label_next);
    HPSPMM_HIP(hipMemcpyAsync(counters.data(), d_changed, counters.size() * sizeof(uint32_t), hipMemcpyDeviceToHost,
                              st));
    HPSPMM_HIP(hipStreamSynchronize(st));
    int64_t changed = 0;
    for (uint32_t c : counters) changed += c;
    if (debug) fprintf(stderr, "cluster sweep %d: %lld of %lld vertices changed their label\n", sweep, (long long)changed, (long long)n);
    if (changed * 200 < n) break;
    if (debug || sweep + 1 == kClusterLookSweeps) {
      // a look on the way: where no clusters are forming by now, none will
      double so_far = 0.0;
      if (int rc = intra_share(&so_far)) return rc;
      if (debug) fprintf(stderr, "cluster: %.4f of the entries inside small clusters after sweep %d\n", so_far, sweep);
      if (sweep + 1 == kClusterLookSweeps && so_far < kClusterLookMinIntra && opt.cluster_sweeps <= 0) break;
    }
  }
  if (int rc = intra_share(intra_share_out)) return rc;
  if (debug) fprintf(stderr, "cluster: %.4f of the entries inside clusters of at most %d vertices\n", *intra_share_out, kClusterMaxSize);
  *d_label_out = d_label;
  d_label = nullptr;  // (the guard keeps what is still named here)
  return HPSPMM_OK;
}

// Finds a processing order for the rows by label propagation: rows of one label next to each other,
// labels in increasing order, rows of a label in increasing order.  A square matrix is taken as a
// graph on its rows (row r adjacent to the rows whose numbers are its column indices); any other
// as the bipartite graph of its rows and columns, whose column side (the transposed pattern) is
// built here by a stable sort of the nonzeros by column.  d_order_out receives a device array of
// `rows` entries (caller frees); no order (NULL, status OK) when the temporaries do not fit.
int cluster_rows(hpspmm_plan* p, const int32_t* d_rowptr, const int32_t* d_col, const PlanOptions& opt,
                 hipStream_t st, int32_t** d_order_out, double* intra_share_out) {
  const int64_t rows = p->rows, cols = p->cols, nnz = p->nnz;
  *d_order_out = nullptr;
  *intra_share_out = 0.0;
  int32_t* d_label = nullptr;
  struct Guard {
    int32_t** q;
    ~Guard() {
      if (*q) (void)hipFree(*q);
    }
  } guard{&d_label};
  if (rows == cols) {
    if (int rc = cluster_graph(rows, nnz, d_rowptr, d_col, opt, st, &d_label, intra_share_out)) return rc;
  } else {
    const int64_t n = rows + cols;
    if (n >= ((int64_t)1 << 31) - 1 || 2 * nnz >= ((int64_t)1 << 31) - hpspmm::kSortTile) return HPSPMM_OK;
    if (int rc = ensure_row_expansion(p, d_rowptr, st)) return rc;
    DeviceTemps tmp;
    const int64_t sort_tiles = ceil_div(nnz, sort_tile());
    uint32_t* keys[2] = {nullptr, nullptr};
    int32_t* vals[2] = {nullptr, nullptr};
    uint32_t *d_hist = nullptr, *d_sscan = nullptr;
    int32_t *d_rowptr2 = nullptr, *d_col2 = nullptr;
    if (tmp.alloc(&keys[0], (size_t)nnz) || tmp.alloc(&keys[1], (size_t)nnz) || tmp.alloc(&vals[0], (size_t)nnz) ||
        tmp.alloc(&vals[1], (size_t)nnz) || tmp.alloc(&d_hist, (size_t)(256 * sort_tiles + 1)) ||
        tmp.alloc(&d_sscan, (size_t)scan_scratch_words(256 * sort_tiles)) || tmp.alloc(&d_rowptr2, (size_t)n + 1) ||
        tmp.alloc(&d_col2, (size_t)(2 * nnz)))
      return HPSPMM_OK;  // no room: no order
    // the nonzeros by column (stable: the rows of a column in increasing order)
    HPSPMM_HIP(hipMemcpyAsync(keys[0], d_col, (size_t)nnz * sizeof(int32_t), hipMemcpyDeviceToDevice, st));
    HPSPMM_HIP(hipMemcpyAsync(vals[0], p->d_nnz_row, (size_t)nnz * sizeof(int32_t), hipMemcpyDeviceToDevice, st));
    int col_bits = 1;
    while (col_bits < 32 && ((int64_t)1 << col_bits) < cols) ++col_bits;
    int cur = 0;
    if (int rc = radix_sort_pairs(nnz, keys, vals, d_hist, d_sscan, col_bits, st, &cur)) return rc;
    // (radix_sort_pairs leaves the sorted keys beside the sorted values)
    const unsigned grid = (unsigned)ceil_div(nnz, hpspmm::kBlock);
    HPSPMM_HIP(hipMemcpyAsync(d_rowptr2, d_rowptr, (size_t)rows * sizeof(int32_t), hipMemcpyDeviceToDevice, st));
    hipLaunchKernelGGL(hpspmm::bipartite_colptr_kernel, dim3((unsigned)ceil_div(cols + 1, hpspmm::kBlock)),
                       dim3(hpspmm::kBlock), 0, st, nnz, keys[cur], cols, (int32_t)nnz, d_rowptr2 + rows);
    hipLaunchKernelGGL(hpspmm::bipartite_shift_kernel, dim3(grid), dim3(hpspmm::kBlock), 0, st, nnz, d_col, (int32_t)rows,
                       d_col2);
    HPSPMM_HIP(hipMemcpyAsync(d_col2 + nnz, vals[cur], (size_t)nnz * sizeof(int32_t), hipMemcpyDeviceToDevice, st));
    if (int rc = cluster_graph(n, 2 * nnz, d_rowptr2, d_col2, opt, st, &d_label, intra_share_out)) return rc;
  }
  // rows ordered by label, the rows of a label in increasing order: a stable sort, hence the same
  // order on every run (the labels of the column vertices, behind those of the rows, are not looked at)
  if (!d_label) return HPSPMM_OK;
  int32_t* d_order = nullptr;
  if (int rc = sort_rows_by_label(rows, d_label, rows == cols ? rows : rows + cols, st, &d_order)) return rc;
  *d_order_out = d_order;
  return HPSPMM_OK;
}

}  // namespace hpspmm_host
