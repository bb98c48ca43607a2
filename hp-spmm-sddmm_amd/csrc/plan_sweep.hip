// Sweep strategy: construction of the layout.
#include "host.hpp"

#include "rank_kernels.hpp"
#include "routed_plan_kernels.hpp"

namespace hpspmm_host {

namespace {

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
// picoseconds per nonzero and microseconds per band and window at K = 32 / 64 / 128
constexpr double kSweepPsPerNnz[3] = {6.5, 8.8, 13.4}, kSweepUsPerWindow[3] = {1.44, 1.72, 1.36};
constexpr int64_t kSweepMinNnz = (int64_t)1 << 21;
constexpr int64_t kSweepMinBBytes = (int64_t)5 << 20;  // social graph: 6 MB of B, sweep 103 / 127 us against 123 / 141; 3 MB: 90 / 65 against 87 / 63

// Gives back what an abandoned attempt at the sweep layout has allocated in the plan so far.
void drop_sweep_buffers(hpspmm_plan* p) {
  for (void** q : {(void**)&p->d_sw_part_base, (void**)&p->d_sw_base, (void**)&p->d_sw_len, (void**)&p->d_sw_ends,
                   (void**)&p->d_sw_slot_row, (void**)&p->d_vcol, (void**)&p->d_vsrc, (void**)&p->d_partial,
                   (void**)&p->d_sw_split_rows, (void**)&p->d_zero_rows, (void**)&p->d_sw_zrow}) {
    if (*q) (void)hipFree(*q);
    *q = nullptr;
  }
}

}  // namespace

// Builds the sweep layout on top of a segments plan.  Returns HPSPMM_OK
// with p->strategy left at SEGMENTS when the matrix does not qualify, cannot be laid out this way, or
// the device has no room for the temporaries of the construction.  Diagnostics: the sweep_* fields of
// hpspmm_plan_options (bytes of B per window, lead, spin limit, nonzeros per piece, priorities)
// override the defaults.
int build_sweep(hpspmm_plan* p, const int32_t* d_rowptr, const int32_t* d_col, bool forced, double other_us,
                const PlanOptions& opt, hipStream_t st) {
  const int64_t rows = p->rows, nnz = p->nnz, k = p->k;
  if (nnz <= 0) return HPSPMM_OK;
  // gather offsets are 32-bit, stream entries keep the column in 24 bits
  if (p->cols * p->k_full * 4 >= ((int64_t)1 << 32) || p->cols > ((int64_t)1 << hpspmm::kSweepColBits)) return HPSPMM_OK;
  if (!forced && (nnz < kSweepMinNnz || p->cols * k * 4 < kSweepMinBBytes)) return HPSPMM_OK;
  const int P = (int)(64 / (k / 4));
  const int WS = P * hpspmm::kSweepSlots;
  const int wpb = sweep_waves_for(k);

  // one workgroup fills a CU, and a band fills the device exactly: every CU then runs the same
  // load (a CU with less runs its wavefronts faster, and they leave the others behind)
  int per_cu = 0;
  if (int rc = sweep_prepare_kernels(k, &per_cu)) return rc;
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
  const int32_t limit = std::max(1, std::min<int>(opt.sweep_limit > 0 ? opt.sweep_limit : (int)limit64, kSweepMaxLimit));

  const int wlog2 = opt.sweep_window_log2 > 0 ? opt.sweep_window_log2 : kSweepWindowLog2;
  int wshift = 0;  // log2 of the columns per window
  while (wshift < 30 && (((int64_t)1 << (wshift + 1)) * k * 4) <= ((int64_t)1 << wlog2)) ++wshift;
  const int64_t n_windows = ceil_div(p->cols, (int64_t)1 << wshift);
  if (n_windows > kSweepMaxWindows) return HPSPMM_OK;
  // What a sweep takes: every gather hits, and every band walks all the windows at the pace of the
  // slowest wavefront.  Over matrices of 25 to 200 uniformly placed nonzeros per row, 30k to 500k rows
  // and columns, square and 16 : 1 either way: 6.5 / 8.8 / 13.4 ps per nonzero and 1.44 / 1.72 / 1.36 us
  // per band and window at K = 32 / 64 / 128, within 25 % everywhere and 10 % rms.  Chosen where
  // that is below `other_us` (a share of what whole rows are expected to take in stored order).  Every
  // non-empty row is at least one piece: the first test rules the layout out for most matrices before
  // any kernel has run.
  const int ki = k == 32 ? 0 : k == 64 ? 1 : 2;
  auto expected_us = [&](int64_t bands) {
    return kSweepPsPerNnz[ki] * (double)nnz * 1e-6 + kSweepUsPerWindow[ki] * (double)(bands * n_windows);
  };
  if (!forced && (other_us <= 0 || expected_us(ceil_div(nonempty, band_waves * WS)) > other_us)) return HPSPMM_OK;
  DeviceTemps tmp;
  // A row must meet the windows in the order of its entries.  Where the columns of the rows are not
  // stored in increasing order the layout is built from a copy in which they are (two stable radix
  // sorts of the nonzeros: by column, then by row), and the value indices of the streams lead back
  // to where the caller has every entry.
  const int32_t* d_stored_at = nullptr;
  if (!columns_sorted(p, d_rowptr, d_col, st)) {
    if (nnz >= ((int64_t)1 << 31) - hpspmm::kSortTile) return HPSPMM_OK;
    if (int rc = ensure_row_expansion(p, d_rowptr, st)) return rc;
    const int64_t sort_tiles = ceil_div(nnz, sort_tile());
    uint32_t* keys[2] = {nullptr, nullptr};
    int32_t* vals[2] = {nullptr, nullptr};
    uint32_t *d_hist = nullptr, *d_sscan = nullptr;
    int32_t* d_scol = nullptr;
    if (tmp.alloc(&keys[0], (size_t)nnz) || tmp.alloc(&keys[1], (size_t)nnz) || tmp.alloc(&vals[0], (size_t)nnz) ||
        tmp.alloc(&vals[1], (size_t)nnz) || tmp.alloc(&d_hist, (size_t)(256 * sort_tiles + 1)) ||
        tmp.alloc(&d_sscan, (size_t)scan_scratch_words(256 * sort_tiles)) || tmp.alloc(&d_scol, (size_t)nnz))
      return HPSPMM_OK;  // no room: the plan stays what it was
    const dim3 g(grid_for(nnz, 1 << 16)), b(hpspmm::kBlock);
    int col_bits = 1, row_bits = 1;
    while (col_bits < 32 && ((int64_t)1 << col_bits) < p->cols) ++col_bits;
    while (row_bits < 32 && ((int64_t)1 << row_bits) < rows) ++row_bits;
    int cur = 0;
    hipLaunchKernelGGL(hpspmm::sweep_sort_keys_kernel, g, b, 0, st, nnz, d_col, (const int32_t*)nullptr, keys[0], vals[0]);
    if (int rc = radix_sort_pairs(nnz, keys, vals, d_hist, d_sscan, col_bits, st, &cur)) return rc;
    if (cur != 0) std::swap(keys[0], keys[1]), std::swap(vals[0], vals[1]);
    hipLaunchKernelGGL(hpspmm::sweep_sort_keys_kernel, g, b, 0, st, nnz, p->d_nnz_row, (const int32_t*)vals[0], keys[0],
                       (int32_t*)nullptr);
    if (int rc = radix_sort_pairs(nnz, keys, vals, d_hist, d_sscan, row_bits, st, &cur)) return rc;
    // the columns in that order
    hipLaunchKernelGGL(hpspmm::sweep_sort_keys_kernel, g, b, 0, st, nnz, d_col, (const int32_t*)vals[cur],
                       reinterpret_cast<uint32_t*>(d_scol), (int32_t*)nullptr);
    d_stored_at = vals[cur];
    d_col = d_scol;
  }

  // pieces per row, their scans
  uint32_t *d_pbase = nullptr, *d_part = nullptr, *d_scan0 = nullptr;
  // (no room for a temporary or a buffer of the layout: the plan stays what it was, like any other
  // matrix that cannot be laid out this way)
  if (tmp.alloc(&d_pbase, (size_t)rows + 1 + (size_t)scan_scratch_words(rows + 1)) != HPSPMM_OK) return HPSPMM_OK;
  d_scan0 = d_pbase + rows + 1;
  if (hipMalloc(&p->d_sw_part_base, (size_t)(rows + 1) * sizeof(uint32_t)) != hipSuccess) {
    (void)hipGetLastError();
    p->d_sw_part_base = nullptr;
    return HPSPMM_OK;
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
  // (the same test with the bands there really are: long rows are several pieces)
  if (n_bands > kSweepMaxBands || (!forced && expected_us(n_bands) > other_us)) {
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
  // Where every row enters every window and where every slot's runs lie are tables of rows x windows
  // and slots x windows words: a few words per nonzero on a matrix the layout suits, tens of gigabytes
  // on one of millions of short rows (which only a forcing flag brings this far): 2 GiB + 64 bytes per
  // nonzero is the most they may take.
  if ((int64_t)rows * (n_windows + 1) + n_slots * n_windows > 16 * nnz + ((int64_t)1 << 29) || tmp.reserve() != HPSPMM_OK) {
    drop_sweep_buffers(p);
    return HPSPMM_OK;
  }
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
    drop_sweep_buffers(p);
    return HPSPMM_OK;
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
    (void)hipStreamSynchronize(st);  // kernels of this attempt may still be reading its temporaries
    drop_sweep_buffers(p);
    return HPSPMM_OK;
  }
  hipLaunchKernelGGL(hpspmm::sweep_clear_stream_kernel, dim3(grid_for(total, 1 << 16)), dim3(hpspmm::kBlock), 0, st, total,
                     p->d_vcol, p->d_vsrc);
  hipLaunchKernelGGL(hpspmm::sweep_fill_kernel, wave_grid, dim3(hpspmm::kBlock), 0, st, (int32_t)n_windows, wshift, limit,
                     (int32_t)WS, (int32_t)(k / 4), d_piece_of, d_piece_row, d_pbase, d_rowptr, d_col, d_wstart, d_run_at,
                     p->d_sw_ends, p->d_sw_base, p->d_sw_len, d_stored_at, p->d_vcol, p->d_vsrc);
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
  p->sw.lead = std::max(1, opt.sweep_lead > 0 ? opt.sweep_lead : sweep_lead(k));
  p->sw.spin_limit = opt.sweep_spin >= 0 ? opt.sweep_spin : kSweepSpinLimit;
  p->sw.priorities = opt.sweep_priorities >= 0 ? opt.sweep_priorities : 1;
  if (opt.report)
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

}  // namespace hpspmm_host
