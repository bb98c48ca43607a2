// Plan-time kernels of the routed strategy (classes, chunks, run tables, the class-major fill) and
// the device-wide scan they and the other layouts use.
#pragma once

#include "routed_kernels.hpp"

namespace hpspmm {

// ---- plan-time kernels -----------------------------------------------------

// Hub class of a nonzero in column c: mapped = colmap[c] is the compact-buffer
// row of a cached column or -1.  A cached column of popularity rank s sits in
// compact-buffer row (s % 8) * hub_rows_per_slice + s / 8 and belongs to slice
// s % 8, phase (s / 8) % nsub, so that every (slice, phase) gets the same mix
// of hot and cold columns; the other columns are spread by a multiplicative hash.
__device__ __forceinline__ int hub_class_of(int32_t c, int32_t mapped, int32_t hub_rows_per_slice, int nsub) {
  int slice, sub;
  if (mapped >= 0) {
    slice = mapped / hub_rows_per_slice;
    sub = (mapped - slice * hub_rows_per_slice) % nsub;
  } else {
    const uint32_t h = (uint32_t)c * 0x9E3779B1u;
    slice = (int)(h >> 29);
    sub = (int)((((h >> 13) & 0xFFFFu) * (uint32_t)nsub) >> 16);
  }
  return sub * kSlices + slice;
}

// The same when the plan has cut the columns into 8 * nsub consecutive ranges of equal nonzero count
// instead (colrange[c] = range of column c; slice = range / nsub, phase = range % nsub): in a row
// with sorted columns the nonzeros of one class are then consecutive, so the values can be read
// where the caller keeps them.  `single` = the row keeps everything in phase 0.
__device__ __forceinline__ int range_class_of(int range, int nsub, bool single) {
  const int slice = range / nsub;
  return single ? slice : (range - slice * nsub) * kSlices + slice;
}

// A routed row shorter than this many times the routing threshold keeps all its nonzeros in phase 0
// (one partial-result row per slice instead of one per slice and phase; 233k-vertex social graph,
// K = 128: 3.77 -> 3.70 ms with 2, no further gain with 4, where R-MAT loses 0.1 ms).
constexpr int kSinglePhaseFactor = 2;

// *flag |= 1 if some row has a column index smaller than the one before it (row[] = row of every nonzero).
HPSPMM_KERNEL __launch_bounds__(kBlock) void columns_unsorted_kernel(int64_t nnz, const int32_t* __restrict__ row,
                                                                  const int32_t* __restrict__ col,
                                                                  int32_t* __restrict__ flag) {
  bool bad = false;
  for (int64_t j = (int64_t)blockIdx.x * kBlock + threadIdx.x; j + 1 < nnz; j += (int64_t)gridDim.x * kBlock)
    bad |= row[j] == row[j + 1] && col[j] > col[j + 1];
  if (__ballot(bad) != 0 && (threadIdx.x & 63) == 0) atomicOr(flag, 1);
}

// flag[r] = 1 if row r is routed (r < rows), flag[rows] = 0.
HPSPMM_KERNEL __launch_bounds__(kBlock) void routed_flag_kernel(int64_t rows, const int32_t* __restrict__ rowptr,
                                                             int32_t min_row_nnz, uint32_t* __restrict__ flag) {
  const int64_t r = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (r > rows) return;
  flag[r] = r < rows && rowptr[r + 1] - rowptr[r] >= min_row_nnz ? 1u : 0u;
}

// routed_rows[ridx[r]] = r for every routed row (ridx = exclusive scan of the routed flags).
HPSPMM_KERNEL __launch_bounds__(kBlock) void routed_list_kernel(int64_t rows, const int32_t* __restrict__ rowptr,
                                                             int32_t min_row_nnz, const uint32_t* __restrict__ ridx,
                                                             int32_t* __restrict__ routed_rows) {
  const int64_t r = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (r < rows && rowptr[r + 1] - rowptr[r] >= min_row_nnz) routed_rows[ridx[r]] = (int32_t)r;
}

// coldcnt[r] = nonzeros of row r if it is a short row, else 0 (r < rows); coldcnt[rows] = 0 (the
// scan's total slot).  One thread per row: most rows of a large skewed matrix are short or empty.
HPSPMM_KERNEL __launch_bounds__(kBlock) void routed_cold_count_kernel(int64_t rows, const int32_t* __restrict__ rowptr,
                                                                   int32_t min_row_nnz,
                                                                   uint32_t* __restrict__ coldcnt) {
  const int64_t r = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (r > rows) return;
  uint32_t n = 0;
  if (r < rows) {
    const int32_t len = rowptr[r + 1] - rowptr[r];
    if (len < min_row_nnz) n = (uint32_t)len;
  }
  coldcnt[r] = n;
}

// The routed rows are counted and laid out in chunks of kRoutedChunk consecutive nonzeros, one
// wavefront each: a hub row of 10^5 nonzeros on a single wavefront was the critical path of the
// whole plan.  nch[i] = chunks of routed row i (nch[n_routed] = 0: the scan's total slot).
constexpr int kRoutedChunk = 4096;

HPSPMM_KERNEL __launch_bounds__(kBlock) void routed_row_chunks_kernel(int64_t n_routed,
                                                                   const int32_t* __restrict__ routed_rows,
                                                                   const int32_t* __restrict__ rowptr,
                                                                   uint32_t* __restrict__ nch) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i > n_routed) return;
  uint32_t n = 0;
  if (i < n_routed) {
    const int32_t row = routed_rows[i];
    n = (uint32_t)((rowptr[row + 1] - rowptr[row] + kRoutedChunk - 1) / kRoutedChunk);
  }
  nch[i] = n;
}

// chunk_row[c] = routed-row number of chunk c (chunk_base = exclusive scan of nch).
HPSPMM_KERNEL __launch_bounds__(kBlock) void routed_chunk_rows_kernel(int64_t n_routed,
                                                                   const uint32_t* __restrict__ chunk_base,
                                                                   int32_t* __restrict__ chunk_row) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= n_routed) return;
  for (uint32_t c = chunk_base[i]; c < chunk_base[i + 1]; ++c) chunk_row[c] = (int32_t)i;
}

// Bounds of chunk c: nonzeros [lb, hb) of routed row number i; `single` = the row keeps everything in phase 0.
struct RoutedChunk {
  int32_t i, lb, hb;
  bool single;
};
__device__ __forceinline__ RoutedChunk routed_chunk(int64_t c, const int32_t* __restrict__ chunk_row,
                                                    const uint32_t* __restrict__ chunk_base,
                                                    const int32_t* __restrict__ routed_rows,
                                                    const int32_t* __restrict__ rowptr, int32_t min_row_nnz) {
  RoutedChunk k;
  k.i = chunk_row[c];
  const int32_t row = routed_rows[k.i];
  const int32_t row_lb = rowptr[row], row_hb = rowptr[row + 1];
  k.lb = row_lb + (int32_t)(c - chunk_base[k.i]) * kRoutedChunk;
  k.hb = k.lb + kRoutedChunk < row_hb ? k.lb + kRoutedChunk : row_hb;
  k.single = row_hb - row_lb < kSinglePhaseFactor * min_row_nnz;
  return k;
}

// One wavefront per chunk: cnt[x * n_chunks + c] = its nonzeros in hub class x.
// cnt[nhub * n_chunks] = 0 (the scan's total slot) is written by the first wavefront.
HPSPMM_KERNEL __launch_bounds__(kBlock) void routed_count_kernel(int64_t n_chunks, const int32_t* __restrict__ chunk_row,
                                                              const uint32_t* __restrict__ chunk_base,
                                                              const int32_t* __restrict__ routed_rows,
                                                              const int32_t* __restrict__ rowptr,
                                                              const int32_t* __restrict__ col,
                                                              const int32_t* __restrict__ colmap,
                                                              int32_t hub_rows_per_slice, int nsub,
                                                              const uint8_t* __restrict__ colrange,
                                                              int32_t min_row_nnz, uint32_t* __restrict__ cnt) {
  const int lane = threadIdx.x & 63;
  const int64_t c = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  const int nhub = kSlices * nsub;
  if (c == 0 && lane == 0) cnt[(int64_t)nhub * n_chunks] = 0;
  if (c >= n_chunks) return;
  const RoutedChunk ch = routed_chunk(c, chunk_row, chunk_base, routed_rows, rowptr, min_row_nnz);
  uint32_t mine = 0;  // lane x < nhub accumulates the count of class x
  for (int32_t j0 = ch.lb; j0 < ch.hb; j0 += 64) {
    const int32_t j = j0 + lane;
    int cls = -1;
    if (j < ch.hb) {
      const int32_t cc = col[j];
      cls = colrange ? range_class_of(colrange[cc], nsub, ch.single)
                     : hub_class_of(cc, colmap[cc], hub_rows_per_slice, ch.single ? 1 : nsub);
    }
    for (int x = 0; x < nhub; ++x) {
      const uint64_t m = __ballot(cls == x);
      if (lane == x) mine += (uint32_t)__popcll(m);
    }
  }
  if (lane < nhub) cnt[(int64_t)lane * n_chunks + c] = mine;
}

// Class of the class-major position q, or -1 for the padding between the classes.
__device__ __forceinline__ int routed_class_of_position(const RoutedLayout& lay, int64_t q) {
  for (int x = 0; x <= lay.nhub; ++x)
    if (q >= lay.cls_begin[x] && q < lay.cls_end[x]) return x;
  return -1;
}

// flag[q] = 1 if position q holds the first entry of a run (q < vtotal), flag[vtotal] = 0 (the
// scan's total slot).  vrow[q] = routed-row number (hub classes) or row (cold class) of the entry.
HPSPMM_KERNEL __launch_bounds__(kBlock) void routed_run_flags_kernel(RoutedLayout lay, int64_t vtotal,
                                                                     const int32_t* __restrict__ vrow,
                                                                     uint32_t* __restrict__ flag) {
  for (int64_t q = (int64_t)blockIdx.x * kBlock + threadIdx.x; q <= vtotal; q += (int64_t)gridDim.x * kBlock) {
    uint32_t f = 0;
    if (q < vtotal) {
      const int x = routed_class_of_position(lay, q);
      if (x >= 0) f = q == lay.cls_begin[x] || vrow[q] != vrow[q - 1];
    }
    flag[q] = f;
  }
}

// before[q] = run starts before position q (the exclusive scan of flag).  Every entry word gets its
// final form (see kRunStart); run_row[r] = row of run r; seg_run[g] = run of the first entry of
// segment g (segments that begin in the padding between classes are never read).
HPSPMM_KERNEL __launch_bounds__(kBlock) void routed_runs_kernel(RoutedLayout lay, int64_t vtotal,
                                                                const uint32_t* __restrict__ flag,
                                                                const uint32_t* __restrict__ before,
                                                                const int32_t* __restrict__ vrow,
                                                                int32_t* __restrict__ vent,
                                                                int32_t* __restrict__ run_row,
                                                                int32_t* __restrict__ seg_run) {
  for (int64_t q = (int64_t)blockIdx.x * kBlock + threadIdx.x; q < vtotal; q += (int64_t)gridDim.x * kBlock) {
    const uint32_t f = flag[q];
    const int32_t w = vent[q];  // column, or ~slot
    const bool hot = w < 0;
    const int x = routed_class_of_position(lay, q);
    int32_t payload = hot ? ~w : w;
    bool in_lds = false;
    if (hot && x >= 0 && lay.lds_rows > 0) {
      const int64_t h = lay.hub_rows_per_slice;
      const int64_t slice = payload / h, place = payload - slice * h;
      if (x < lay.nhub) {
        in_lds = slice == x && place < lay.lds_rows;
        if (in_lds) payload = (int32_t)place;
      } else {
        const int per = lay.lds_rows / kSlices;
        in_lds = place < per;
        if (in_lds) payload = (int32_t)(slice * per + place);
      }
    }
    vent[q] = (hot ? INT32_MIN : 0) | (in_lds ? kInLds : 0) | (payload & kEntryPayload) | (f ? kRunStart : 0);
    if (f) run_row[before[q]] = vrow[q];
    if ((q & (((int64_t)1 << lay.shift) - 1)) == 0 && x >= 0)
      seg_run[q >> lay.shift] = (int32_t)(before[q] + f) - 1;
  }
}

// rvptr[r * nhub + x] = virtual index of the first class-x nonzero of routed
// row number r (r = n_routed: one past the class), from the exclusive scan of
// the class-major chunk counts (scanned[x * n_chunks + c]) and the padded class
// origins.  The end of the (r, x) run is rvptr[(r + 1) * nhub + x].
HPSPMM_KERNEL __launch_bounds__(kBlock) void routed_vptr_kernel(RoutedLayout lay, int64_t n_chunks,
                                                             const uint32_t* __restrict__ chunk_base,
                                                             const uint32_t* __restrict__ scanned,
                                                             int32_t* __restrict__ rvptr) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= (lay.n_routed + 1) * lay.nhub) return;
  const int64_t r = i / lay.nhub;
  const int x = (int)(i - r * lay.nhub);
  const int64_t local = (int64_t)scanned[(int64_t)x * n_chunks + chunk_base[r]] - (int64_t)scanned[(int64_t)x * n_chunks];
  rvptr[i] = (int32_t)(lay.cls_begin[x] + local);
}

// coldptr[r] = virtual index of the first cold-class nonzero of row r (r = rows: one past the class).
HPSPMM_KERNEL __launch_bounds__(kBlock) void routed_coldptr_kernel(int64_t rows, int64_t cold_begin,
                                                                const uint32_t* __restrict__ scanned,
                                                                int32_t* __restrict__ coldptr) {
  const int64_t r = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (r > rows) return;
  coldptr[r] = (int32_t)(cold_begin + (int64_t)scanned[r]);
}

// Scatter the nonzeros of the routed rows into class-major order, keeping the stored order inside
// every run.  One wavefront per chunk (its first slot in class x follows from the scan of the chunk
// counts); positions within the chunk from ballots.
HPSPMM_KERNEL __launch_bounds__(kBlock) void routed_fill_kernel(RoutedLayout lay, int64_t n_chunks,
                                                             const int32_t* __restrict__ chunk_row,
                                                             const uint32_t* __restrict__ chunk_base,
                                                             const uint32_t* __restrict__ scanned,
                                                             const int32_t* __restrict__ routed_rows,
                                                             const int32_t* __restrict__ rowptr,
                                                             const int32_t* __restrict__ col,
                                                             const int32_t* __restrict__ colmap,
                                                             int32_t hub_rows_per_slice,
                                                             const uint8_t* __restrict__ colrange,
                                                             int32_t min_row_nnz,
                                                             int32_t* __restrict__ vcol, int32_t* __restrict__ vpos,
                                                             int32_t* __restrict__ vsrc /* or NULL */,
                                                             int32_t* __restrict__ vrow) {
  const int lane = threadIdx.x & 63;
  const int64_t c = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  if (c >= n_chunks) return;
  const int nsub = lay.nsub;
  const int nhub = lay.nhub;
  const RoutedChunk ch = routed_chunk(c, chunk_row, chunk_base, routed_rows, rowptr, min_row_nnz);
  int32_t cursor = 0;  // lane x: next slot of class x
  if (lane < nhub)
    cursor = (int32_t)(lay.cls_begin[lane] + (int64_t)scanned[(int64_t)lane * n_chunks + c] -
                       (int64_t)scanned[(int64_t)lane * n_chunks]);
  const uint64_t below = (1ull << lane) - 1ull;
  for (int32_t j0 = ch.lb; j0 < ch.hb; j0 += 64) {
    const int32_t j = j0 + lane;
    const bool valid = j < ch.hb;
    const int32_t cc = valid ? col[j] : 0;
    const int32_t mapped = valid ? colmap[cc] : -1;
    const int cls = !valid      ? -1
                    : colrange ? range_class_of(colrange[cc], nsub, ch.single)
                               : hub_class_of(cc, mapped, hub_rows_per_slice, ch.single ? 1 : nsub);
    for (int x = 0; x < nhub; ++x) {
      const uint64_t m = __ballot(cls == x);
      if (m == 0) continue;
      const int32_t start = __shfl(cursor, x);
      if (cls == x) {
        const int32_t pos = start + (int32_t)__popcll(m & below);
        vcol[pos] = mapped >= 0 ? ~mapped : cc;
        vpos[j] = pos;
        if (vsrc) vsrc[pos] = j;
        vrow[pos] = ch.i;
      }
      if (lane == x) cursor += (int32_t)__popcll(m);
    }
  }
}

// The nonzeros of the short rows go to the cold class in stored order.  One thread per nonzero
// (nnz_row[j] = its row): a wavefront per row would idle on the millions of rows of a few nonzeros.
HPSPMM_KERNEL __launch_bounds__(kBlock) void routed_fill_cold_kernel(int64_t nnz, const int32_t* __restrict__ nnz_row,
                                                                  const int32_t* __restrict__ rowptr,
                                                                  const int32_t* __restrict__ col,
                                                                  const int32_t* __restrict__ colmap,
                                                                  int32_t min_row_nnz,
                                                                  const int32_t* __restrict__ coldptr,
                                                                  int32_t* __restrict__ vcol,
                                                                  int32_t* __restrict__ vpos,
                                                                  int32_t* __restrict__ vsrc /* or NULL */,
                                                                  int32_t* __restrict__ vrow) {
  const int64_t j = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (j >= nnz) return;
  const int32_t row = nnz_row[j];
  const int32_t lb = rowptr[row];
  if (rowptr[row + 1] - lb >= min_row_nnz) return;
  const int32_t c = col[j];
  const int32_t mapped = colmap[c];
  const int32_t pos = coldptr[row] + ((int32_t)j - lb);
  vcol[pos] = mapped >= 0 ? ~mapped : c;  // ~compact-buffer row if the column is cached
  vpos[j] = pos;
  if (vsrc) vsrc[pos] = (int32_t)j;
  vrow[pos] = row;
}

// What the final kernel has to do with every row: nothing (stored by the main kernel, or routed),
// write zeros (no nonzeros), or add carry slots (a short row whose run crosses a segment boundary).
HPSPMM_KERNEL __launch_bounds__(kBlock) void routed_action_kernel(int64_t rows, const int32_t* __restrict__ rowptr,
                                                               int32_t min_row_nnz,
                                                               const int32_t* __restrict__ coldptr, int shift,
                                                               uint8_t* __restrict__ action) {
  const int64_t r = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (r >= rows) return;
  const int32_t len = rowptr[r + 1] - rowptr[r];
  uint8_t a = kActionNone;
  if (len == 0) {
    a = kActionZero;
  } else if (len < min_row_nnz) {
    const int64_t start = coldptr[r];
    if ((start >> shift) != ((start + len - 1) >> shift)) a = kActionCross;
  }
  action[r] = a;
}


HPSPMM_KERNEL __launch_bounds__(kBlock) void routed_chunk_kernel(RoutedLayout lay, int64_t nnz,
                                                              const int32_t* __restrict__ vpos,
                                                              uint16_t* __restrict__ lslot,
                                                              int32_t* __restrict__ chunk_base,
                                                              int32_t* __restrict__ chunk_pref) {
  __shared__ int32_t s_min[kMaxClasses];
  __shared__ int32_t s_cnt[kMaxClasses];
  __shared__ int32_t s_pref[kMaxClasses];
  const int ncls = lay.nhub + 1;
  const int64_t j0 = (int64_t)blockIdx.x * kPermChunk;
  for (int x = threadIdx.x; x < ncls; x += kBlock) {
    s_min[x] = INT32_MAX;
    s_cnt[x] = 0;
  }
  __syncthreads();
  auto class_of_position = [&](int32_t p) {
    int x = 0;
    while (x + 1 < ncls && (int64_t)p >= lay.cls_begin[x + 1]) ++x;
    return x;
  };
  for (int i = threadIdx.x; i < kPermChunk; i += kBlock) {
    const int64_t j = j0 + i;
    if (j >= nnz) break;
    const int32_t p = vpos[j];
    const int x = class_of_position(p);
    atomicMin(&s_min[x], p);
    atomicAdd(&s_cnt[x], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int32_t run = 0;
    for (int x = 0; x < ncls; ++x) {
      s_pref[x] = run;
      run += s_cnt[x];
    }
  }
  __syncthreads();
  for (int x = threadIdx.x; x < ncls; x += kBlock) {
    chunk_base[(int64_t)blockIdx.x * ncls + x] = s_cnt[x] ? s_min[x] : 0;
    chunk_pref[(int64_t)blockIdx.x * ncls + x] = s_pref[x];
  }
  for (int i = threadIdx.x; i < kPermChunk; i += kBlock) {
    const int64_t j = j0 + i;
    if (j >= nnz) break;
    const int32_t p = vpos[j];
    const int x = class_of_position(p);
    lslot[j] = (uint16_t)(s_pref[x] + (p - s_min[x]));
  }
}

}  // namespace hpspmm
