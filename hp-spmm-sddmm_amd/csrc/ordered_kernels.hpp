// gfx950 device code of the *ordered* strategy for FP32 CSR SpMM.
//
// Graphs with community structure reuse rows of B only among the few dozen
// rows of A of one community.  Processing those rows next to each other is not
// enough on this machine: a sub-wave returns to the same row of B one row of A
// later, i.e. after some 50 gathers or ~9 us, and under full-rate streaming an
// L2 of 4 MB is turned over every ~4 us (measured on the 2.4M-vertex
// co-purchase graph with its rows grouped by community: L2 hits rise from 3 %
// to 12 % only).  The ordered strategy therefore makes the reuse explicit:
//
//   * the rows of A are processed in a given order (a permutation of the row
//     numbers, supplied by the caller - the reference's HP-SpMM reads one from
//     a .cugraph_reorder file, spmm/mm/spmm_common.cpp:237-296 - or found by
//     the plan's own clustering); C is written at the original row numbers;
//   * the nonzeros, laid out in that order, are cut into windows of
//     kWavesPerBlock * P segments, one workgroup each.  The plan finds, per
//     window, the columns that occur at least twice in it and gives the most
//     frequent ones a slot in a workgroup-local LDS copy of B (their column
//     index is rewritten as ~slot);
//   * the workgroup first fetches those rows of B into LDS, once, then runs
//     the tile engine of the segments kernel, reading a slotted column from
//     LDS and every other one from memory.
//
// A row's nonzeros keep their stored order, so what the kernel streams is one
// entry word per nonzero - column or LDS slot, and a flag on the first entry of
// every row (kRunStart, as in the routed strategy's column tiles) - and the
// value, read where the caller keeps it: a row's values are contiguous there,
// at the entry's position plus a per-row offset.  Rows and offsets are kept row
// by row (run_row, run_delta).  8 bytes per nonzero; with a column, a source
// index and a row per nonzero it was 16 (co-purchase graph, K = 64: 2.93 -> 2.8 ms).
// A row cut by a segment boundary inside one window is added up by the window's workgroup itself
// (the partial sums wait in registers and meet in LDS once the segments are done); only the rows
// that cross a window boundary go through carry slots in memory as in the segments strategy, and a
// fix-up kernel adds those up from the plan's list of such rows.  The order of the additions is the
// same either way: the part in the row's first segment, then segment after segment.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "routed_kernels.hpp"
#include "spmm_kernels.hpp"

namespace hpspmm {

// ---- plan-time kernels -----------------------------------------------------

// Label propagation, one sweep: every row takes the label that is most frequent
// among (a sample of at most 32 of) its neighbours' labels - the rows whose
// indices are its column indices; the matrix is taken as a graph, which is
// meant for square, structurally symmetric A (the host hands over the
// bipartite graph of rows and columns for any other).  Ties are broken by a hash that
// changes with the sweep, except that a row keeps its label when that is among
// the most frequent.  A sweep reads label_in and writes label_out (two buffers,
// so the outcome does not depend on the order in which the wavefronts run: two
// plans of one matrix get the same labels), and only half of the rows may
// change - of every pair of rows (2w, 2w + 1) the one a hash of w and the sweep
// picks: with every row updated at once from the old labels, neighbours swap
// labels back and forth instead of settling.  Half a wavefront per pair (it
// copies the label of the row that sits the sweep out); the 32 sampled labels
// are sorted by a bitonic network of shuffles within the half.  A sweep is
// bound by the random 4-byte reads of the neighbours' labels: 32 samples a row
// instead of 64 halve them (co-purchase graph, 2.4 M rows of 50 nonzeros: 0.60
// -> 0.37 ms a sweep, 13 sweeps instead of 11 until fewer than 0.5 % of the rows
// change, the SpMM on the resulting order 2.92 -> 2.93 ms).  The
// kClusterCounters entries of changed[] together count the rows whose label changed.
constexpr int kClusterCounters = 1024;
constexpr int kClusterSamples = 32;     // lanes per row
constexpr int kClusterRowsPerHalf = 4;  // pairs a half-wavefront takes, their loads in flight together

// The label that row r takes: lab = the sampled neighbour labels of the lanes of this half of the
// wavefront (INT32_MAX where a lane has none), mine = the row's own.  Same value in every lane of
// the half; every lane of the wavefront must call it.
__device__ __forceinline__ int32_t cluster_vote(int32_t lab, int32_t mine, int64_t r, uint32_t sweep, int hl, int half) {
  const auto half_ballot = [&](bool x) { return (uint32_t)(__ballot(x) >> (32 * half)); };
  const int self_count = __popc(half_ballot(lab == mine));
#pragma unroll
  for (int size = 2; size <= kClusterSamples; size <<= 1) {
#pragma unroll
    for (int j = size >> 1; j > 0; j >>= 1) {
      const int32_t other = __shfl_xor(lab, j);
      const bool up = (hl & size) == 0;
      const bool lower = (hl & j) == 0;
      const int32_t lo = lab < other ? lab : other;
      const int32_t hi = lab < other ? other : lab;
      lab = (lower == up) ? lo : hi;
    }
  }
  const int32_t prev = __shfl_up(lab, 1);
  const bool real = lab != INT32_MAX;
  const bool head = real && (hl == 0 || lab != prev);
  const uint32_t heads = half_ballot(head);
  const int n_real = __popc(half_ballot(real));
  int32_t next_label = mine;
  // (no branch on n_real: it differs between the halves, and the shuffles below need every lane)
  unsigned long long key = 0;
  if (head) {
    const uint32_t later = hl < 31 ? (heads >> (hl + 1)) : 0u;
    const int next = later ? hl + 1 + __ffs((int)later) - 1 : n_real;
    const uint32_t h = ((uint32_t)lab * 0x9E3779B1u) ^ (sweep * 0x85EBCA6Bu) ^ ((uint32_t)r * 0xC2B2AE35u);
    key = ((unsigned long long)(uint32_t)(next - hl) << 32) | (h >> 1);
  }
  unsigned long long best = key;
  int32_t best_lab = lab;
#pragma unroll
  for (int off = kClusterSamples / 2; off > 0; off >>= 1) {
    const unsigned long long o = __shfl_xor(best, off);
    const int32_t ol = __shfl_xor(best_lab, off);
    if (o > best || (o == best && ol < best_lab)) {
      best = o;
      best_lab = ol;
    }
  }
  const int best_count = (int)(best >> 32);
  if (n_real != 0 && self_count < best_count && best_lab != mine) next_label = best_lab;
  return next_label;
}

// A sweep is a chain of three dependent round trips per row (row pointer, columns, labels) and
// little else, so a half-wavefront takes kClusterRowsPerHalf pairs and issues each stage for all of
// them before it needs any of the answers.
HPSPMM_KERNEL __launch_bounds__(kBlock) void cluster_sweep_kernel(int64_t rows, const int32_t* __restrict__ rowptr,
                                                               const int32_t* __restrict__ col,
                                                               const int32_t* __restrict__ label_in,
                                                               int32_t* __restrict__ label_out, uint32_t sweep,
                                                               uint32_t* __restrict__ changed) {
  constexpr int R = kClusterRowsPerHalf;
  const int lane = threadIdx.x & 63;
  const int hl = lane & 31, half = lane >> 5;
  const int64_t w0 = (((int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6)) * 2 + half) * R;
  int64_t r[R];
  bool live[R];
  int32_t mine[R], lb[R], n[R], c[R], lab[R];
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int64_t w = w0 + i;
    live[i] = 2 * w < rows;
    r[i] = 0;
    if (live[i]) {
      const uint32_t turn = (((uint32_t)w * 0x9E3779B1u) ^ ((sweep + 1u) * 0x85EBCA6Bu)) * 0xC2B2AE35u;
      r[i] = 2 * w + (int64_t)((turn >> 31) & 1u) < rows ? 2 * w + (int64_t)((turn >> 31) & 1u) : 2 * w;
      const int64_t idle = r[i] ^ 1;  // the other row of the pair keeps its label in this sweep
      if (hl == 1 && idle < rows) label_out[idle] = label_in[idle];
    }
  }
#pragma unroll
  for (int i = 0; i < R; ++i) {
    mine[i] = live[i] ? label_in[r[i]] : 0;
    lb[i] = live[i] ? rowptr[r[i]] : 0;
    n[i] = live[i] ? rowptr[r[i] + 1] - lb[i] : 0;
  }
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int32_t stride = (n[i] + kClusterSamples - 1) / kClusterSamples;
    c[i] = hl * stride < n[i] ? col[lb[i] + hl * stride] : -1;
  }
#pragma unroll
  // (an entry on the diagonal has no vote: with one, every row of A + I would find its own label among
  // the most frequent ones in the first sweep and keep it, and nothing would ever move)
  for (int i = 0; i < R; ++i)
    lab[i] = (c[i] >= 0 && (int64_t)c[i] < rows && (int64_t)c[i] != r[i]) ? label_in[c[i]] : INT32_MAX;  // sorts behind every label
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int32_t next_label = cluster_vote(lab[i], mine[i], r[i], sweep, hl, half);
    if (live[i] && hl == 0) {
      label_out[r[i]] = next_label;
      if (next_label != mine[i])
        atomicAdd(&changed[r[i] & (kClusterCounters - 1)], 1u);  // spread: one counter would serialise the first sweep
    }
  }
}

// What the labels are worth: counts the nonzeros (r, c) with label[c] == label[r] in clusters of
// at most max_size rows (size[l] = rows carrying label l) - the nonzeros whose row of B a
// workgroup can expect to meet again within its window once the rows are ordered by label.  Hot
// columns also produce reuse inside a window, but that is the routed strategy's and the hub
// cache's business; a graph without communities ends up in one giant cluster or in singletons and
// scores nothing here.  One wavefront per row; intra[] has kClusterCounters entries.
HPSPMM_KERNEL __launch_bounds__(kBlock) void cluster_intra_kernel(int64_t rows, int64_t stride,
                                                               const int32_t* __restrict__ rowptr,
                                                               const int32_t* __restrict__ col,
                                                               const int32_t* __restrict__ label,
                                                               const int32_t* __restrict__ size, int32_t max_size,
                                                               uint32_t* __restrict__ intra) {
  const int lane = threadIdx.x & 63;
  const int64_t r = ((int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6)) * stride;  // every stride-th row
  if (r >= rows) return;
  const int32_t mine = label[r];
  if (size[mine] > max_size) return;
  const int32_t lb = rowptr[r], hb = rowptr[r + 1];
  uint32_t cnt = 0;
  for (int32_t j = lb + lane; j < hb; j += 64) {
    const int32_t c = col[j];
    cnt += ((int64_t)c < rows && label[c] == mine) ? 1u : 0u;
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) cnt += __shfl_xor(cnt, off);
  if (lane == 0 && cnt) atomicAdd(&intra[(r / stride) & (kClusterCounters - 1)], cnt);
}

// label[r] = r.
HPSPMM_KERNEL __launch_bounds__(kBlock) void cluster_init_kernel(int64_t rows, int32_t* __restrict__ label) {
  const int64_t r = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (r < rows) label[r] = (int32_t)r;
}

// len[i] = number of nonzeros of the i-th row in processing order, some[i] = 1 if it has any;
// len[rows] = some[rows] = 0.
HPSPMM_KERNEL __launch_bounds__(kBlock) void ordered_len_kernel(int64_t rows, const int32_t* __restrict__ rowptr,
                                                             const int32_t* __restrict__ order,
                                                             uint32_t* __restrict__ len, uint32_t* __restrict__ some) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i > rows) return;
  uint32_t n = 0;
  if (i < rows) {
    const int32_t r = order[i];
    n = (uint32_t)(rowptr[r + 1] - rowptr[r]);
  }
  len[i] = n;
  some[i] = n != 0;
}

// seen[order[i]] += 1: a permutation leaves every counter at exactly one.
HPSPMM_KERNEL __launch_bounds__(kBlock) void ordered_mark_kernel(int64_t rows, const int32_t* __restrict__ order,
                                                              int32_t* __restrict__ seen,
                                                              int32_t* __restrict__ bad) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= rows) return;
  const int32_t r = order[i];
  if (r < 0 || (int64_t)r >= rows) {
    atomicOr(bad, 1);
    return;
  }
  if (atomicAdd(&seen[r], 1) != 0) atomicOr(bad, 2);
}

// A rows x cols pattern as a graph of rows + cols vertices (vertex rows + c stands for column c),
// for the label propagation above: row r is adjacent to the columns it has an entry in, column c to
// the rows that have one in it.
// out[j] = col[j] + by: the neighbours of the row vertices.
HPSPMM_KERNEL __launch_bounds__(kBlock) void bipartite_shift_kernel(int64_t nnz, const int32_t* __restrict__ col,
                                                                 int32_t by, int32_t* __restrict__ out) {
  const int64_t j = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (j < nnz) out[j] = col[j] + by;
}

// colptr[c] = base + the number of entries in columns below c, for c in [0, cols], from the column
// of every nonzero in increasing order (sorted[nnz]): one thread per column bisects the sorted list
// (the same work whatever the gaps between the columns that occur).
HPSPMM_KERNEL __launch_bounds__(kBlock) void bipartite_colptr_kernel(int64_t nnz, const uint32_t* __restrict__ sorted,
                                                                  int64_t cols, int32_t base,
                                                                  int32_t* __restrict__ colptr) {
  const int64_t c = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (c > cols) return;
  int64_t lo = 0, hi = nnz;  // first position whose column is >= c
  while (lo < hi) {
    const int64_t mid = lo + ((hi - lo) >> 1);
    if ((int64_t)sorted[mid] < c) lo = mid + 1;
    else hi = mid;
  }
  colptr[c] = base + (int32_t)lo;
}

// Lays the nonzeros out in processing order.  One wavefront per position i: row r = order[i] starts
// at pstart[i] and is run prun[i] (the scans of len and some); start[r] = pstart[i].  oent = the
// column of every nonzero, a row's nonzeros in stored order, the first one flagged kRunStart;
// run_row / run_delta of the row's run; seg_run[g] for every segment that begins within the row.
HPSPMM_KERNEL __launch_bounds__(kBlock) void ordered_fill_kernel(int64_t rows, const int32_t* __restrict__ rowptr,
                                                              const int32_t* __restrict__ col,
                                                              const int32_t* __restrict__ order,
                                                              const uint32_t* __restrict__ pstart,
                                                              const uint32_t* __restrict__ prun, int shift,
                                                              int32_t* __restrict__ start,
                                                              int32_t* __restrict__ oent,
                                                              int32_t* __restrict__ run_row,
                                                              int32_t* __restrict__ run_delta,
                                                              int32_t* __restrict__ seg_run) {
  const int lane = threadIdx.x & 63;
  const int64_t i = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  if (i >= rows) return;
  const int32_t r = order[i];
  const int32_t lb = rowptr[r];
  const int32_t hb = rowptr[r + 1];
  const int32_t p0 = (int32_t)pstart[i];
  if (lane == 0) start[r] = p0;
  if (hb == lb) return;
  const int32_t run = (int32_t)prun[i];
  if (lane == 0) {
    run_row[run] = r;
    run_delta[run] = lb - p0;
  }
  const int64_t seg = (int64_t)1 << shift;
  for (int64_t g = (p0 + seg - 1) / seg + lane; g * seg < (int64_t)p0 + (hb - lb); g += 64) seg_run[g] = run;
  for (int32_t j = lb + lane; j < hb; j += 64) oent[p0 + (j - lb)] = col[j] | (j == lb ? kRunStart : 0);
}

// Per window of `window` consecutive nonzeros (in processing order; window <=
// kOrderedMaxWindow): the columns that occur at least twice, the `cap` most
// frequent of them (ties: an occurrence count is either kept whole or dropped
// whole), in increasing column order -> wcols[w * cap + slot] (-1 = unused
// slot); the entry words of those columns (ocol: column in bits 0..28, kRunStart)
// get bit 31 and the slot for the column.  One workgroup per
// window.  Most columns of a window occur once, so two bitmaps first tell which
// hash values were seen twice; only those nonzeros are counted exactly, in an LDS
// hash table (as many slots as a window has nonzeros: it cannot overflow);
// then a histogram of the counts, a threshold, the compaction of the selected
// columns and a bitonic sort of those few.  Every step depends only on the set
// of the window's columns, not on the order the threads run in: the same plan
// every time.  served[0] += rewritten nonzeros.
constexpr int kOrderedMaxWindow = 8192;
constexpr int kOrderedHistMax = 65;       // occurrence counts are told apart up to this one
constexpr int kOrderedBitmapWords = 1024;  // 32768 bits per bitmap
constexpr int kOrderedMaxCap = 512;        // LDS slots a window can ask for, at most

HPSPMM_KERNEL __launch_bounds__(kBlock) void ordered_hot_kernel(int64_t nnz, int window, int cap,
                                                             int32_t* __restrict__ ocol,
                                                             int32_t* __restrict__ wcols,
                                                             unsigned long long* __restrict__ served) {
  __shared__ uint32_t s_once[kOrderedBitmapWords];
  __shared__ uint32_t s_twice[kOrderedBitmapWords];
  __shared__ int32_t s_key[kOrderedMaxWindow];        // hash table: column, -1 = free
  __shared__ uint32_t s_cnt[kOrderedMaxWindow / 2];   // two 16-bit occurrence counts per word
  __shared__ int32_t s_sel[kOrderedMaxCap];           // selected columns
  __shared__ int32_t s_hist[kOrderedHistMax + 1];     // s_hist[t] = columns that occur >= t times, t in [2, kOrderedHistMax]
  __shared__ int32_t s_count;
  const int tid = threadIdx.x;
  const int64_t w = blockIdx.x;
  const int64_t p0 = w * window;
  const int n = nnz - p0 < window ? (int)(nnz - p0) : window;
  for (int i = tid; i < kOrderedBitmapWords; i += kBlock) {
    s_once[i] = 0;
    s_twice[i] = 0;
  }
  for (int i = tid; i < kOrderedMaxWindow; i += kBlock) s_key[i] = -1;
  for (int i = tid; i < kOrderedMaxWindow / 2; i += kBlock) s_cnt[i] = 0;
  for (int i = tid; i <= kOrderedHistMax; i += kBlock) s_hist[i] = 0;
  for (int i = tid; i < kOrderedMaxCap; i += kBlock) s_sel[i] = INT32_MAX;
  if (tid == 0) s_count = 0;
  __syncthreads();
  auto bit_of = [](int32_t c) { return ((uint32_t)c * 0x9E3779B1u) >> 17; };  // 15 bits
  for (int i = tid; i < n; i += kBlock) {
    const uint32_t h = bit_of(ocol[p0 + i] & kEntryPayload);
    const uint32_t m = 1u << (h & 31);
    if (atomicOr(&s_once[h >> 5], m) & m) atomicOr(&s_twice[h >> 5], m);
  }
  __syncthreads();
  // exact counts of the columns whose hash value was seen twice
  for (int i = tid; i < n; i += kBlock) {
    const int32_t c = ocol[p0 + i] & kEntryPayload;
    const uint32_t h = bit_of(c);
    if (!((s_twice[h >> 5] >> (h & 31)) & 1u)) continue;
    uint32_t slot = ((uint32_t)c * 0x85EBCA6Bu) >> 19;  // 13 bits
    for (;;) {
      const int32_t seen = atomicCAS(&s_key[slot], -1, c);
      if (seen == -1 || seen == c) break;
      slot = (slot + 1) & (kOrderedMaxWindow - 1);
    }
    atomicAdd(&s_cnt[slot >> 1], 1u << (16 * (slot & 1)));
  }
  __syncthreads();
  auto count_of = [&](int slot) { return (int)((s_cnt[slot >> 1] >> (16 * (slot & 1))) & 0xFFFFu); };
  for (int i = tid; i < kOrderedMaxWindow; i += kBlock) {
    const int len = s_key[i] >= 0 ? count_of(i) : 0;
    if (len >= 2) atomicAdd(&s_hist[len < kOrderedHistMax ? len : kOrderedHistMax], 1);
  }
  __syncthreads();
  if (tid == 0)  // s_hist[t] = columns with exactly t occurrences  ->  with at least t
    for (int t = kOrderedHistMax - 1; t >= 2; --t) s_hist[t] += s_hist[t + 1];
  __syncthreads();
  const int limit = cap < kOrderedMaxCap ? cap : kOrderedMaxCap;
  int threshold = 2;
  while (threshold < kOrderedHistMax && s_hist[threshold] > limit) ++threshold;
  const bool fits = s_hist[threshold] <= limit;  // always, as long as cap >= window / kOrderedHistMax
  if (fits) {
    for (int i = tid; i < kOrderedMaxWindow; i += kBlock)
      if (s_key[i] >= 0 && count_of(i) >= threshold) s_sel[atomicAdd(&s_count, 1)] = s_key[i];
  }
  __syncthreads();
  const int m = s_count;
  // the selected columns in increasing order (unused entries hold INT32_MAX and sort behind them)
  for (int size = 2; size <= kOrderedMaxCap; size <<= 1) {
    for (int stride = size >> 1; stride > 0; stride >>= 1) {
      for (int i = tid; i < kOrderedMaxCap / 2; i += kBlock) {
        const int lo = ((i / stride) * stride * 2) + (i % stride);
        const int hi = lo + stride;
        const bool up = ((lo & size) == 0);
        const int32_t a = s_sel[lo], b = s_sel[hi];
        if ((a > b) == up) {
          s_sel[lo] = b;
          s_sel[hi] = a;
        }
      }
      __syncthreads();
    }
  }
  for (int i = tid; i < cap; i += kBlock) wcols[w * cap + i] = i < m ? s_sel[i] : -1;
  unsigned long long mine = 0;
  for (int i = tid; i < n; i += kBlock) {
    const int32_t w = ocol[p0 + i];
    const int32_t c = w & kEntryPayload;
    int lo = 0, hi = m;
    while (lo < hi) {
      const int mid = (lo + hi) >> 1;
      if (s_sel[mid] < c) lo = mid + 1;
      else hi = mid;
    }
    if (lo < m && s_sel[lo] == c) {
      ocol[p0 + i] = INT32_MIN | (w & kRunStart) | lo;  // the LDS slot, the first-of-row flag kept
      ++mine;
    }
  }
  for (int off = 32; off > 0; off >>= 1) mine += __shfl_down(mine, off);
  if ((tid & 63) == 0 && mine) atomicAdd(served, mine);
}

// What the fix-up kernel has to do with every row: write zeros (kActionZero: no nonzeros), add carry
// slots (kActionCross: its nonzeros lie in more than one stretch of 2^shift positions - the ordered
// plan passes the length of a window here, the main kernel adds up the rows cut inside one), or nothing.
HPSPMM_KERNEL __launch_bounds__(kBlock) void ordered_action_kernel(int64_t rows, const int32_t* __restrict__ rowptr,
                                                                   const int32_t* __restrict__ start, int shift,
                                                                   uint8_t* __restrict__ action) {
  const int64_t r = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (r >= rows) return;
  const int32_t len = rowptr[r + 1] - rowptr[r];
  const int64_t p0 = start[r];
  action[r] = len == 0 ? kActionZero : (p0 >> shift) != ((p0 + len - 1) >> shift) ? kActionCross : kActionNone;
}

// ---- SpMM kernel -----------------------------------------------------------

// One workgroup per window = kWavesPerBlock * P segments of 2^shift nonzeros.
// Dynamic LDS: cap * K floats, the window's slotted rows of B.
// oent = entry words (bit 31: bits 0..29 are an LDS slot, else a column; kRunStart: first entry of
// its row); run_row / run_delta per run (= non-empty row, in processing order); seg_run[g] = run of
// segment g's first entry; start[r] = position of row r's first nonzero.
template <int K, int kLd = 0>
__global__ __launch_bounds__(kBlock) void spmm_ordered_kernel(
    const int32_t* __restrict__ rowptr, const int32_t* __restrict__ start, const int32_t* __restrict__ oent,
    const int32_t* __restrict__ run_row, const int32_t* __restrict__ run_delta, const int32_t* __restrict__ seg_run,
    const float* __restrict__ val, const int32_t* __restrict__ wcols, int cap, const float* __restrict__ B,
    float* __restrict__ C, float* __restrict__ carry, int64_t nnz, int shift, int64_t nblocks, bool remap,
    uint32_t ld_arg) {
  constexpr int G = K / 4;
  constexpr int P = 64 / G;
  constexpr int TL = kTile / G;
  const uint32_t ld = row_length<K, kLd>(ld_arg);  // floats between the rows of B and of C
  __shared__ __attribute__((aligned(16))) int32_t s_col[kWavesPerBlock * P * kTileStride];
  __shared__ __attribute__((aligned(16))) float s_val[kWavesPerBlock * P * kTileStride];
  __shared__ __attribute__((aligned(16))) int32_t s_row[kWavesPerBlock * P * kTileStride];
  extern __shared__ __attribute__((aligned(16))) float s_b[];  // [cap][K]

  const int64_t blk = xcd_remap(blockIdx.x, nblocks, remap);
  if (blk < 0) return;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int l = lane % G;

  // the window's rows of B; every thread of the workgroup reaches the barrier
  for (int i = tid; i < cap * G; i += kBlock) {
    const int slot = i / G;
    const int32_t c = wcols[blk * cap + slot];
    if (c >= 0 && lane_columns<K, kLd>(ld_arg, i % G) > 0)
      *reinterpret_cast<float4*>(s_b + slot * K + 4 * (i % G)) = load_b_ld(B, c, i % G, ld);
  }
  __syncthreads();

  const int wseg = (tid >> 6) * P + lane / G;  // this sub-wave's segment within the window
  const int64_t g = blk * (kWavesPerBlock * P) + wseg;
  const int64_t s = g << shift;
  const bool active = s < nnz;  // (every thread stays for the barriers at the end)
  const int64_t e = (s + ((int64_t)1 << shift)) < nnz ? (s + ((int64_t)1 << shift)) : nnz;
  const int64_t wbeg = (blk * (kWavesPerBlock * P)) << shift;       // the window: positions [wbeg, wend)
  const int64_t wend = wbeg + ((int64_t)(kWavesPerBlock * P) << shift);
  const int sbase = wseg * kTileStride;

  const int nv = lane_columns<K, kLd>(ld_arg, l);
  const bool in_tile = nv > 0;
  const bool c_aligned = c_rows_aligned<kLd>(ld_arg);
  const uint32_t ldc = c_row_length<K, kLd>(ld_arg);
  // Partial sums of the rows this segment shares with its neighbours: of the row that began in an
  // earlier segment (head) and of the row that goes on into the next one (tail).  They stay here when
  // the whole row lies inside the window, and go to the carry slots in memory when it does not.
  float4 head_acc = make_float4(0.f, 0.f, 0.f, 0.f), tail_acc = head_acc;
  bool head_here = false, tail_here = false;
  int32_t tail_row = 0;
  int64_t tail_last = 0;  // last position of the tail row
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  if (active) {
    // `run` = the run of the entry before the next tile whose rows are looked up: to begin with, the run
    // of the segment's first entry, less one if that entry starts it
    const int32_t first_run = seg_run[g];
    int32_t run = first_run - ((oent[s] & kRunStart) != 0);
    int32_t cur = run_row[first_run];
    // (where the first row lies is looked up here, with the other loads of the start: inside the walk
    // the two dependent loads would stall the wavefront at the first change of row)
    const int64_t first_rs = start[cur];
    const int64_t first_re = first_rs + (rowptr[cur + 1] - rowptr[cur]);
    bool head_pending = first_rs < s;
    const bool head_inside = first_rs >= wbeg && first_re <= wend;

    auto flush_to = [&](bool is_tail) {
      if (head_pending) {
        if (head_inside) {
          head_acc = acc;
          head_here = true;
        } else if (in_tile) {
          store_result(carry + (uint64_t)(2 * g) * K + 4 * l, acc);
        }
        head_pending = false;
        return;
      }
      if (is_tail) {
        const int64_t rs = start[cur];
        const int64_t re = rs + (rowptr[cur + 1] - rowptr[cur]);
        if (rs >= wbeg && re <= wend) {
          tail_acc = acc;
          tail_here = true;
          tail_row = cur;
          tail_last = re - 1;
        } else if (in_tile) {
          store_result(carry + (uint64_t)(2 * g + 1) * K + 4 * l, acc);
        }
        return;
      }
      // (what a lane beyond the tile holds is never read)
      if (in_tile) store_c_row<kLd, true>(C + (uint64_t)(uint32_t)cur * ldc + 4 * l, acc, nv, c_aligned);
    };
    auto flush = [&]() { flush_to(false); };
    // One flat load per gather, its address selected between the LDS copy and memory: a branch
    // per gather would make every load of a batch wait for the one before it.
    const float* lds_b = s_b;
    // a lane beyond the tile gathers what lane 0 gathers (a valid address, no branch in the loop); its
    // sums are never stored
    const int lg = in_tile ? l : 0;
    auto loadb = [&](int32_t c) {
      const uint32_t idx = (uint32_t)(c & kEntryPayload);
      const float* row = c < 0 ? lds_b + idx * (uint32_t)K : B + (uint64_t)idx * (uint64_t)ld;
      return *reinterpret_cast<const float4*>(row + 4 * lg);
    };

    // Two-deep prefetch.  look(t): the entry words of tile t and, from the run starts among them (a lane
    // counts those of its TL entries, the sub-wave scans the counts), the row and the value offset of
    // every entry.  take(t): the values of tile t through the offsets looked up one step earlier.  (The
    // plan's arrays are allocated by the library, hence always aligned for the vector loads.)
    int32_t ec[TL], er[TL], ed[TL];
    auto look = [&](int64_t t) {
      const int64_t q = t + l * TL;
      load_run<TL>(ec, oent, q, e, true);  // 0 beyond e: a plain entry of the run before
      int32_t starts = 0;
#pragma unroll
      for (int j = 0; j < TL; ++j) starts += (ec[j] & kRunStart) != 0;
      int32_t incl = starts;
#pragma unroll
      for (int off = 1; off < G; off <<= 1) {
        const int32_t o = __shfl_up(incl, off, G);
        if (l >= off) incl += o;
      }
      int32_t at = run + incl - starts;
#pragma unroll
      for (int j = 0; j < TL; ++j) {
        at += (ec[j] & kRunStart) != 0;
        er[j] = run_row[at];
        ed[j] = run_delta[at];
      }
      run += __shfl(incl, G - 1, G);
    };
    TileRegs<TL> m;
    auto take = [&](int64_t t) {
      const int64_t q = t + l * TL;
#pragma unroll
      for (int j = 0; j < TL; ++j) {
        m.c[j] = ec[j];
        m.r[j] = er[j];
        m.v[j] = q + j < e ? val[q + j + ed[j]] : 0.f;
      }
    };
    look(s);
    take(s);
    if (s + kTile < e) look(s + kTile);
    for (int64_t t = s; t < e; t += kTile) {
      stage_tile<TL>(m, sbase + l * TL, s_col, s_val, s_row);
      wave_lds_fence();
      if (t + kTile < e) {
        take(t + kTile);
        if (t + 2 * kTile < e) look(t + 2 * kTile);
      }
      const int cnt = (e - t) < kTile ? (int)(e - t) : kTile;
      consume_tile(cnt, sbase, s_col, s_val, s_row, cur, acc, loadb, flush);
      wave_lds_fence();
    }
    flush_to((int64_t)start[cur] + (rowptr[cur + 1] - rowptr[cur]) > e);
  }  // active

  // The rows cut inside the window.  The window's rows of B are not needed any more: their LDS takes
  // the head sums, one row of K floats per segment of the window (cap >= kWavesPerBlock * P: the host
  // checks).  Every thread of the workgroup reaches both barriers.
  __syncthreads();
  if (head_here && in_tile) *reinterpret_cast<float4*>(s_b + wseg * K + 4 * l) = head_acc;
  __syncthreads();
  if (tail_here && in_tile) {
    // the part in the row's first segment, then the heads of the segments it goes on into, in that
    // order - as the fix-up kernel adds the carry slots of a row
    float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);
    sum.x += tail_acc.x;
    sum.y += tail_acc.y;
    sum.z += tail_acc.z;
    sum.w += tail_acc.w;
    const int last = (int)((tail_last - wbeg) >> shift);
    for (int w = wseg + 1; w <= last; ++w) {
      const float4 h = *reinterpret_cast<const float4*>(s_b + w * K + 4 * l);
      sum.x += h.x;
      sum.y += h.y;
      sum.z += h.z;
      sum.w += h.w;
    }
    store_c_row<kLd, true>(C + (uint64_t)(uint32_t)tail_row * ldc + 4 * l, sum, nv, c_aligned);
  }
}

// Fix-up after the ordered kernel, from the plan's lists: workgroups [0, cross_blocks) - one
// sub-wave per row whose nonzeros lie in more than one window: tail[ga] + head[ga + 1] + ... +
// head[gb] from the carry slots of its segments, in that order; the others - one sub-wave per row
// without nonzeros: zeros.  Every other row was stored by the main kernel.
template <int K, int kLd = 0>
__global__ __launch_bounds__(kBlock) void spmm_ordered_fixup_kernel(
    const int32_t* __restrict__ rowptr, const int32_t* __restrict__ start, const int32_t* __restrict__ cross_rows,
    int64_t n_cross, int64_t cross_blocks, const int32_t* __restrict__ zero_rows, int64_t n_zero,
    const float* __restrict__ carry, float* __restrict__ C, int shift, uint32_t ld_arg) {
  constexpr int G = K / 4;
  constexpr int P = 64 / G;
  const uint32_t ld = c_row_length<K, kLd>(ld_arg);
  const bool c_aligned = c_rows_aligned<kLd>(ld_arg);
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int l = lane % G;
  const int nv = lane_columns<K, kLd>(ld_arg, l);
  if (nv == 0) return;
  const int sub = (tid >> 6) * P + lane / G;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  if ((int64_t)blockIdx.x >= cross_blocks) {
    const int64_t idx = ((int64_t)blockIdx.x - cross_blocks) * (kWavesPerBlock * P) + sub;
    if (idx < n_zero) store_c_row<kLd, false>(C + (uint64_t)(uint32_t)zero_rows[idx] * ld + 4 * l, acc, nv, c_aligned);
    return;
  }
  const int64_t idx = (int64_t)blockIdx.x * (kWavesPerBlock * P) + sub;
  if (idx >= n_cross) return;
  const int64_t row = cross_rows[idx];
  const int64_t p0 = start[row];
  const int64_t ga = p0 >> shift;
  const int64_t gb = (p0 + (rowptr[row + 1] - rowptr[row]) - 1) >> shift;
  const float* cbase = carry + 4 * l;
  auto add = [&](const float4& t) {
    acc.x += t.x;
    acc.y += t.y;
    acc.z += t.z;
    acc.w += t.w;
  };
  add(*reinterpret_cast<const float4*>(cbase + (uint64_t)(2 * ga + 1) * K));
  int64_t g = ga + 1;
  for (; g + kBatch <= gb + 1; g += kBatch) {
    float4 slot[kBatch];
#pragma unroll
    for (int t = 0; t < kBatch; ++t) slot[t] = *reinterpret_cast<const float4*>(cbase + (uint64_t)(2 * (g + t)) * K);
#pragma unroll
    for (int t = 0; t < kBatch; ++t) add(slot[t]);
  }
  for (; g <= gb; ++g) add(*reinterpret_cast<const float4*>(cbase + (uint64_t)(2 * g) * K));
  store_c_row<kLd, false>(C + (uint64_t)row * ld + 4 * l, acc, nv, c_aligned);
}

}  // namespace hpspmm
