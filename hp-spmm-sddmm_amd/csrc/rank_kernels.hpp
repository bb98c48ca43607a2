// Plan-time device code: column popularity ranking.
//
// Several strategies want the `want` most referenced columns of A in order of decreasing nonzero
// count (ties by lower index, so that the choice is reproducible).  Everything happens on the
// device: a histogram of the column indices, a radix select of the want-th largest count (four
// passes over the counters, 8 bits each), a stable compaction of the selected columns (flags, scan,
// scatter: ties in index order) and a rank-by-counting sort of the at most 2^17 selected keys.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "spmm_kernels.hpp"

namespace hpspmm {

// count[col[j]] += 1 for every `stride`-th nonzero (count[] zeroed by the caller); stride 1 = all.
// A column of a power-law graph receives up to 10^5 of these increments, and atomics on one address
// are served one after the other (the 163k increments of R-MAT's hottest column alone took 12 ms).
// So every workgroup first counts its stretch of kCountChunk sampled nonzeros in an LDS table
// (open addressing by a hash of the column, a handful of probes; a nonzero that finds no slot goes
// to memory directly) and then adds each table entry to memory once: the increments of a hot column
// reach memory once per workgroup instead of once per nonzero.
constexpr int kCountChunk = 1 << 15;
constexpr int kCountSlots = 1 << 12;
constexpr int kCountProbes = 4;

HPSPMM_KERNEL __launch_bounds__(kBlock) void count_columns_strided_kernel(int64_t nnz, int64_t stride,
                                                                       const int32_t* __restrict__ col,
                                                                       int32_t* __restrict__ count) {
  __shared__ int32_t s_key[kCountSlots];
  __shared__ int32_t s_cnt[kCountSlots];
  for (int i = threadIdx.x; i < kCountSlots; i += kBlock) {
    s_key[i] = -1;
    s_cnt[i] = 0;
  }
  __syncthreads();
  const int64_t n = (nnz + stride - 1) / stride;
  const int64_t i0 = (int64_t)blockIdx.x * kCountChunk;
  const int64_t i1 = i0 + kCountChunk < n ? i0 + kCountChunk : n;
  for (int64_t i = i0 + threadIdx.x; i < i1; i += kBlock) {
    const int32_t c = col[i * stride];
    uint32_t slot = ((uint32_t)c * 0x9E3779B1u) >> 20;  // 12 bits
    bool placed = false;
#pragma unroll
    for (int probe = 0; probe < kCountProbes && !placed; ++probe) {
      const int32_t seen = atomicCAS(&s_key[slot], -1, c);
      if (seen == -1 || seen == c) {
        atomicAdd(&s_cnt[slot], 1);
        placed = true;
      }
      slot = (slot + 1) & (kCountSlots - 1);
    }
    if (!placed) atomicAdd(&count[c], 1);
  }
  __syncthreads();
  for (int i = threadIdx.x; i < kCountSlots; i += kBlock)
    if (s_cnt[i]) atomicAdd(&count[s_key[i]], s_cnt[i]);
}

// hist[b] += number of counters whose bits above `shift + 8` equal those of `prefix` and whose byte
// at `shift` is b (hist[256] zeroed by the caller).  With shift = 24 every counter takes part.
HPSPMM_KERNEL __launch_bounds__(kBlock) void select_histogram_kernel(int64_t n, const int32_t* __restrict__ count,
                                                                  uint32_t prefix, int shift,
                                                                  uint32_t* __restrict__ hist) {
  __shared__ uint32_t s_hist[256];
  s_hist[threadIdx.x] = 0;
  __syncthreads();
  const uint32_t high_mask = shift >= 24 ? 0u : ~((1u << (shift + 8)) - 1u);
  const int64_t step = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += step) {
    const uint32_t v = (uint32_t)count[i];
    if ((v & high_mask) == (prefix & high_mask)) atomicAdd(&s_hist[(v >> shift) & 255u], 1u);
  }
  __syncthreads();
  if (s_hist[threadIdx.x]) atomicAdd(&hist[threadIdx.x], s_hist[threadIdx.x]);
}

// above[i] = count[i] > threshold, equal[i] = count[i] == threshold (i < n); both get a trailing 0 at n
// so that their exclusive scans end in the totals.
HPSPMM_KERNEL __launch_bounds__(kBlock) void select_flags_kernel(int64_t n, const int32_t* __restrict__ count,
                                                              int32_t threshold, uint32_t* __restrict__ above,
                                                              uint32_t* __restrict__ equal) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i > n) return;
  const int32_t c = i < n ? count[i] : INT32_MIN;
  above[i] = c > threshold ? 1u : 0u;
  equal[i] = (i < n && c == threshold) ? 1u : 0u;
}

// The selected columns in index order: every column above the threshold, then the first `ties`
// columns at the threshold.  key = (~count << 32) | index sorts by decreasing count, then index.
HPSPMM_KERNEL __launch_bounds__(kBlock) void select_compact_kernel(int64_t n, const int32_t* __restrict__ count,
                                                                int32_t threshold,
                                                                const uint32_t* __restrict__ above_scan,
                                                                const uint32_t* __restrict__ equal_scan,
                                                                uint32_t n_above, uint32_t ties,
                                                                unsigned long long* __restrict__ keys) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= n) return;
  const int32_t c = count[i];
  int64_t slot = -1;
  if (c > threshold) slot = above_scan[i];
  else if (c == threshold && equal_scan[i] < ties) slot = (int64_t)n_above + equal_scan[i];
  if (slot >= 0) keys[slot] = ((unsigned long long)(~(uint32_t)c) << 32) | (uint32_t)i;
}

// The selected keys taken apart for the radix sort: sort_key[i] = high word (the inverted count:
// ascending = most referenced first), id[i] = low word (the column).  *served += the counts.
HPSPMM_KERNEL __launch_bounds__(kBlock) void rank_split_kernel(int32_t m, const unsigned long long* __restrict__ keys,
                                                            uint32_t* __restrict__ sort_key, int32_t* __restrict__ id,
                                                            unsigned long long* __restrict__ served) {
  const int32_t i = (int32_t)blockIdx.x * kBlock + threadIdx.x;
  unsigned long long c = 0;
  if (i < m) {
    const unsigned long long mine = keys[i];
    sort_key[i] = (uint32_t)(mine >> 32);
    id[i] = (int32_t)(uint32_t)mine;
    c = (unsigned long long)(~(uint32_t)(mine >> 32));
  }
  for (int off = 32; off > 0; off >>= 1) c += __shfl_down(c, off);
  if ((threadIdx.x & 63) == 0 && c) atomicAdd(served, c);
}

// Popularity rank s -> compact-buffer slot (s % slices) * per_slice + s / slices:
// colmap[ids[s]] = slot, slot_src[slot] = ids[s] (both preset to -1 by the caller).
HPSPMM_KERNEL __launch_bounds__(kBlock) void hot_slots_kernel(int32_t m, const int32_t* __restrict__ ids, int slices,
                                                           int32_t per_slice, int32_t* __restrict__ colmap,
                                                           int32_t* __restrict__ slot_src) {
  const int32_t s = (int32_t)blockIdx.x * kBlock + threadIdx.x;
  if (s >= m) return;
  const int32_t slot = (s % slices) * per_slice + s / slices;
  colmap[ids[s]] = slot;
  slot_src[slot] = ids[s];
}

// colmap[ids[s]] = s.
HPSPMM_KERNEL __launch_bounds__(kBlock) void hot_index_kernel(int32_t m, const int32_t* __restrict__ ids,
                                                           int32_t* __restrict__ colmap) {
  const int32_t s = (int32_t)blockIdx.x * kBlock + threadIdx.x;
  if (s < m) colmap[ids[s]] = s;
}

// Column ranges of equal nonzero count: range[c] = min(groups - 1, (nonzeros in columns < c) / target),
// from the exclusive scan of the column counts.
HPSPMM_KERNEL __launch_bounds__(kBlock) void column_range_kernel(int64_t cols, const uint32_t* __restrict__ before,
                                                              int64_t target, int groups,
                                                              uint8_t* __restrict__ range) {
  const int64_t c = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (c >= cols) return;
  const int64_t r = (int64_t)before[c] / target;
  range[c] = (uint8_t)(r < groups - 1 ? r : groups - 1);
}

// hot[range[ids[s]]] += 1 (hot[] zeroed by the caller; at most 64 ranges), through a workgroup's LDS
// histogram: a few dozen counters would otherwise take every increment one after the other.
HPSPMM_KERNEL __launch_bounds__(kBlock) void range_hot_count_kernel(int32_t m, const int32_t* __restrict__ ids,
                                                                 const uint8_t* __restrict__ range,
                                                                 uint32_t* __restrict__ hot) {
  __shared__ uint32_t s_hot[64];
  if (threadIdx.x < 64) s_hot[threadIdx.x] = 0;
  __syncthreads();
  const int32_t s = (int32_t)blockIdx.x * kBlock + threadIdx.x;
  if (s < m) atomicAdd(&s_hot[range[ids[s]] & 63], 1u);
  __syncthreads();
  if (threadIdx.x < 64 && s_hot[threadIdx.x]) atomicAdd(&hot[threadIdx.x], s_hot[threadIdx.x]);
}

// ---------------------------------------------------------------------------------------------
// Stable radix sort of (key, value) pairs by 8-bit digits, least significant first: three kernels a
// pass (digit counts per tile, their scan - the caller's -, scatter).  Used to order the rows by
// cluster label with the rows of one label in increasing order.
// ---------------------------------------------------------------------------------------------
constexpr int kSortItems = 8;                     // elements per thread
constexpr int kSortTile = kBlock * kSortItems;    // elements per workgroup

// hist[d * n_tiles + tile] = elements of the tile whose digit is d.
HPSPMM_KERNEL __launch_bounds__(kBlock) void sort_count_kernel(int64_t n, const uint32_t* __restrict__ keys, int shift,
                                                            int64_t n_tiles, uint32_t* __restrict__ hist) {
  __shared__ uint32_t s_hist[256];
  s_hist[threadIdx.x] = 0;
  __syncthreads();
  const int64_t base = (int64_t)blockIdx.x * kSortTile;
  for (int q = 0; q < kSortItems; ++q) {
    const int64_t i = base + q * kBlock + threadIdx.x;
    if (i < n) atomicAdd(&s_hist[(keys[i] >> shift) & 255u], 1u);
  }
  __syncthreads();
  hist[(int64_t)threadIdx.x * n_tiles + blockIdx.x] = s_hist[threadIdx.x];
}

// Scatter of one pass: element i of the tile goes to offsets[d * n_tiles + tile] + (number of
// elements of the tile before i with the same digit d).  That number is found round by round (256
// consecutive elements a round), wavefront by wavefront within a round (running counts per digit in
// LDS) and by ballots within a wavefront - in index order throughout, which is what keeps the sort stable.
HPSPMM_KERNEL __launch_bounds__(kBlock) void sort_scatter_kernel(int64_t n, const uint32_t* __restrict__ keys_in,
                                                              const int32_t* __restrict__ vals_in, int shift,
                                                              int64_t n_tiles, const uint32_t* __restrict__ offsets,
                                                              uint32_t* __restrict__ keys_out,
                                                              int32_t* __restrict__ vals_out) {
  __shared__ uint32_t s_run[256];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  s_run[threadIdx.x] = offsets[(int64_t)threadIdx.x * n_tiles + blockIdx.x];
  __syncthreads();
  const int64_t base = (int64_t)blockIdx.x * kSortTile;
  const uint64_t below = (1ull << lane) - 1ull;
  for (int q = 0; q < kSortItems; ++q) {
    const int64_t i = base + q * kBlock + threadIdx.x;
    const bool valid = i < n;
    const uint32_t key = valid ? keys_in[i] : 0u;
    const int32_t val = valid ? vals_in[i] : 0;
    const uint32_t d = (key >> shift) & 255u;
    // lanes of this wavefront that hold a valid element with the same digit
    uint64_t same = __ballot(valid);
#pragma unroll
    for (int b = 0; b < 8; ++b) {
      const uint64_t set = __ballot((d >> b) & 1u);
      same &= ((d >> b) & 1u) ? set : ~set;
    }
    const uint32_t before = (uint32_t)__popcll(same & below);
    uint32_t dest = 0;
    for (int w = 0; w < kWavesPerBlock; ++w) {
      if (wave == w && valid) {
        dest = s_run[d] + before;
      }
      __syncthreads();
      if (wave == w && valid && before == 0) s_run[d] += (uint32_t)__popcll(same);
      __syncthreads();
    }
    if (valid) {
      keys_out[dest] = key;
      vals_out[dest] = val;
    }
  }
}

// keys[r] = label[r], vals[r] = r.
HPSPMM_KERNEL __launch_bounds__(kBlock) void label_pairs_kernel(int64_t rows, const int32_t* __restrict__ label,
                                                             uint32_t* __restrict__ keys, int32_t* __restrict__ vals) {
  const int64_t r = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (r >= rows) return;
  keys[r] = (uint32_t)label[r];
  vals[r] = (int32_t)r;
}

// size[label[r]] += 1 (size[] zeroed by the caller).
HPSPMM_KERNEL __launch_bounds__(kBlock) void label_sizes_kernel(int64_t rows, const int32_t* __restrict__ label,
                                                             int32_t* __restrict__ size) {
  const int64_t r = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (r < rows) atomicAdd(&size[label[r]], 1);
}

// Locality of the stored order: how often a gather of a row of B finds that row among the last
// `capacity` distinct ones.  One workgroup per sample walks the column indices from its start
// (wrapping at the end), one chunk of kLocalityBlock in every kLocalityDeal - what one XCD gets of
// consecutive pieces of the matrix -, marks every column in a bit table of its own and counts the
// columns it had not marked before.  The walk ends once `capacity` distinct columns have been seen
// or after max_walk nonzeros.  out[4 s ..]: nonzeros walked and distinct columns when the count first
// reached capacity / 2 (0, 0 if it never did), the same two at the end: the slope between the two
// points is the share of the gathers that miss a cache of about 3/4 of that capacity.
constexpr int kLocalityBlock = 1024;
constexpr int kLocalityDeal = 8;
constexpr int kLocalityBits = 22;  // bits per table; columns beyond that many are hashed into it
HPSPMM_KERNEL __launch_bounds__(kLocalityBlock) void locality_walk_kernel(int64_t nnz, const int32_t* __restrict__ col,
                                                                         int64_t sample_stride, int hashed,
                                                                         uint32_t capacity, uint32_t max_walk,
                                                                         uint32_t* __restrict__ tables,
                                                                         uint32_t* __restrict__ out) {
  __shared__ uint32_t s_new[3];
  uint32_t* table = tables + ((size_t)blockIdx.x << (kLocalityBits - 5));
  if (threadIdx.x < 3) s_new[threadIdx.x] = 0;
  __syncthreads();
  const int64_t base = (int64_t)blockIdx.x * sample_stride;
  uint32_t walked = 0, distinct = 0, half_walked = 0, half_distinct = 0;
  for (uint32_t it = 0; walked < max_walk && distinct < capacity; ++it) {
    const int64_t q = (base + (int64_t)it * kLocalityDeal * kLocalityBlock + threadIdx.x) % nnz;
    const uint32_t c = (uint32_t)col[q];
    // (masked: the column indices of an unchecked matrix may be anything)
    const uint32_t h = (hashed ? (c * 2654435761u) >> (32 - kLocalityBits) : c) & ((1u << kLocalityBits) - 1u);
    const uint32_t bit = 1u << (h & 31);
    const bool fresh = !(atomicOr(&table[h >> 5], bit) & bit);
    const unsigned long long m = __ballot(fresh);
    if ((threadIdx.x & 63) == 0 && m) atomicAdd(&s_new[it % 3], (uint32_t)__popcll(m));
    __syncthreads();
    distinct += s_new[it % 3];
    walked += kLocalityBlock;
    // the counter of the round after the next: last read before this barrier, next added to after the next one
    if (threadIdx.x == 0) s_new[(it + 2) % 3] = 0;
    if (half_walked == 0 && distinct >= capacity / 2) {
      half_walked = walked;
      half_distinct = distinct;
    }
  }
  if (threadIdx.x == 0) {
    out[4 * blockIdx.x + 0] = half_walked;
    out[4 * blockIdx.x + 1] = half_distinct;
    out[4 * blockIdx.x + 2] = walked;
    out[4 * blockIdx.x + 3] = distinct;
  }
}

}  // namespace hpspmm
