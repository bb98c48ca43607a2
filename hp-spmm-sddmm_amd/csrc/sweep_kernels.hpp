// gfx950 device code of the *sweep* strategy for FP32 CSR SpMM.
//
// For a matrix with long rows whose B is larger than the L2s but small against the gather volume
// (nnz * K * 4 bytes), the gather can be made L2-resident by construction instead of by popularity:
// all wavefronts walk the columns of B in the same order and at about the same pace, window after
// window of half a megabyte of B, so that at any moment the whole chip reads one short stretch of B
// that every L2 holds.  What makes that possible without writing partial results to memory is that
// the accumulators of a row stay on the chip for the whole walk:
//
//   * one workgroup fills a CU; each of its wavefronts owns 8 accumulator slots per sub-wave in LDS
//     (8 KB per wavefront for every K).  A slot belongs to one *piece*: a whole row, or every m-th
//     nonzero of a row longer than the piece limit (interleaved, so that every piece sees the same
//     column distribution).  Pieces are sorted by length and dealt to the wavefronts in serpentine
//     order, which evens out the wavefronts' totals; one *band* is as many pieces as the resident
//     wavefronts have slots, and the bands are worked through one after the other (workgroups start
//     in index order);
//   * the stream of a sub-wave lists, window after window, nonzeros of its wavefront's pieces whose
//     column lies in the window: one word with the column, the accumulator slot and two flags, and
//     the index of the value in the caller's array.  A *run* - the nonzeros of one piece in one
//     window - goes to one sub-wave as a whole; its last entry carries the flag that adds the
//     running sum onto the slot.  The sub-waves of a wavefront run in lockstep, so the plan deals
//     the runs of every window to them longest first, each to the sub-wave with the least so far,
//     and pads the window's chunk to the longest sub-wave (padding gathers a row of zeros);
//   * pace: the hardware serves the oldest wavefront of a SIMD first, which alone spreads the
//     wavefronts of a CU over a quarter of the running time.  Every wavefront therefore posts the
//     window it has reached in LDS and sets its own priority by how far ahead of the CU's slowest
//     wavefront it is (s_setprio), and sleeps when it is more than `lead` windows ahead (a bounded
//     wait that only throttles: results never depend on it).  Across CUs nothing is exchanged:
//     every band fills the device exactly, so all CUs carry the same load and stay within a few
//     windows of each other (measured; polling shared counters in memory cost more than it gained);
//   * when its stream ends a wavefront stores its slots: a whole row straight to C, a piece of a
//     split row to a partial-result row that the final kernel adds up in piece order (it also
//     writes the zeros of empty rows).  No atomics; bit-reproducible for a given plan.
#pragma once

#include <hip/hip_runtime.h>
#include <limits.h>
#include <stdint.h>

#include "routed_kernels.hpp"
#include "spmm_kernels.hpp"

namespace hpspmm {

constexpr int kSweepSlots = 8;  // accumulator slots per sub-wave
// A stream entry's first word: column in bits 0..23, accumulator slot of the wavefront in bits
// 24..29, bit 30 = padding (gathers zeros, value 0), bit 31 = last entry of its run (add the running
// sum onto the slot).
constexpr int kSweepColBits = 24;
constexpr int32_t kSweepColMask = (1 << kSweepColBits) - 1;
constexpr int32_t kSweepPad = 1 << 30;
constexpr int32_t kSweepFlush = INT32_MIN;
constexpr int32_t kSweepUnused = INT32_MIN;  // slot_row[]: the slot holds no piece

// Wavefronts per workgroup: as many as the 160 KB of LDS of a CU hold accumulators and staging
// tiles for (and a workgroup may have).
template <int K>
constexpr int sweep_waves() { return K == 32 ? 15 : 16; }

// LDS of one workgroup, in bytes: accumulators, staging tiles (entry word, value), pace keeping.
template <int K>
constexpr size_t sweep_lds_bytes() {
  constexpr int P = 64 / (K / 4);
  return (size_t)sweep_waves<K>() * (P * kSweepSlots * K * 4 + 2 * P * kTileStride * 4) + 128;
}

struct SweepLayout {
  int64_t n_waves;   // wavefronts over all bands
  int32_t n_windows;
  int32_t lead;        // windows a wavefront may be ahead of the slowest of its workgroup before it sleeps
  int32_t spin_limit;  // sleeps before a wavefront stops waiting for good (0 = never wait)
  int32_t priorities;  // 0 = leave the wavefront priorities alone (diagnostics)
};

// ---- plan-time kernels -----------------------------------------------------

// pieces[r] = number of pieces of row r (0 for an empty row), parts[r] = the same if the row is split,
// else 0 (its partial-result rows); both get a trailing 0 for the scans' totals.
HPSPMM_KERNEL __launch_bounds__(kBlock) void sweep_row_pieces_kernel(int64_t rows, const int32_t* __restrict__ rowptr,
                                                                  int32_t limit, uint32_t* __restrict__ pieces,
                                                                  uint32_t* __restrict__ parts) {
  const int64_t r = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (r > rows) return;
  uint32_t m = 0;
  if (r < rows) m = (uint32_t)((rowptr[r + 1] - rowptr[r] + limit - 1) / limit);
  pieces[r] = m;
  parts[r] = m > 1 ? m : 0u;
}

// Sort keys: piece number pbase[r] + k (piece k of row r) gets key = limit - length, so that an
// ascending stable sort lists the pieces by decreasing length, ties in row order.
HPSPMM_KERNEL __launch_bounds__(kBlock) void sweep_piece_keys_kernel(int64_t rows, const int32_t* __restrict__ rowptr,
                                                                  int32_t limit, const uint32_t* __restrict__ pbase,
                                                                  uint32_t* __restrict__ keys,
                                                                  int32_t* __restrict__ vals,
                                                                  int32_t* __restrict__ piece_row) {
  const int64_t r = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (r >= rows) return;
  const int32_t len = rowptr[r + 1] - rowptr[r];
  const int32_t m = (len + limit - 1) / limit;
  const uint32_t base = pbase[r];
  for (int32_t k = 0; k < m; ++k) {
    const int32_t mine = (len - k + m - 1) / m;
    keys[base + k] = (uint32_t)(limit - mine);
    vals[base + k] = (int32_t)(base + k);
    piece_row[base + k] = (int32_t)r;
  }
}

// The i-th longest piece goes to band i % n_bands; within the band, pieces are dealt to the band's
// wavefronts in rounds, alternately forwards and backwards; round j fills slot j of every wavefront.
// piece_of[wavefront * slots + round] = piece (preset to -1).
HPSPMM_KERNEL __launch_bounds__(kBlock) void sweep_assign_kernel(int64_t n_pieces, const int32_t* __restrict__ order,
                                                              int32_t n_bands, int32_t band_waves, int32_t slots,
                                                              int32_t* __restrict__ piece_of) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= n_pieces) return;
  const int32_t band = (int32_t)(i % n_bands);
  const int64_t within = i / n_bands;
  const int32_t round = (int32_t)(within / band_waves);
  const int32_t pos = (int32_t)(within % band_waves);
  const int32_t bin = (round & 1) ? band_waves - 1 - pos : pos;
  const int32_t slot = (band * band_waves + bin) * slots + round;
  piece_of[slot] = order[i];
}

// wstart[r * (n_windows + 1) + p] = index of the first nonzero of row r whose column lies in window
// p or beyond (p = n_windows: one past the row).  Columns must be sorted within a row.  One thread
// per nonzero fills the entries between its predecessor's window and its own.
HPSPMM_KERNEL __launch_bounds__(kBlock) void sweep_row_windows_kernel(int64_t nnz, const int32_t* __restrict__ nnz_row,
                                                                   const int32_t* __restrict__ rowptr,
                                                                   const int32_t* __restrict__ col, int wshift,
                                                                   int32_t n_windows, int32_t* __restrict__ wstart) {
  const int64_t j = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (j >= nnz) return;
  const int32_t r = nnz_row[j];
  const int32_t lb = rowptr[r], hb = rowptr[r + 1];
  int32_t* w = wstart + (int64_t)r * (n_windows + 1);
  const int32_t p = col[j] >> wshift;
  const int32_t before = (int32_t)j == lb ? -1 : (col[j - 1] >> wshift);
  for (int32_t q = before + 1; q <= p; ++q) w[q] = (int32_t)j;
  if ((int32_t)j == hb - 1)
    for (int32_t q = p + 1; q <= n_windows; ++q) w[q] = hb;
}

// Number of x in [0, n) with x % m == k (k < m).
__device__ __forceinline__ int32_t sweep_count_below(int32_t n, int32_t m, int32_t k) { return (n + m - 1 - k) / m; }

// One workgroup per wavefront of the layout, one thread per window (looped).  For window p the
// thread deals the runs of the wavefront's slots to its P sub-waves, longest run first, each to the
// sub-wave with the shortest chunk so far (ties: lower slot, lower sub-wave - reproducible):
// run_at[slot * n_windows + p] = sub-wave << 28 | position of the run within that sub-wave's chunk.
// The chunk of the wavefront is the longest of its sub-waves: chunk_end[wave * n_windows + p] = end
// of that chunk in the sub-wave streams (inclusive prefix sum over the windows); wave_len[wave] =
// length of every sub-wave stream of the wavefront, rounded up to whole tiles of 32 entries.
template <int P>
__global__ __launch_bounds__(kBlock) void sweep_chunks_kernel(int32_t n_windows, int32_t limit,
                                                              const int32_t* __restrict__ piece_of,
                                                              const int32_t* __restrict__ piece_row,
                                                              const uint32_t* __restrict__ pbase,
                                                              const int32_t* __restrict__ rowptr,
                                                              const int32_t* __restrict__ wstart,
                                                              int32_t* __restrict__ run_at,
                                                              int32_t* __restrict__ chunk_end,
                                                              uint32_t* __restrict__ wave_len) {
  constexpr int WS = P * kSweepSlots;
  __shared__ int32_t s_row[WS], s_lb[WS], s_m[WS], s_k[WS];
  __shared__ uint32_t s_wave[kWavesPerBlock];
  const int64_t wave = blockIdx.x;
  if (threadIdx.x < WS) {
    const int32_t piece = piece_of[wave * WS + threadIdx.x];
    int32_t row = -1, lb = 0, m = 1, k = 0;
    if (piece >= 0) {
      row = piece_row[piece];
      lb = rowptr[row];
      m = (rowptr[row + 1] - lb + limit - 1) / limit;
      k = piece - (int32_t)pbase[row];
    }
    s_row[threadIdx.x] = row;
    s_lb[threadIdx.x] = lb;
    s_m[threadIdx.x] = m;
    s_k[threadIdx.x] = k;
  }
  __syncthreads();
  uint32_t carry = 0;
  for (int32_t p0 = 0; p0 < n_windows; p0 += kBlock) {
    const int32_t p = p0 + threadIdx.x;
    uint32_t longest = 0;
    if (p < n_windows) {
      // key = length << 8 | (255 - slot): sorted downwards, the runs come longest first, ties lower slot first
      int32_t key[WS];
#pragma unroll
      for (int slot = 0; slot < WS; ++slot) {
        const int32_t row = s_row[slot];
        int32_t len = 0;
        if (row >= 0) {
          const int32_t* w = wstart + (int64_t)row * (n_windows + 1) + p;
          const int32_t a = w[0] - s_lb[slot], b = w[1] - s_lb[slot];
          len = sweep_count_below(b, s_m[slot], s_k[slot]) - sweep_count_below(a, s_m[slot], s_k[slot]);
        }
        key[slot] = len > 0 ? (len << 8 | (255 - slot)) : 0;
      }
      // bitonic network over the registers (every index a compile-time constant)
#pragma unroll
      for (int span = 2; span <= WS; span <<= 1) {
#pragma unroll
        for (int step = span >> 1; step > 0; step >>= 1) {
#pragma unroll
          for (int i = 0; i < WS; ++i) {
            const int l = i ^ step;
            if (l > i) {
              const int32_t x = key[i], y = key[l];
              const int32_t hi = x > y ? x : y, lo = x > y ? y : x;
              const bool down = (i & span) == 0;
              key[i] = down ? hi : lo;
              key[l] = down ? lo : hi;
            }
          }
        }
      }
      uint32_t load[P];
      for (int q = 0; q < P; ++q) load[q] = 0;
#pragma unroll
      for (int i = 0; i < WS; ++i) {
        if (key[i] != 0) {
          const int32_t len = key[i] >> 8, slot = 255 - (key[i] & 255);
          int q = 0;
          for (int t = 1; t < P; ++t)
            if (load[t] < load[q]) q = t;
          run_at[(wave * WS + slot) * n_windows + p] = (int32_t)((uint32_t)q << 28 | load[q]);
          load[q] += (uint32_t)len;
        }
      }
      for (int q = 0; q < P; ++q) longest = load[q] > longest ? load[q] : longest;
    }
    uint32_t total;
    const uint32_t before = block_exclusive_scan(longest, s_wave, total);
    if (p < n_windows) chunk_end[wave * n_windows + p] = (int32_t)(carry + before + longest);
    carry += total;
  }
  if (threadIdx.x == 0) wave_len[wave] = (carry + (uint32_t)(kTile - 1)) & ~(uint32_t)(kTile - 1);
}

// stream_len[w] = P * wave_len[w] (entries of the wavefront in the stream arrays); [n_waves] = 0.
HPSPMM_KERNEL __launch_bounds__(kBlock) void sweep_stream_lengths_kernel(int64_t n_waves, int P,
                                                                      const uint32_t* __restrict__ wave_len,
                                                                      uint32_t* __restrict__ stream_len) {
  const int64_t w = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (w > n_waves) return;
  stream_len[w] = w < n_waves ? wave_len[w] * (uint32_t)P : 0u;
}

// Padding everywhere: the padding flag, value index -1 (= the value 0).
HPSPMM_KERNEL __launch_bounds__(kBlock) void sweep_clear_stream_kernel(int64_t n, int32_t* __restrict__ vent,
                                                                    int32_t* __restrict__ vsrc) {
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock) {
    vent[i] = kSweepPad;
    vsrc[i] = -1;
  }
}

// Every nonzero goes to its place: wave_base + sub-wave * wave_len + start of the window's chunk +
// position of its run in the chunk + rank in the run.  One workgroup per wavefront of the layout,
// its threads over the nonzeros of the wavefront's pieces one after the other: reads of a piece are
// consecutive, the entries of a run are written by neighbouring lanes, and what a workgroup writes
// is one wavefront's streams and nothing else, so the L2 sees every line of them completed within a
// short time (one thread per nonzero of the matrix, in matrix order, wrote a few bytes here and a
// few there all over the streams: 2-3 ms instead of well under one on 115 M nonzeros).
HPSPMM_KERNEL __launch_bounds__(kBlock) void sweep_fill_kernel(int32_t n_windows, int wshift, int32_t limit, int32_t slots,
                                                            int32_t lanes, const int32_t* __restrict__ piece_of,
                                                            const int32_t* __restrict__ piece_row,
                                                            const uint32_t* __restrict__ pbase,
                                                            const int32_t* __restrict__ rowptr,
                                                            const int32_t* __restrict__ col,
                                                            const int32_t* __restrict__ wstart,
                                                            const int32_t* __restrict__ run_at,
                                                            const int32_t* __restrict__ chunk_end,
                                                            const uint32_t* __restrict__ wave_base,
                                                            const uint32_t* __restrict__ wave_len,
                                                            const int32_t* __restrict__ stored_at,
                                                            int32_t* __restrict__ vent, int32_t* __restrict__ vsrc) {
  constexpr int kMaxSlots = 64;  // 8 slots for each of at most 8 sub-waves
  __shared__ int32_t s_row[kMaxSlots], s_lb[kMaxSlots], s_m[kMaxSlots], s_k[kMaxSlots], s_size[kMaxSlots];
  __shared__ int32_t s_begin[kMaxSlots + 1];  // entries of the slots before this one
  const int64_t wave = blockIdx.x;
  if ((int)threadIdx.x < kMaxSlots) {
    int32_t row = -1, lb = 0, m = 1, k = 0, size = 0;
    if ((int)threadIdx.x < slots) {
      const int32_t piece = piece_of[wave * slots + threadIdx.x];
      if (piece >= 0) {
        row = piece_row[piece];
        lb = rowptr[row];
        const int32_t len = rowptr[row + 1] - lb;
        m = (len + limit - 1) / limit;
        k = piece - (int32_t)pbase[row];
        size = sweep_count_below(len, m, k);
      }
    }
    s_row[threadIdx.x] = row;
    s_lb[threadIdx.x] = lb;
    s_m[threadIdx.x] = m;
    s_k[threadIdx.x] = k;
    s_size[threadIdx.x] = size;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int32_t sum = 0;
    for (int i = 0; i < kMaxSlots; ++i) {
      s_begin[i] = sum;
      sum += s_size[i];
    }
    s_begin[kMaxSlots] = sum;
  }
  __syncthreads();
  const int64_t base = wave_base[wave];
  const int64_t wlen = wave_len[wave];
  const int32_t* ends = chunk_end + wave * n_windows;
  const int32_t total = s_begin[kMaxSlots];
  const int32_t per_lane = kTile / lanes;
  for (int32_t e = threadIdx.x; e < total; e += kBlock) {
    int slot = 0;  // the last slot with s_begin[slot] <= e (empty slots repeat a value: the last of them has the entries)
#pragma unroll
    for (int step = kMaxSlots / 2; step > 0; step >>= 1)
      if (s_begin[slot + step] <= e) slot += step;
    const int32_t row = s_row[slot], lb = s_lb[slot], m = s_m[slot], k = s_k[slot];
    const int32_t x = e - s_begin[slot];  // the piece's x-th nonzero
    const int32_t j = lb + k + x * m;     // a piece takes every m-th nonzero of its row
    const int32_t c = col[j];
    const int32_t p = c >> wshift;
    const int32_t* w = wstart + (int64_t)row * (n_windows + 1) + p;
    const int32_t first = sweep_count_below(w[0] - lb, m, k);
    const bool last = sweep_count_below(w[1] - lb, m, k) == x + 1;
    const uint32_t at = (uint32_t)run_at[(wave * slots + slot) * n_windows + p];
    const int64_t pos = base + (int64_t)(at >> 28) * wlen + (p > 0 ? ends[p - 1] : 0) + (at & 0x0FFFFFFFu) + (x - first);
    vent[pos] = c | (slot << kSweepColBits) | (last ? kSweepFlush : 0);
    // The value indices of a tile of 32 entries are stored lane-major: lane l of the sub-wave (of
    // `lanes` lanes) fetches 32 / lanes of them with one load, and they belong to the entries l, l +
    // lanes, ... of the tile, so that one gather instruction of the values covers neighbouring entries
    // (mostly one line of the value array per piece instead of one per lane).
    const int32_t u = (int32_t)(pos % kTile);  // the streams start at multiples of 32
    // (col[] may be a copy with every row's columns in increasing order: stored_at[] then says where
    // entry j of the copy lies in the caller's arrays)
    vsrc[pos - u + (u % lanes) * per_lane + u / lanes] = stored_at ? stored_at[j] : j;
  }
}

// Sort keys for bringing the columns of every row into increasing order: pass 1 sorts the nonzeros
// by column (key = col[j], value = j), pass 2, stable, by row (key = row of the value).
HPSPMM_KERNEL __launch_bounds__(kBlock) void sweep_sort_keys_kernel(int64_t nnz, const int32_t* __restrict__ key_of,
                                                                 const int32_t* __restrict__ at,
                                                                 uint32_t* __restrict__ keys, int32_t* __restrict__ vals) {
  for (int64_t q = (int64_t)blockIdx.x * kBlock + threadIdx.x; q < nnz; q += (int64_t)gridDim.x * kBlock) {
    const int32_t j = at ? at[q] : (int32_t)q;
    keys[q] = (uint32_t)key_of[j];
    if (!at) vals[q] = j;
  }
}

// slot_row[slot] = what the slot's result is: row r >= 0 (a whole row, stored to C), ~i (partial
// result row i of a split row) or kSweepUnused.
HPSPMM_KERNEL __launch_bounds__(kBlock) void sweep_slot_rows_kernel(int64_t n_slots, const int32_t* __restrict__ piece_of,
                                                                 const int32_t* __restrict__ piece_row,
                                                                 const uint32_t* __restrict__ pbase,
                                                                 const uint32_t* __restrict__ part_base,
                                                                 const int32_t* __restrict__ rowptr, int32_t limit,
                                                                 int32_t* __restrict__ slot_row) {
  const int64_t s = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (s >= n_slots) return;
  const int32_t piece = piece_of[s];
  int32_t out = kSweepUnused;
  if (piece >= 0) {
    const int32_t row = piece_row[piece];
    const int32_t m = (rowptr[row + 1] - rowptr[row] + limit - 1) / limit;
    out = m == 1 ? row : ~(int32_t)(part_base[row] + ((uint32_t)piece - pbase[row]));
  }
  slot_row[s] = out;
}

// list[] <- every row with more than `limit` nonzeros (which = 1) or with none (which = 0), order
// unspecified; *count must be zero on entry.
HPSPMM_KERNEL __launch_bounds__(kBlock) void sweep_collect_rows_kernel(int64_t rows, const int32_t* __restrict__ rowptr,
                                                                    int32_t limit, int which,
                                                                    int32_t* __restrict__ list,
                                                                    int32_t* __restrict__ count) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  bool hit = false;
  if (i < rows) {
    const int32_t len = rowptr[i + 1] - rowptr[i];
    hit = which ? len > limit : len == 0;
  }
  const uint64_t mask = __ballot(hit);
  if (mask == 0) return;
  const int lane = threadIdx.x & 63;
  int32_t base = 0;
  if (lane == 0) base = atomicAdd(count, (int32_t)__popcll(mask));
  base = __shfl(base, 0);
  if (hit) list[base + __popcll(mask & ((1ull << lane) - 1ull))] = (int32_t)i;
}

// dst[q] = val[vsrc[q]], 0 for padding: the values in the order of the index stream, once, for a
// caller who has declared them constant.
HPSPMM_KERNEL __launch_bounds__(kBlock) void sweep_gather_values_kernel(int64_t n, const int32_t* __restrict__ vsrc,
                                                                     const float* __restrict__ val,
                                                                     float* __restrict__ dst) {
  for (int64_t q = (int64_t)blockIdx.x * kBlock + threadIdx.x; q < n; q += (int64_t)gridDim.x * kBlock)
    dst[q] = vsrc[q] < 0 ? 0.f : val[vsrc[q]];
}

// ---- SpMM kernels ----------------------------------------------------------

// One wavefront per entry of wave_base / wave_len; its P sub-waves consume P streams of wave_len
// entries each, side by side.  kInPlace: vval is the caller's value array and vsrc[q] the index into
// it of stream position q (fetched two tiles ahead, so that the value loads of the next tile never
// wait for their indices); otherwise vval holds the values in stream order.
template <int K, bool kInPlace, int kLd = 0>
__global__ __launch_bounds__(sweep_waves<K>() * 64) void spmm_sweep_kernel(
    SweepLayout lay, const uint32_t* __restrict__ wave_base, const uint32_t* __restrict__ wave_len,
    const int32_t* __restrict__ chunk_end, const int32_t* __restrict__ vent, const float* __restrict__ vval,
    const int32_t* __restrict__ vsrc, const int32_t* __restrict__ slot_row, const float* __restrict__ B,
    const float* __restrict__ zrow, float* __restrict__ partial, float* __restrict__ C, uint32_t ld_arg) {
  constexpr int G = K / 4;
  constexpr int P = 64 / G;
  constexpr int TL = kTile / G;
  const uint32_t ld = row_length<K, kLd>(ld_arg);  // floats between the rows of B and of C
  constexpr int WS = P * kSweepSlots;  // accumulator slots of a wavefront: WS * K floats = 8 KB
  constexpr int WPB = sweep_waves<K>();
  extern __shared__ __attribute__((aligned(16))) unsigned char s_raw[];
  float* s_acc = reinterpret_cast<float*>(s_raw);
  int32_t* s_ent = reinterpret_cast<int32_t*>(s_acc + WPB * WS * K);
  float* s_val = reinterpret_cast<float*>(s_ent + WPB * P * kTileStride);
  int32_t* s_at = reinterpret_cast<int32_t*>(s_val + WPB * P * kTileStride);  // [16] window each wavefront is in

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wv = tid >> 6;
  const int l = lane % G;
  const int q = lane / G;
  const int64_t wave = __builtin_amdgcn_readfirstlane((int)((int64_t)blockIdx.x * WPB + wv));
  float* acc_wave = s_acc + wv * (WS * K);
  const int32_t n_windows = lay.n_windows;

  if (tid < 16) s_at[tid] = tid < WPB ? 0 : INT32_MAX;
#pragma unroll
  for (int i = 0; i < WS * K / 4 / 64; ++i)
    *reinterpret_cast<float4*>(acc_wave + 4 * (i * 64 + lane)) = make_float4(0.f, 0.f, 0.f, 0.f);
  __syncthreads();

  // the window the slowest wavefront of the workgroup is in
  auto slowest = [&]() {
    int32_t least = __hip_atomic_load(&s_at[lane & 15], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) {
      const int32_t o = __shfl_xor(least, off);
      least = o < least ? o : least;
    }
    return __builtin_amdgcn_readfirstlane(least);
  };

  const int32_t len = (int32_t)__builtin_amdgcn_readfirstlane((int)wave_len[wave]);
  const int64_t s = (int64_t)wave_base[wave] + (int64_t)q * len;
  const int64_t e = s + len;
  const int sbase = (wv * P + q) * kTileStride;
  const int32_t* ends = chunk_end + wave * n_windows;

  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  // the plan checks that B is below 4 GB: a 32-bit byte offset
  const int nv = lane_columns<K, kLd>(ld_arg, l);
  const bool in_tile = nv > 0;
  // a lane beyond the tile gathers what lane 0 gathers (a valid address, no branch in the loop); its
  // sums are never stored to C
  const int lg = in_tile ? l : 0;
  auto loadb = [&](int32_t w) {
    const uint32_t off = (uint32_t)(w & kSweepColMask) * (ld * 4u) + (uint32_t)(16 * lg);
    const char* base =
        (w & kSweepPad) ? reinterpret_cast<const char*>(zrow) + 16 * lg : reinterpret_cast<const char*>(B) + off;
    return *reinterpret_cast<const float4*>(base);
  };

  int32_t src[TL], ent[TL];
  float val[TL];
  auto fetch_src = [&](int64_t t) {
    if constexpr (kInPlace) load_run<TL>(src, vsrc, t + l * TL, e, true);
  };
  auto fetch = [&](int64_t t) {
    const int64_t pos = t + l * TL;
    load_run<TL>(ent, vent, pos, e, true);
    if constexpr (kInPlace) {
#pragma unroll
      for (int i = 0; i < TL; ++i) {  // of the tile's entries l, l + G, ...
        // padding (index -1) is the value 0: whatever else it read must not meet the zeros it gathers as inf * 0
        const float v = vval[src[i] < 0 ? 0 : src[i]];
        val[i] = src[i] < 0 ? 0.f : v;
      }
    } else {
      load_run<TL>(val, vval, pos, e, true);
    }
  };
  auto stage = [&]() {
    const int at = sbase + l * TL;
    if constexpr (TL == 4) {
      *reinterpret_cast<int4*>(s_ent + at) = make_int4(ent[0], ent[1], ent[2], ent[3]);
    } else if constexpr (TL == 2) {
      *reinterpret_cast<int2*>(s_ent + at) = make_int2(ent[0], ent[1]);
    } else {
      s_ent[at] = ent[0];
    }
    // the values arrive lane-major (see sweep_fill_kernel) and are staged in processing order
#pragma unroll
    for (int i = 0; i < TL; ++i) s_val[sbase + i * G + l] = val[i];
  };

  // window bookkeeping, uniform over the wavefront: `window` = the one the next tile starts in
  int32_t window = 0;
  int32_t bound = n_windows > 0 ? __builtin_amdgcn_readfirstlane(ends[0]) : INT32_MAX;
  bool waiting = lay.spin_limit > 0;

  fetch_src(s);
  fetch(s);
  fetch_src(s + kTile);
  for (int32_t rel = 0; rel < len; rel += kTile) {
    const int64_t t = s + rel;
    if (rel >= bound) {
      do {
        ++window;
        bound = window < n_windows ? __builtin_amdgcn_readfirstlane(ends[window]) : INT32_MAX;
      } while (rel >= bound);
      if (lane == 0) __hip_atomic_store(&s_at[wv], window, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      int32_t least = slowest();
      if (waiting && window - lay.lead >= least) {
        __builtin_amdgcn_s_setprio(0);
        int spins = 0;
        do {
          if (++spins > lay.spin_limit) {
            waiting = false;
            break;
          }
          __builtin_amdgcn_s_sleep(32);
          least = slowest();
        } while (window - lay.lead >= least);
      }
      // the further ahead of the slowest wavefront of the CU, the lower the priority
      if (lay.priorities) {
        const int32_t ahead = window - least;
        if (ahead <= 0) __builtin_amdgcn_s_setprio(3);
        else if (ahead == 1) __builtin_amdgcn_s_setprio(2);
        else if (ahead == 2) __builtin_amdgcn_s_setprio(1);
        else __builtin_amdgcn_s_setprio(0);
      }
    }
    stage();
    wave_lds_fence();
    if (rel + kTile < len) {
      fetch(t + kTile);
      fetch_src(t + 2 * kTile);
    }
    const int cnt = (len - rel) < kTile ? (len - rel) : kTile;  // a multiple of 8
    for (int u = 0; u < cnt; u += kBatch) {
      int32_t w[kBatch];
      float v[kBatch];
      float4 b[kBatch];
#pragma unroll
      for (int i = 0; i < kBatch; ++i) {
        w[i] = s_ent[sbase + u + i];
        v[i] = s_val[sbase + u + i];
      }
#pragma unroll
      for (int i = 0; i < kBatch; ++i) b[i] = loadb(w[i]);
#pragma unroll
      for (int i = 0; i < kBatch; ++i) {
        fma4(acc, v[i], b[i]);
        if (w[i] < 0) {
          float4* a = reinterpret_cast<float4*>(acc_wave + ((w[i] >> kSweepColBits) & (WS - 1)) * K + 4 * l);
          float4 sum = *a;
          sum.x += acc.x;
          sum.y += acc.y;
          sum.z += acc.z;
          sum.w += acc.w;
          *a = sum;
          acc = make_float4(0.f, 0.f, 0.f, 0.f);
        }
      }
    }
    wave_lds_fence();
  }
  // out of the way of the others
  if (lane == 0) __hip_atomic_store(&s_at[wv], INT32_MAX, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);

  // results: sub-wave q stores slots q * 8 .. q * 8 + 7 (any sub-wave may have added to them)
  wave_lds_fence();
#pragma unroll 1
  for (int i = 0; i < kSweepSlots; ++i) {
    const int slot = q * kSweepSlots + i;
    const int32_t dest = slot_row[wave * WS + slot];
    if (dest == kSweepUnused) continue;
    const float4 sum = *reinterpret_cast<const float4*>(acc_wave + slot * K + 4 * l);
    float* out = dest >= 0 ? C + (uint64_t)(uint32_t)dest * c_row_length<K, kLd>(ld_arg)
                           : partial + (uint64_t)(uint32_t)~dest * K;
    if (in_tile) {  // (what a lane beyond the tile holds is never read)
      if (dest >= 0) store_c_row<kLd, true>(out + 4 * l, sum, nv, c_rows_aligned<kLd>(ld_arg));
      else store_result(out + 4 * l, sum);
    }
  }
}

// Final pass.  Workgroups [0, split_blocks): one sub-wave per split row adds the row's partial
// results in piece order and writes C.  The others: rows without nonzeros get zeros.
template <int K, int kLd = 0>
__global__ __launch_bounds__(kBlock) void spmm_sweep_final_kernel(
    const int32_t* __restrict__ rowptr, int32_t limit, const int32_t* __restrict__ split_rows, int64_t n_split,
    int64_t split_blocks, const uint32_t* __restrict__ part_base, const int32_t* __restrict__ zero_rows,
    int64_t n_zero, const float* __restrict__ partial, float* __restrict__ C, uint32_t ld_arg) {
  constexpr int G = K / 4;
  constexpr int P = 64 / G;
  const uint32_t ld = c_row_length<K, kLd>(ld_arg);  // floats between the rows of C
  const bool c_aligned = c_rows_aligned<kLd>(ld_arg);
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int l = lane % G;
  const int sub = (tid >> 6) * P + lane / G;
  if ((int64_t)blockIdx.x >= split_blocks) {
    const int64_t idx = ((int64_t)blockIdx.x - split_blocks) * (kWavesPerBlock * P) + sub;
    if (idx >= n_zero) return;
    const int nvz = lane_columns<K, kLd>(ld_arg, l);
    if (nvz > 0)
      store_c_row<kLd, false>(C + (uint64_t)(uint32_t)zero_rows[idx] * ld + 4 * l, make_float4(0.f, 0.f, 0.f, 0.f), nvz, c_aligned);
    return;
  }
  const int64_t idx = (int64_t)blockIdx.x * (kWavesPerBlock * P) + sub;
  if (idx >= n_split) return;
  const int32_t row = split_rows[idx];
  const int32_t m = (rowptr[row + 1] - rowptr[row] + limit - 1) / limit;
  const float* src = partial + (uint64_t)part_base[row] * K + 4 * l;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  int32_t k = 0;
  for (; k + kBatch <= m; k += kBatch) {
    float4 part[kBatch];
#pragma unroll
    for (int i = 0; i < kBatch; ++i) part[i] = *reinterpret_cast<const float4*>(src + (uint64_t)(k + i) * K);
#pragma unroll
    for (int i = 0; i < kBatch; ++i) {
      acc.x += part[i].x;
      acc.y += part[i].y;
      acc.z += part[i].z;
      acc.w += part[i].w;
    }
  }
  for (; k < m; ++k) {
    const float4 t = *reinterpret_cast<const float4*>(src + (uint64_t)k * K);
    acc.x += t.x;
    acc.y += t.y;
    acc.z += t.z;
    acc.w += t.w;
  }
  const int nv = lane_columns<K, kLd>(ld_arg, l);
  if (nv > 0) store_c_row<kLd, false>(C + (uint64_t)(uint32_t)row * ld + 4 * l, acc, nv, c_aligned);
}

}  // namespace hpspmm
