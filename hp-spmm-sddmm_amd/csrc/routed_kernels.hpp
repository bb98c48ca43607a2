// gfx950 device code of the *routed* strategy for FP32 CSR SpMM.
//
// On power-law graphs a few thousand columns receive most of the nonzeros, yet
// with eight XCDs each seeing an eighth of a mixed stream those rows of B do
// not survive in any 4 MB L2 (measured: ~15 % L2 hits, the gather runs at the
// fabric's ~7.4 TB/s while an L2-resident gather runs at ~22 TB/s).  The routed
// strategy makes the hot rows L2-resident by construction:
//
//   * every column belongs to one of 8 slices: the most referenced columns by
//     popularity rank, round robin, so that the slices carry equal load, the
//     rest by a hash of the index.  Slice x of B is only ever read by
//     workgroups running on XCD x (workgroup b runs on XCD b % 8), so each L2
//     sees an eighth of the columns and keeps the hot ones (measured on the
//     233k-vertex social graph, K=128: 6.6 ms -> 4.5 ms).  A slice can further
//     be cut into up to 7 phases that an XCD works through one after the other,
//     each with the same mix of hot and cold columns;
//   * the most referenced rows of B are additionally copied, slice by slice,
//     into a compact buffer at the start of every SpMM, which takes them off
//     whatever memory channels their original addresses collide on;
//   * degree binning: only rows with at least `min_row_nnz` nonzeros are
//     routed - a short row would pay one partial-result row per class it
//     touches for a handful of gathers.  Routed rows are numbered 0 ..
//     n_routed-1 in row order; a nonzero of a routed row belongs to the hub
//     class (phase, slice) of its column, all nonzeros of a short row to the
//     last ("cold") class.  The plan lays the nonzeros out class by class, each
//     class in row order, as column (~compact-buffer row if the column is
//     cached) and row arrays (routed-row number in the hub classes, row in the
//     cold class), plus the position of every stored nonzero in that order;
//     every SpMM first scatters the caller's values into the same order
//     (reading them in place would fetch each line of the value array once per
//     class: 3.7 GB instead of 0.46 GB on the social graph);
//   * inside a class the work is cut into fixed-length segments exactly as in
//     the segments strategy.  A run (the nonzeros of one row in one class)
//     that lies inside one segment is complete: in a hub class it is stored to
//     the routed row's partial-result slot of the class, in the cold class
//     straight to C (a short row has no other class).  Runs that cross a
//     segment boundary go through the carry slots;
//   * a final kernel adds, for every routed row, its class results in class
//     order and writes C; it also finishes the short rows whose run crossed a
//     segment boundary and writes zeros for empty rows.  No atomics; results
//     are bit-reproducible for a given plan.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "scan_kernels.hpp"
#include "spmm_kernels.hpp"

namespace hpspmm {

constexpr int kSlices = 8;                 // column slices, one per XCD
constexpr int kMaxSub = 7;                 // phases per slice, at most
constexpr int kMaxHub = kSlices * kMaxSub;  // hub classes, at most: fits one wavefront's lanes
constexpr int kMaxClasses = kMaxHub + 1;   // + the cold class

// What the final kernel does with a short row.
constexpr uint8_t kActionNone = 0;   // the main kernel stored it (or it is routed)
constexpr uint8_t kActionZero = 1;   // no nonzeros: write zeros
constexpr uint8_t kActionCross = 2;  // its run crosses a segment boundary: add the carry slots

// Class x < nhub = 8 * nsub is (phase x / 8, slice x % 8); class nhub is the cold class.
struct RoutedLayout {
  int64_t cls_begin[kMaxClasses];    // first virtual index of the class (multiple of the workgroup quantum)
  int64_t cls_end[kMaxClasses];      // one past its last real entry
  int64_t cls_blocks[kMaxClasses];   // workgroups needed by the class
  int64_t phase_begin[kMaxSub + 1];  // first workgroup of phase p (a multiple of 8); [nsub]: of the cold class
  int64_t rows;
  int64_t n_routed;
  int shift;  // log2(segment length)
  int nsub;   // phases
  int nhub;   // 8 * nsub
  // Column-tile phases (tile_width > 0, then nsub = 1): B and C are worked through in `tiles` tiles of
  // tile_width columns, one after the other on all XCDs; the workgroups of tile t are
  // [t * tile_grid, (t + 1) * tile_grid), its first hub_grid (a multiple of 8) the hub classes, the
  // next cold_grid the cold class, the rest write the tile's zeros of the rows without nonzeros.
  int tile_width;
  int tiles;
  int64_t tile_grid;
  int64_t hub_grid;
  int64_t cold_grid;
  int64_t n_zero;     // rows without nonzeros (listed in zero_rows[])
  int64_t rows_of_b;  // = columns of A
  // Its workgroups have tile_waves wavefronts and keep the lds_rows most referenced rows of their
  // class (of the tile in hand) in LDS: in hub class x the first lds_rows compact-buffer rows of
  // slice x, in the cold class the first lds_rows / 8 of every slice (ranks 0 .. lds_rows - 1 overall).
  int tile_waves;
  int lds_rows;
  int64_t hub_rows_per_slice;
};

// Entry word of the class-major order under column-tile phases: bit 31 = the row of B is in the
// compact buffer (bits 0..29 = its slot there) instead of B (bits 0..29 = the column); bit 30 = first
// entry of its run (the nonzeros of one row in one class).  The rows of the runs are kept run by run
// (run_row[]), not nonzero by nonzero, with the run of every segment's first entry (seg_run[]).
constexpr int32_t kRunStart = 1 << 30;
constexpr int32_t kInLds = 1 << 29;  // the row is among those the workgroup keeps in LDS (bits 0..28 = which)
constexpr int32_t kEntryPayload = kInLds - 1;
constexpr int kRoutedTileWaves = 16;  // wavefronts per workgroup of the column-tile kernel
constexpr int kTileZeroRows = 8;  // rows without nonzeros written per sub-wave of a zero-writing workgroup
constexpr int kTileLdsPad = 4;  // floats between the rows of the LDS copy: rows of different sub-waves on different banks

// dst[q] = val[src[q]]: the values in the plan's order, once, for a caller who has declared them constant.
HPSPMM_KERNEL __launch_bounds__(kBlock) void routed_gather_values_kernel(int64_t n, const int32_t* __restrict__ src,
                                                                      const float* __restrict__ val,
                                                                      float* __restrict__ dst) {
  for (int64_t q = (int64_t)blockIdx.x * kBlock + threadIdx.x; q < n; q += (int64_t)gridDim.x * kBlock)
    dst[q] = val[src[q]];
}

// Chunk tables for the value scatter.  The stored nonzeros are cut into chunks
// of kPermChunk consecutive ones.  Inside a chunk the nonzeros of one class
// occupy consecutive positions of the class-major order (both orders keep the
// stored order within a class), so a chunk maps to at most one run per class:
// chunk_base[c * ncls + x] = first position of class x's run, chunk_pref[c *
// ncls + x] = number of the chunk's nonzeros in classes < x, and lslot[j] =
// chunk_pref + (position - chunk_base) = rank of nonzero j when its chunk is
// sorted by position.  One workgroup per chunk.
constexpr int kPermChunk = 4096;

// Start of every SpMM, two jobs in one launch.  Workgroups [0, gather_blocks):
// Bhot[s, :] = B[src[s], :] for every compact-buffer row with a source column
// (src[s] >= 0).  The others, one per chunk of kPermChunk stored nonzeros:
// the caller's values are brought into the plan's class-major order.  A gather
// in class order would fetch every line of val once per class, a scatter of
// single values costs one L2 transaction for every two or three of them; so
// the chunk is sorted by destination in LDS (lslot) and written out run by
// run in full lines (233k-vertex social graph: 0.28 ms for the plain scatter).
template <int K, int kLd = 0>
__global__ __launch_bounds__(kBlock) void routed_prepare_kernel(int64_t n_bhot, int64_t gather_blocks,
                                                                const int32_t* __restrict__ src,
                                                                const float* __restrict__ B,
                                                                float* __restrict__ Bhot, int64_t nnz, int ncls,
                                                                const float* __restrict__ val,
                                                                const uint16_t* __restrict__ lslot,
                                                                const int32_t* __restrict__ chunk_base,
                                                                const int32_t* __restrict__ chunk_pref,
                                                                float* __restrict__ vval, uint32_t ld_arg,
                                                                int tile_width = 0) {
  constexpr int G = K / 4;
  __shared__ float s_buf[kPermChunk];
  __shared__ int32_t s_base[kMaxClasses];
  __shared__ int32_t s_pref[kMaxClasses + 1];
  if ((int64_t)blockIdx.x < gather_blocks) {
    const int64_t t = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    const int64_t s = t / G;
    const int l = (int)(t % G);
    if (s >= n_bhot) return;
    const int32_t c = src[s];
    if (c < 0) return;
    // column-tile phases keep the buffer tile by tile (tile t of every cached row, then tile t + 1),
    // so that what one phase reads is one dense stretch of memory
    const int tile = tile_width ? 4 * l / tile_width : 0;
    float* dst = tile_width ? Bhot + ((uint64_t)tile * n_bhot + s) * tile_width + (4 * l - tile * tile_width)
                            : Bhot + (uint64_t)s * K + 4 * l;
    *reinterpret_cast<float4*>(dst) =
        lane_columns<K, kLd>(ld_arg, l) > 0 ? load_b_ld(B, c, l, row_length<K, kLd>(ld_arg)) : make_float4(0.f, 0.f, 0.f, 0.f);
    return;
  }
  const int64_t chunk = (int64_t)blockIdx.x - gather_blocks;
  const int64_t j0 = chunk * kPermChunk;
  const int n = nnz - j0 < kPermChunk ? (int)(nnz - j0) : kPermChunk;
  for (int x = threadIdx.x; x < ncls; x += kBlock) {
    s_base[x] = chunk_base[chunk * ncls + x];
    s_pref[x] = chunk_pref[chunk * ncls + x];
  }
  if (threadIdx.x == 0) s_pref[ncls] = n;
  constexpr int kPer = kPermChunk / kBlock;
  float v[kPer];
  uint16_t q[kPer];
#pragma unroll
  for (int i = 0; i < kPer; ++i) {
    const int t = i * kBlock + threadIdx.x;
    v[i] = t < n ? val[j0 + t] : 0.f;
    q[i] = t < n ? lslot[j0 + t] : (uint16_t)0;
  }
#pragma unroll
  for (int i = 0; i < kPer; ++i)
    if (i * kBlock + (int)threadIdx.x < n) s_buf[q[i]] = v[i];
  __syncthreads();
  // thread t of every pass writes sorted element t: consecutive threads, consecutive addresses within a run
  int x = 0;
#pragma unroll 1
  for (int i = 0; i < kPer; ++i) {
    const int t = i * kBlock + threadIdx.x;
    if (t >= n) break;
    while (s_pref[x + 1] <= t) ++x;  // t grows with i, so the class only moves forward
    vval[s_base[x] + (t - s_pref[x])] = s_buf[t];
  }
}

// ---- SpMM kernels ----------------------------------------------------------

// Workgroups [phase_begin[p], phase_begin[p + 1]): phase p; its workgroup number
// i serves class (p, i % 8) - and runs on XCD i % 8 - as that class's i / 8-th
// workgroup.  Workgroups from phase_begin[nsub] on: the cold class.  The
// hardware starts workgroups in index order, so every XCD works through its
// slice one phase, i.e. one set of B rows, at a time.
// Each sub-wave owns one segment of its class; see the carry rule of the
// segments kernel - in a hub class "stored to C" becomes "stored to the routed
// row's partial-result slot of the class".
// kInPlace: vval is the caller's value array in its own order and vsrc[q] the index into it of
// the class-major position q (column-range slices: consecutive positions of a run are consecutive
// indices, so these loads stay coalesced).  kHub: vcol may hold ~(compact-buffer row); without it
// every entry is a plain column and the gather address is B plus a 32-bit byte offset (the plan
// checks that B is below 4 GB), three instructions instead of eight.
template <int K, bool kInPlace, bool kHub, int kLd = 0>
__global__ __launch_bounds__(kBlock) void spmm_routed_kernel(RoutedLayout lay, const int32_t* __restrict__ rvptr,
                                                             const int32_t* __restrict__ coldptr,
                                                             const int32_t* __restrict__ vcol,
                                                             const float* __restrict__ vval,
                                                             const int32_t* __restrict__ vsrc,
                                                             const int32_t* __restrict__ vrow,
                                                             const float* __restrict__ B,
                                                             const float* __restrict__ Bhot,
                                                             float* __restrict__ partial,
                                                             float* __restrict__ carry, float* __restrict__ C,
                                                             int64_t first_block, uint32_t ld_arg) {
  constexpr int G = K / 4;
  constexpr int P = 64 / G;
  const uint32_t ld = row_length<K, kLd>(ld_arg);  // floats between the rows of B and of C
  constexpr int TL = kTile / G;
  __shared__ __attribute__((aligned(16))) int32_t s_col[kWavesPerBlock * P * kTileStride];
  __shared__ __attribute__((aligned(16))) float s_val[kWavesPerBlock * P * kTileStride];
  __shared__ __attribute__((aligned(16))) int32_t s_row[kWavesPerBlock * P * kTileStride];

  // first_block: 0 in an ordinary launch; a diagnostic launch of one part of the grid passes the
  // number of its first workgroup (a multiple of 8, so that the workgroup -> XCD dealing is kept)
  const int64_t bid = (int64_t)blockIdx.x + first_block;
  const int nhub = lay.nhub;
  int p = 0;
  while (p < lay.nsub && bid >= lay.phase_begin[p + 1]) ++p;
  const int64_t rel = bid - lay.phase_begin[p];
  const bool hub = p < lay.nsub;
  int x;
  int64_t i;
  if (hub) {
    x = p * kSlices + (int)(rel % kSlices);
    i = rel / kSlices;
  } else {
    x = nhub;
    i = rel;
  }
  if (i >= lay.cls_blocks[x]) return;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int l = lane % G;
  const int nv = lane_columns<K, kLd>(ld_arg, l);
  const bool in_tile = nv > 0;
  const bool c_aligned = c_rows_aligned<kLd>(ld_arg);
  const int shift = lay.shift;
  const int64_t g = (lay.cls_begin[x] >> shift) + (i * kWavesPerBlock + (tid >> 6)) * P + lane / G;
  const int64_t s = g << shift;
  const int64_t cls_end = lay.cls_end[x];
  if (s >= cls_end) return;
  const int64_t e = (s + ((int64_t)1 << shift)) < cls_end ? (s + ((int64_t)1 << shift)) : cls_end;
  const int sbase = ((tid >> 6) * P + lane / G) * kTileStride;
  // first index of a run: rvptr[number * nhub + x] in a hub class, coldptr[row] in the cold class
  const int32_t* vp = hub ? rvptr + x : coldptr;
  const int64_t vstride = hub ? nhub : 1;
  float* out = hub ? partial + (uint64_t)x * K : C;
  const uint64_t ostride = hub ? (uint64_t)nhub * K : (uint64_t)c_row_length<K, kLd>(ld_arg);

  int32_t cur = vrow[s];
  bool head_pending = (int64_t)vp[(int64_t)cur * vstride] < s;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);

  auto flush_to = [&](bool is_tail) {
    const bool to_c = !hub && !head_pending && !is_tail;  // a row of C; else a carry slot or a partial row (aligned, K floats)
    float* dst = head_pending ? carry + (uint64_t)(2 * g) * K
                              : (is_tail ? carry + (uint64_t)(2 * g + 1) * K : out + (uint64_t)(uint32_t)cur * ostride);
    head_pending = false;
    if (in_tile) {  // (what a lane beyond the tile holds is never read)
      if (to_c) store_c_row<kLd, true>(dst + 4 * l, acc, nv, c_aligned);
      else store_result(dst + 4 * l, acc);
    }
  };
  auto flush = [&]() { flush_to(false); };
  // a lane beyond the tile gathers what lane 0 gathers (a valid address, no branch in the loop); its
  // sums are never stored
  const int lg = in_tile ? l : 0;
  auto loadb = [&](int32_t c) {
    if constexpr (kHub) {
      return load_b_hub_ld<K, true>(B, Bhot, c, lg, ld);
    } else {
      const uint32_t off = (uint32_t)c * (ld * 4u) + (uint32_t)(16 * lg);
      return *reinterpret_cast<const float4*>(reinterpret_cast<const char*>(B) + off);
    }
  };

  // the plan's arrays are allocated by the library, hence always aligned for the vector loads
  // In place the value of a position needs its index first: the indices are fetched two tiles ahead
  // (`src`), so that the value loads of the next tile never wait for them - fetched together with
  // the values, every tile began with a full memory round trip (social graph, K = 32: +0.16 ms).
  int32_t src[TL];
  auto fetch_src = [&](int64_t t) {
    if constexpr (kInPlace) load_run<TL>(src, vsrc, t + l * TL, e, true);  // 0 beyond e: a readable index
  };
  auto fetch = [&](TileRegs<TL>& m, int64_t t) {
    const int64_t q = t + l * TL;
    load_run<TL>(m.c, vcol, q, e, true);
    if constexpr (kInPlace) {
#pragma unroll
      for (int i = 0; i < TL; ++i) m.v[i] = vval[src[i]];
    } else {
      load_run<TL>(m.v, vval, q, e, true);
    }
    load_run<TL>(m.r, vrow, q, e, true);
  };
  TileRegs<TL> m;
  fetch_src(s);
  fetch(m, s);
  fetch_src(s + kTile);
  for (int64_t t = s; t < e; t += kTile) {
    stage_tile<TL>(m, sbase + l * TL, s_col, s_val, s_row);
    wave_lds_fence();
    if (t + kTile < e) {
      fetch(m, t + kTile);
      fetch_src(t + 2 * kTile);
    }
    const int cnt = (e - t) < kTile ? (int)(e - t) : kTile;
    consume_tile(cnt, sbase, s_col, s_val, s_row, cur, acc, loadb, flush);
    wave_lds_fence();
  }
  flush_to((int64_t)vp[(int64_t)(cur + 1) * vstride] > e);
}

// The same work under column-tile phases (RoutedLayout::tile_width = W): workgroup b serves tile
// b / tile_grid of B and C - W columns of rows that are `ld` floats long - and, within the tile's
// range of workgroups, hub class (b % 8) - on XCD b % 8 - or the cold class.  All XCDs are on one
// tile at a time, so an L2 has to hold W / ld of what it would of whole rows: four times as many of
// its slice's hot rows of B stay resident at W = 32, ld = 128, for no partial-result row more (the
// runs of a row in the 8 classes are what they were; every tile writes its W columns of them).  The
// price: the streams are read once per tile - hence entry words that carry the run starts (8 bytes
// per nonzero with the value, instead of 12 with a row word) - and every gather is W * 4 bytes.
// Carry slots and partial-result rows are `ld` floats long, as the final kernel reads them.
// WPB = wavefronts per workgroup (RoutedLayout::tile_waves).  Dynamic LDS: the staging tiles of the
// workgroup's sub-waves, then lds_rows rows of W + kTileLdsPad floats: the most referenced rows of the
// workgroup's class, copied from the compact buffer when the workgroup starts.  A gather is one flat
// load whose address is selected between that copy, the compact buffer and B.  (What bounds the
// kernel is how many requests a CU's L1 can have under way to the L2: with L2 hits and misses mixed
// it sustains about 115 G lines/s, the fabric idling - every gather the LDS serves is one request fewer.)
template <int W, int WPB>
__global__ __launch_bounds__(WPB * 64) void spmm_routed_tiles_kernel(
    RoutedLayout lay, const int32_t* __restrict__ rvptr, const int32_t* __restrict__ coldptr,
    const int32_t* __restrict__ vent, const float* __restrict__ vval, const int32_t* __restrict__ run_row,
    const int32_t* __restrict__ seg_run, const int32_t* __restrict__ zero_rows, const float* __restrict__ B,
    const float* __restrict__ Bhot, float* __restrict__ partial, float* __restrict__ carry, float* __restrict__ C,
    int64_t first_block, uint32_t ld, int64_t n_bhot) {
  constexpr int G = W / 4;
  constexpr int P = 64 / G;
  constexpr int TL = kTile / G;
  constexpr int kStage = WPB * P * kTileStride;
  constexpr int kRow = W + kTileLdsPad;
  extern __shared__ __attribute__((aligned(16))) unsigned char s_raw[];
  int32_t* s_col = reinterpret_cast<int32_t*>(s_raw);
  float* s_val = reinterpret_cast<float*>(s_col + kStage);
  int32_t* s_row = reinterpret_cast<int32_t*>(s_val + kStage);
  float* s_b = reinterpret_cast<float*>(s_row + kStage);  // [lds_rows][kRow]

  const int64_t bid = (int64_t)blockIdx.x + first_block;
  const int64_t tile = bid / lay.tile_grid;
  const int64_t rel = bid - tile * lay.tile_grid;
  const int nhub = lay.nhub;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int l = lane % G;
  const uint32_t k0 = (uint32_t)tile * W;  // first column of the tile
  if (rel >= lay.hub_grid + lay.cold_grid) {
    // The tile's columns of the rows without nonzeros, kTileZeroRows rows per sub-wave, after the
    // tile's other work (as part of the final kernel these rows were half its time; spread among the
    // hub workgroups instead, their lines pushed rows of B out of the L2s and cost more than they hid).
    const int64_t first = ((rel - lay.hub_grid - lay.cold_grid) * (WPB * P) + (tid >> 6) * P + lane / G) * kTileZeroRows;
    const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int64_t j = first; j < first + kTileZeroRows && j < lay.n_zero; ++j)
      store_result(C + (uint64_t)(uint32_t)zero_rows[j] * ld + k0 + 4 * l, zero);
    return;
  }
  const bool hub = rel < lay.hub_grid;
  const int x = hub ? (int)(rel % kSlices) : nhub;
  const int64_t i = hub ? rel / kSlices : rel - lay.hub_grid;
  if (i >= lay.cls_blocks[x]) return;

  const float* hot_tile = Bhot + (uint64_t)tile * (uint64_t)n_bhot * W;

  // the class's most referenced rows (of this tile) into LDS; every thread of the workgroup reaches the barrier
  {
    const int rows = lay.lds_rows;
    const int per = rows / kSlices;
    for (int j = tid; j < rows * G; j += WPB * 64) {
      const int slot = j / G, part = j - slot * G;
      const int64_t src = hub ? (int64_t)x * lay.hub_rows_per_slice + slot
                              : (int64_t)(slot / per) * lay.hub_rows_per_slice + slot % per;
      *reinterpret_cast<float4*>(s_b + slot * kRow + 4 * part) =
          *reinterpret_cast<const float4*>(hot_tile + (uint64_t)src * W + 4 * part);
    }
    __syncthreads();
  }

  const int shift = lay.shift;
  const int64_t g = (lay.cls_begin[x] >> shift) + (i * WPB + (tid >> 6)) * P + lane / G;
  const int64_t s = g << shift;
  const int64_t cls_end = lay.cls_end[x];
  if (s >= cls_end) return;
  const int64_t e = (s + ((int64_t)1 << shift)) < cls_end ? (s + ((int64_t)1 << shift)) : cls_end;
  const int sbase = ((tid >> 6) * P + lane / G) * kTileStride;
  const int32_t* vp = hub ? rvptr + x : coldptr;
  const int64_t vstride = hub ? nhub : 1;
  float* out = (hub ? partial + (uint64_t)x * ld : C) + k0 + 4 * l;
  const uint64_t ostride = hub ? (uint64_t)nhub * ld : (uint64_t)ld;
  float* cslot = carry + (uint64_t)(2 * g) * ld + k0 + 4 * l;
  const float* bt = B + k0 + 4 * l;
  const float* hot_t = hot_tile + 4 * l;
  const float* lds_t = s_b + 4 * l;

  // `run` = the run of the entry before the next tile to be fetched: to begin with, the run of the
  // segment's first entry, less one if that entry starts it
  const int32_t first_run = seg_run[g];
  int32_t run = first_run - ((vent[s] & kRunStart) != 0);
  int32_t cur = run_row[first_run];
  bool head_pending = (int64_t)vp[(int64_t)cur * vstride] < s;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);

  auto flush_to = [&](bool is_tail) {
    float* dst = head_pending ? cslot : (is_tail ? cslot + ld : out + (uint64_t)(uint32_t)cur * ostride);
    head_pending = false;
    store_result(dst, acc);
  };
  auto flush = [&]() { flush_to(false); };
  auto loadb = [&](int32_t c) {
    const uint32_t idx = (uint32_t)(c & kEntryPayload);
    const float* mem = c < 0 ? hot_t + (uint64_t)idx * W : bt + (uint64_t)idx * ld;
    const float* src = (c & kInLds) ? lds_t + idx * kRow : mem;
    return *reinterpret_cast<const float4*>(src);
  };
  // One tile of entries into registers: entry words and values as they lie, the row of every entry
  // from the run starts - a lane counts those among its TL entries, the sub-wave scans the counts, and
  // run_row[] (a few lines, reused by every tile of the segment) gives the rows.
  auto fetch = [&](TileRegs<TL>& m, int64_t t) {
    const int64_t q = t + l * TL;
    load_run<TL>(m.c, vent, q, e, true);  // 0 beyond e: a plain entry of the run before
    load_run<TL>(m.v, vval, q, e, true);
    int32_t starts = 0;
#pragma unroll
    for (int j = 0; j < TL; ++j) starts += (m.c[j] & kRunStart) != 0;
    int32_t incl = starts;
#pragma unroll
    for (int off = 1; off < G; off <<= 1) {
      const int32_t o = __shfl_up(incl, off, G);
      if (l >= off) incl += o;
    }
    int32_t at = run + incl - starts;
#pragma unroll
    for (int j = 0; j < TL; ++j) {
      at += (m.c[j] & kRunStart) != 0;
      m.r[j] = run_row[at];
    }
    run += __shfl(incl, G - 1, G);
  };
  TileRegs<TL> m;
  fetch(m, s);
  for (int64_t t = s; t < e; t += kTile) {
    stage_tile<TL>(m, sbase + l * TL, s_col, s_val, s_row);
    wave_lds_fence();
    if (t + kTile < e) fetch(m, t + kTile);
    const int cnt = (e - t) < kTile ? (int)(e - t) : kTile;
    consume_tile(cnt, sbase, s_col, s_val, s_row, cur, acc, loadb, flush);
    wave_lds_fence();
  }
  flush_to((int64_t)vp[(int64_t)(cur + 1) * vstride] > e);
}

// Bytes of dynamic LDS of one such workgroup.
template <int W, int WPB>
constexpr size_t routed_tiles_lds_bytes(int lds_rows) {
  return (size_t)3 * WPB * (64 / (W / 4)) * kTileStride * 4 + (size_t)lds_rows * (W + kTileLdsPad) * 4;
}

// list[] <- every row whose action byte equals `which` (order unspecified); *count must be zero on entry.
// A workgroup looks at kCollectRows consecutive rows, 8 per thread, and reserves its part of the list with
// one atomic (one per wavefront of 64 rows took 0.44 ms over 2.4 M rows: 38k atomics on one address).
constexpr int kCollectPerThread = 8;
constexpr int kCollectRows = kBlock * kCollectPerThread;
HPSPMM_KERNEL __launch_bounds__(kBlock) void routed_collect_rows_kernel(int64_t rows, const uint8_t* __restrict__ action,
                                                                     uint8_t which, int32_t* __restrict__ list,
                                                                     int32_t* __restrict__ count) {
  __shared__ uint32_t s_wave[kWavesPerBlock];
  __shared__ int32_t s_base;
  const int64_t first = (int64_t)blockIdx.x * kCollectRows + (int64_t)threadIdx.x * kCollectPerThread;
  uint32_t hits = 0;  // bit j: row first + j is wanted
#pragma unroll
  for (int j = 0; j < kCollectPerThread; ++j)
    if (first + j < rows && action[first + j] == which) hits |= 1u << j;
  uint32_t total;
  const uint32_t before = block_exclusive_scan((uint32_t)__popc(hits), s_wave, total);
  if (threadIdx.x == 0) s_base = total ? atomicAdd(count, (int32_t)total) : 0;
  __syncthreads();
  int32_t at = s_base + (int32_t)before;
#pragma unroll
  for (int j = 0; j < kCollectPerThread; ++j)
    if (hits & (1u << j)) list[at++] = (int32_t)(first + j);
}

// Final pass, one sub-wave per listed row, three parts.
// Workgroups [0, routed_blocks): routed row number i gets the sum of its class
// results - per class the partial-result slot if the run lies in one segment,
// else tail[ga] + head[ga+1] + ... + head[gb] from the carry slots.  The
// kernel is a chain of dependent loads per row, so it is built to have few
// links: the row's 2 * nhub run bounds come in with one coalesced load and are
// kept in wave-local LDS; then, eight classes at a time, the first slot of
// every run (partial or tail); then the second slot of the runs that have one
// (with segments of 512 nonzeros and runs of some tens about one run in eight
// crosses a segment boundary, i.e. most rows have one); then, for a hub row's
// runs over three or more segments, the remaining heads.  The order of the
// additions is therefore: all first slots in class order, all second slots in
// class order, the remaining heads in class and segment order - fixed by the
// plan, so results stay bit-reproducible.
// Workgroups [routed_blocks, routed_blocks + cross_blocks): short rows whose
// cold-class run crossed a segment boundary, from the carry slots alone.
// The rest: rows without nonzeros, which get zeros.
// Rows in none of the lists were stored by the main kernel.
template <int K, int kLd = 0>
__global__ __launch_bounds__(kBlock) void spmm_routed_final_kernel(
    RoutedLayout lay, const int32_t* __restrict__ rvptr, const int32_t* __restrict__ coldptr,
    const int32_t* __restrict__ routed_rows, int64_t routed_blocks, const int32_t* __restrict__ cross_rows,
    int64_t n_cross, int64_t cross_blocks, const int32_t* __restrict__ zero_rows, int64_t n_zero,
    const float* __restrict__ partial, const float* __restrict__ carry, float* __restrict__ C, uint32_t ld_arg) {
  constexpr int G = K / 4;
  constexpr int P = 64 / G;
  const uint32_t ld = c_row_length<K, kLd>(ld_arg);  // floats between the rows of C
  const bool c_aligned = c_rows_aligned<kLd>(ld_arg);
  constexpr int kGroup = kSlices;  // classes whose loads are in flight together; divides nhub
  __shared__ int32_t s_bounds[kWavesPerBlock * P][2 * kMaxHub + 1];  // odd stride: sub-waves on different banks
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int l = lane % G;
  const int nv = lane_columns<K, kLd>(ld_arg, l);
  const bool in_tile = nv > 0;
  const int shift = lay.shift;
  const int nhub = lay.nhub;
  const float* cbase = carry + 4 * l;
  const int sub = (tid >> 6) * P + lane / G;  // sub-wave within the workgroup

  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  auto add = [&](const float4& t) {
    acc.x += t.x;
    acc.y += t.y;
    acc.z += t.z;
    acc.w += t.w;
  };
  // acc += head[g] for g in [g0, gb], 8 slots in flight at a time, added in segment order
  auto add_heads = [&](int64_t g0, int64_t gb) {
    int64_t g = g0;
    for (; g + kBatch <= gb + 1; g += kBatch) {
      float4 slot[kBatch];
#pragma unroll
      for (int t = 0; t < kBatch; ++t)
        slot[t] = *reinterpret_cast<const float4*>(cbase + (uint64_t)(2 * (g + t)) * K);
#pragma unroll
      for (int t = 0; t < kBatch; ++t) add(slot[t]);
    }
    for (; g <= gb; ++g) add(*reinterpret_cast<const float4*>(cbase + (uint64_t)(2 * g) * K));
  };

  if ((int64_t)blockIdx.x >= routed_blocks + cross_blocks) {
    const int64_t idx = ((int64_t)blockIdx.x - routed_blocks - cross_blocks) * (kWavesPerBlock * P) + sub;
    if (idx >= n_zero) return;
    if (in_tile) store_c_row<kLd, false>(C + (uint64_t)(uint32_t)zero_rows[idx] * ld + 4 * l, acc, nv, c_aligned);
    return;
  }
  if ((int64_t)blockIdx.x >= routed_blocks) {
    const int64_t idx = ((int64_t)blockIdx.x - routed_blocks) * (kWavesPerBlock * P) + sub;
    if (idx >= n_cross) return;
    const int64_t row = cross_rows[idx];
    const int64_t ga = coldptr[row] >> shift;
    const int64_t gb = (coldptr[row + 1] - 1) >> shift;
    add(*reinterpret_cast<const float4*>(cbase + (uint64_t)(2 * ga + 1) * K));
    add_heads(ga + 1, gb);
    if (in_tile) store_c_row<kLd, false>(C + (uint64_t)row * ld + 4 * l, acc, nv, c_aligned);
    return;
  }
  const int64_t idx = (int64_t)blockIdx.x * (kWavesPerBlock * P) + sub;
  if (idx >= lay.n_routed) return;
  const int64_t row = routed_rows[idx];
  // bounds of the row's runs: lo[x] = sb[x], hi[x] = sb[nhub + x] (the next routed row's lo)
  int32_t* sb = s_bounds[sub];
  for (int t = l; t < 2 * nhub; t += G) sb[t] = rvptr[idx * nhub + t];
  wave_lds_fence();
  const float* prow = partial + (uint64_t)idx * nhub * K + 4 * l;

  bool any_two = false, any_longer = false;
  for (int x0 = 0; x0 < nhub; x0 += kGroup) {
    float4 slot[kGroup];
    bool some[kGroup];
#pragma unroll
    for (int q = 0; q < kGroup; ++q) {
      const int32_t lo = sb[x0 + q], hi = sb[nhub + x0 + q];
      some[q] = lo != hi;
      const int64_t ga = lo >> shift;
      const int64_t gb = (hi - 1) >> shift;
      const bool two = some[q] && gb > ga;
      any_two |= two;
      any_longer |= some[q] && gb > ga + 1;
      const float* pa = two ? cbase + (uint64_t)(2 * ga + 1) * K : prow + (uint64_t)(x0 + q) * K;
      slot[q] = make_float4(0.f, 0.f, 0.f, 0.f);
      if (some[q]) slot[q] = *reinterpret_cast<const float4*>(pa);
    }
#pragma unroll
    for (int q = 0; q < kGroup; ++q)
      if (some[q]) add(slot[q]);
  }
  if (any_two) {
    for (int x0 = 0; x0 < nhub; x0 += kGroup) {
      float4 slot[kGroup];
      bool two[kGroup];
#pragma unroll
      for (int q = 0; q < kGroup; ++q) {
        const int32_t lo = sb[x0 + q], hi = sb[nhub + x0 + q];
        const int64_t ga = lo >> shift;
        two[q] = lo != hi && ((hi - 1) >> shift) > ga;
        slot[q] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (two[q]) slot[q] = *reinterpret_cast<const float4*>(cbase + (uint64_t)(2 * (ga + 1)) * K);
      }
#pragma unroll
      for (int q = 0; q < kGroup; ++q)
        if (two[q]) add(slot[q]);
    }
  }
  if (any_longer) {
    for (int x = 0; x < nhub; ++x) {
      const int32_t lo = sb[x], hi = sb[nhub + x];
      if (lo == hi) continue;
      const int64_t ga = lo >> shift;
      const int64_t gb = (hi - 1) >> shift;
      if (gb > ga + 1) add_heads(ga + 2, gb);
    }
  }
  if (in_tile) store_c_row<kLd, false>(C + (uint64_t)row * ld + 4 * l, acc, nv, c_aligned);
}

}  // namespace hpspmm
