// gfx950 device code for the rows strategy over *row tiles*: the layout a plan
// builds for a small or medium matrix so that one SpMM is a single launch whose
// every wavefront has the same, short chain of dependent memory round trips.
//
// A small SpMM (the 20k-vertex citation graph: 6 us over the CSR arrays) is
// bound by that chain, not by bandwidth: a sub-wave that walks a CSR row goes
// rowptr -> col/val -> B -> store, and a row longer than one staging step
// repeats col -> B once per step while the rest of its wavefront idles.  Here
// the plan cuts every row into slots of 8 nonzeros and packs 8 slots into a
// 64-entry tile, one tile per wavefront, one 8-byte record per entry:
//
//   tent[tile][64] = { column (-1 = padding), x }
//
// where x carries, in the first lanes of a slot, what the slot needs besides
// its columns: lane 0 the row (-1 = padding slot), lane 1 the index of the
// slot's first value, and in slot 0 lane 2 the tile's depth (entries per slot
// that any of its slots uses) and lane 3 log2 of the slots per row.  One load
// per lane, indexed by the wavefront's own number, brings all of it (first
// round trip); values and rows of B follow together (second).  Keeping it ONE
// load is the point: with columns and slot descriptors in two arrays the
// compiler issued the second load only after the first had arrived.
//
// A row of up to 8 / 16 / 32 / 64 nonzeros takes 1 / 2 / 4 / 8 adjacent slots
// of one tile (tiles hold rows of one size class only, so the reduction over
// a row's slots is the same wavefront shuffle for the whole tile; one-slot
// rows are sorted by length first, so a tile of 3-nonzero rows issues 3
// gathers per lane, not 8); a longer row owns consecutive tiles that one
// wavefront works through - or, in the second kernel below, a whole workgroup
// when the row has more than a few hundred nonzeros.  Long rows come first in
// the grid, since their chain is the longest.
//
// K > 32 is served in 32-column tiles of B and C by K/32 workgroups per group
// of row tiles (workgroup b serves column tile b % (K/32), so an XCD only ever
// touches one column tile of B).  A wavefront that serves two or four column
// tiles itself, with 16 or 32 loads in flight per lane, is slower (20k-vertex
// citation graph, K=128: 5.7 us with one, 6.4 with two, 8.2 with four).
//
// Row lengths other than 32 / 64 / 128 run the same kernels with the lengths
// as arguments (see TileColumns): ceil(K / 32) column tiles, the last one
// narrower, B as it lies or as a copy with padded rows.
//
// What this replaces in the reference: the row-per-warp kernels
// topoCacheSPMMKernel / topoCacheCoarsenSPMMKernel (spmm/mm/spmm_kernel.cu:247-370).
#pragma once

#include "spmm_kernels.hpp"

namespace hpspmm {

constexpr int kSlot = 8;          // nonzeros per slot = lanes per sub-wave at a 32-column tile
constexpr int kSlotsPerTile = 8;  // slots per tile = sub-waves per wavefront
constexpr int kRowTile = kSlot * kSlotsPerTile;

// ---- plan-time kernels: the row-tile layout is built on the device -----------------------------

constexpr int32_t kRowTileWorkgroupRows = 512;  // rows beyond this many nonzeros get a whole workgroup
constexpr int kRowTileGroups = 14;              // sort groups, in the order of the tiles (see rowtile_group)

// Size class of a row: 0..3 = 1 / 2 / 4 / 8 slots of one tile, 4 = tiles of its own.
__device__ __host__ __forceinline__ int rowtile_class(int32_t n) { return n <= 8 ? 0 : n <= 16 ? 1 : n <= 32 ? 2 : n <= 64 ? 3 : 4; }

// Position of a row's group in the tile order: rows that get a workgroup, the other rows with tiles
// of their own, then 8 / 4 / 2 slots a row, then the one-slot rows from 8 nonzeros down to none.
__device__ __forceinline__ int rowtile_group(int32_t n) {
  const int c = rowtile_class(n);
  return c == 4 ? (n > kRowTileWorkgroupRows ? 0 : 1) : c == 3 ? 2 : c == 2 ? 3 : c == 1 ? 4 : 5 + (kSlot - n);
}

// key[r] = group of row r, id[r] = r; count[g] += rows of group g; count[kRowTileGroups] += tiles
// of the rows with tiles of their own; count[kRowTileGroups + 1] != 0 if rowptr is not a row
// pointer array of a matrix with nnz nonzeros (unchecked input: the layout is then not built).
HPSPMM_KERNEL __launch_bounds__(kBlock) void rowtile_classify_kernel(int64_t rows, int64_t nnz,
                                                                  const int32_t* __restrict__ rowptr,
                                                                  uint32_t* __restrict__ key, int32_t* __restrict__ id,
                                                                  uint32_t* __restrict__ count) {
  __shared__ uint32_t s_count[kRowTileGroups + 2];
  if (threadIdx.x < kRowTileGroups + 2) s_count[threadIdx.x] = 0;
  __syncthreads();
  const int64_t r = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (r < rows) {
    const int32_t lb = rowptr[r];
    const int64_t n = (int64_t)rowptr[r + 1] - lb;
    if (n < 0 || lb < 0 || (int64_t)lb + n > nnz) {
      atomicAdd(&s_count[kRowTileGroups + 1], 1u);
      key[r] = 0;
    } else {
      const int g = rowtile_group((int32_t)n);
      key[r] = (uint32_t)g;
      atomicAdd(&s_count[g], 1u);
      if (g < 2) atomicAdd(&s_count[kRowTileGroups], (uint32_t)((n + kRowTile - 1) / kRowTile));
    }
    id[r] = (int32_t)r;
  }
  __syncthreads();
  if (threadIdx.x < kRowTileGroups + 2 && s_count[threadIdx.x]) atomicAdd(&count[threadIdx.x], s_count[threadIdx.x]);
}

// tiles[i] = tiles of the i-th row with tiles of its own (order[] = rows sorted by group), [n] = 0.
HPSPMM_KERNEL __launch_bounds__(kBlock) void rowtile_long_tiles_kernel(int64_t n, const int32_t* __restrict__ order,
                                                                    const int32_t* __restrict__ rowptr,
                                                                    uint32_t* __restrict__ tiles) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i > n) return;
  uint32_t t = 0;
  if (i < n) {
    const int32_t r = order[i];
    t = (uint32_t)((rowptr[r + 1] - rowptr[r] + kRowTile - 1) / kRowTile);
  }
  tiles[i] = t;
}

// ldesc[i] = {first tile, tiles} of the i-th such row, from the scan of tiles[].
HPSPMM_KERNEL __launch_bounds__(kBlock) void rowtile_ldesc_kernel(int64_t n, const uint32_t* __restrict__ first,
                                                               int2* __restrict__ ldesc) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i < n) ldesc[i] = make_int2((int)first[i], (int)(first[i + 1] - first[i]));
}

struct RowTileLayout {
  int64_t tiles, loop_tiles;
  int64_t first[4];  // first tile of size class 0..3
  int64_t start[5];  // first position in order[] of size class 0..4
  int64_t count[5];  // rows of size class 0..4
};

// Every record of the layout, one thread each: record e of slot q belongs to slot j of some row, or
// to no row (padding).  Lane 0 of a slot carries the row, lane 1 the index of the slot's first value,
// lanes 2 and 3 of a tile's first slot the tile's depth and log2 of the slots per row.
HPSPMM_KERNEL __launch_bounds__(kBlock) void rowtile_fill_kernel(RowTileLayout lay, const int32_t* __restrict__ order,
                                                              const int2* __restrict__ ldesc,
                                                              const int32_t* __restrict__ rowptr,
                                                              const int32_t* __restrict__ col, int2* __restrict__ tent) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= lay.tiles * kRowTile) return;
  const int e = (int)(i % kSlot);
  const int64_t q = i / kSlot;  // slot
  const int64_t t = q / kSlotsPerTile;
  int32_t row = -1;
  int64_t j = 0;  // the row's slot number
  int lg = 3, depth = kSlot;
  if (t < lay.loop_tiles) {
    // the row whose tiles include t: the last one that starts at or before t
    int64_t lo = 0, hi = lay.count[4];
    while (hi - lo > 1) {
      const int64_t mid = (lo + hi) >> 1;
      if ((int64_t)ldesc[mid].x <= t) lo = mid; else hi = mid;
    }
    row = order[lay.start[4] + lo];
    j = q - (int64_t)ldesc[lo].x * kSlotsPerTile;
  } else {
    const int c = t >= lay.first[0] ? 0 : t >= lay.first[1] ? 1 : t >= lay.first[2] ? 2 : 3;
    lg = c;
    const int64_t rel = q - lay.first[c] * kSlotsPerTile;
    const int64_t g = rel >> c;
    if (g < lay.count[c]) {
      row = order[lay.start[c] + g];
      j = rel & (((int64_t)1 << c) - 1);
    }
    if (c == 0) {  // one-slot rows are sorted by length, longest first: the tile's first row has its depth
      const int32_t r0 = order[lay.start[0] + (t - lay.first[0]) * kSlotsPerTile];
      depth = rowptr[r0 + 1] - rowptr[r0];
    }
  }
  int2 rec = make_int2(-1, e == 0 ? -1 : 0);
  if (row >= 0) {
    const int32_t lb = rowptr[row], n = rowptr[row + 1] - lb;
    const int64_t at = j * kSlot + e;
    rec.x = at < n ? col[lb + at] : -1;
    rec.y = e == 0 ? row : e == 1 ? (int32_t)(lb + j * kSlot) : 0;
  }
  if (q % kSlotsPerTile == 0) {
    if (e == 2) rec.y = depth;
    if (e == 3) rec.y = lg;
  }
  tent[i] = rec;
}

// Where a lane's four columns lie in a launch over 32-column tiles.  K > 0: rows of B and C of K
// floats, K a multiple of 32, everything a constant.  K == 0: the row lengths come with the launch
// (ldb floats between the rows of B, ldc between those of C = the columns there are), the last
// column tile may be narrower than 32, and the lanes beyond it gather what lane 0 gathers (no
// branch around the loads) and store nothing.
//   kLd = 1: ldb = ldc, a multiple of 4: every lane that stores owns four aligned floats.
//   kLd = 2: ldb >= ldc, ldb a multiple of 4 (B is a copy with padded rows); C's rows of any length.
//   kLd = 3: ldb = ldc, any number from 4 up; B is gathered with 16-byte loads at 4-byte alignment,
//            and the lane that owns the last nv < 4 columns of a row gathers the row's last four
//            floats instead (so that it reads nothing beyond the row) and finds its columns in
//            the last nv components of its sums.
struct TileColumns {
  uint32_t ldb;  // floats between the rows of B
  uint32_t ldc;  // ... of C
  int k0;        // first column of the tile
  int lb;        // this lane's offset into the tile when it gathers (kLd = 3: may be as low as -3)
  int nv;        // how many of this lane's four columns exist in C (0 ... 4)
  bool aligned;  // C's rows start at multiples of 16 bytes
  int sub;       // which of the entries that a slot works on at a time this lane is on (kSub < 8, see below)
};
// kSub = lanes per entry.  8: the slot's 8 lanes gather the 32 columns of one entry after the other.
// 4 and 1, for row lengths of at most 16 and 4 columns (one column tile): the slot works on 2 or 8
// of its entries at a time, lane l on entry l / kSub with columns 4 (l % kSub) ...; the partial sums
// of the lanes that share columns are added up before the row's slots are (reduce_slot).
template <int K, int kLd, int kSub>
__device__ __forceinline__ TileColumns tile_columns(uint32_t ldb, uint32_t ldc, int tile, int l) {
  TileColumns tc;
  tc.k0 = tile * 32;
  tc.sub = l / kSub;
  const int lc = l % kSub;  // this lane's group of four columns
  if constexpr (kLd == 0) {
    tc.ldb = tc.ldc = (uint32_t)K;
    tc.lb = 4 * lc;
    tc.nv = 4;
    tc.aligned = true;
  } else {
    tc.ldb = ldb;
    tc.ldc = ldc;
    tc.aligned = kLd == 1 || (kLd == 2 && ldc % 4 == 0);
    const int left = (int)ldc - (tc.k0 + 4 * lc);
    tc.nv = left < 0 ? 0 : left > 4 ? 4 : left;
    if constexpr (kLd == 3) tc.lb = left >= 4 ? 4 * lc : (int)ldb - 4 - tc.k0;  // (also a lane beyond the row: in bounds)
    else tc.lb = left > 0 ? 4 * lc : 0;
  }
  return tc;
}
// Adds up the partial sums of the lanes of a slot that share columns (kSub < 8), in a fixed order.
template <int kSub>
__device__ __forceinline__ void reduce_slot(float4& acc) {
#pragma unroll
  for (int off = kSub; off < kSlot; off <<= 1) {
    acc.x += __shfl_xor(acc.x, off);
    acc.y += __shfl_xor(acc.y, off);
    acc.z += __shfl_xor(acc.z, off);
    acc.w += __shfl_xor(acc.w, off);
  }
}
// Column tiles of a launch.
template <int K, int kLd>
__device__ __forceinline__ int column_tiles(uint32_t ldc) {
  return kLd ? (int)((ldc + 31u) / 32u) : K / 32;
}
// Which column tile and which group of row tiles workgroup b serves.  The tuned row lengths deal the
// column tiles round robin (b % T: with T = 1, 2, 4 column tiles an XCD only ever touches one of
// them).  same_xcd: the T tiles of a group go to workgroups b, b + 8, b + 16 ... - one XCD, one after
// the other - for rows of B that are not a whole number of 128-byte lines: the line that two
// neighbouring tiles share is then fetched into one L2 once instead of into two.
//
// chunks (tuned row lengths): the groups are dealt round robin all the same, but 2^chunk_log2
// consecutive groups at a time.  All XCDs still work on the same stretch of the layout (the tiles lie
// sorted by the length class of their rows: no XCD gets the heavier ones), and rows up to a chunk
// apart share an L2 - what a mesh, a banded matrix or blocks along the diagonal need for the rows of
// B that neighbouring rows have in common to be fetched into one L2 instead of eight.  The groups of
// the long rows, the first long_groups of the layout, stay dealt one at a time: they are the heaviest.
// A workgroup beyond the end gets group n_groups, which has no work.  The kernels that deal chunks
// are instantiations of their own (kChunks): the others take an empty argument in its place - a few
// more argument words alone cost a launch of microseconds 0.2 us.
struct TileChunks {
  int32_t long_groups, long_per, n_groups, chunk_log2;
};
struct NoTileChunks {};
template <bool kChunks>
using TileChunksArg = typename std::conditional<kChunks, TileChunks, NoTileChunks>::type;
template <int kLd>
__device__ __forceinline__ void tile_of_workgroup(uint32_t b, int T, bool same_xcd, const NoTileChunks&, int& tile,
                                                  int32_t& group);
template <int kLd>
__device__ __forceinline__ void tile_of_workgroup(uint32_t b, int T, bool, const TileChunks& tc, int& tile, int32_t& group) {
  static_assert(kLd == 0, "chunks are dealt at the tuned row lengths only");
  const uint32_t xcd = b % (uint32_t)kXcds, j = b / (uint32_t)kXcds;
  const uint32_t ways = (uint32_t)kXcds / (uint32_t)T, r = xcd / (uint32_t)T, L = (uint32_t)tc.chunk_log2;
  tile = (int)(xcd % (uint32_t)T);
  const uint32_t i = j - (uint32_t)tc.long_per;
  const uint32_t g = j < (uint32_t)tc.long_per ? j * ways + r
                                               : (uint32_t)tc.long_groups + (((i >> L) * ways + r) << L) + (i & ((1u << L) - 1u));
  const bool idle = j < (uint32_t)tc.long_per ? g >= (uint32_t)tc.long_groups : g >= (uint32_t)tc.n_groups;
  group = idle ? tc.n_groups : (int32_t)g;
}
template <int kLd>
__device__ __forceinline__ void tile_of_workgroup(uint32_t b, int T, bool same_xcd, const NoTileChunks&, int& tile,
                                                  int32_t& group) {
  if (kLd != 0 && same_xcd) {
    const uint32_t per = (uint32_t)kXcds * (uint32_t)T, r = b % per;
    tile = (int)(r / (uint32_t)kXcds);
    group = (int32_t)((b / per) * (uint32_t)kXcds + r % (uint32_t)kXcds);
  } else {
    tile = (int)(b % (uint32_t)T);
    group = (int32_t)(b / (uint32_t)T);
  }
}
// A lane's part of a row of C.
template <int kLd>
__device__ __forceinline__ void store_tile_row(float* __restrict__ C, int32_t row, int l, const TileColumns& tc,
                                               const float4& v) {
  float* p = C + (uint64_t)(uint32_t)row * tc.ldc + tc.k0 + 4 * l;
  if constexpr (kLd == 0) {
    store_result(p, v);
  } else if constexpr (kLd == 3) {
    // the lane of a row's last nv < 4 columns has gathered the row's last four floats
    const float4 r = tc.nv == 3 ? make_float4(v.y, v.z, v.w, 0.f) : tc.nv == 2 ? make_float4(v.z, v.w, 0.f, 0.f)
                   : tc.nv == 1 ? make_float4(v.w, 0.f, 0.f, 0.f) : v;
    if (tc.nv > 0) store_c_row<2, true>(p, r, tc.nv, false);
  } else if (tc.nv > 0) {
    store_c_row<kLd, true>(p, v, tc.nv, tc.aligned);
  }
}

// acc += the first N products of the slot whose columns are staged in s_col; `c` is this lane's
// own column, `v` its value (load already issued), `zrow` = 32 zeros in device memory, 4 more in front of them.  Nothing in
// here is conditional: a padding entry among the first N gathers the zero row instead of a row of
// B (so that a non-finite value in an unreferenced row of B cannot leak in).  With `if (c >= 0)`
// around the gathers the compiler copied a loaded register inside the batch and waited for it
// there - one more dependent round trip in a kernel that is nothing but round trips.
template <int N, bool kUnaligned, int kSub>
__device__ __forceinline__ void gather_n(float4& acc, int32_t c, float v, int tid, int base, const TileColumns& tc,
                                         const int32_t* s_col, float* s_val, const float* __restrict__ B,
                                         const float* __restrict__ zrow) {
  constexpr int R = kSlot / kSub;      // entries of the slot in work at a time
  constexpr int S = (N + R - 1) / R;   // steps (an entry beyond the first N is padding in every slot of the tile)
  int32_t cc[S];
  float4 b[S];
#pragma unroll
  for (int i = 0; i < S; ++i) cc[i] = s_col[base + i * R + tc.sub];
#pragma unroll
  for (int i = 0; i < S; ++i) {
    const float* src = cc[i] >= 0 ? B + (uint64_t)(uint32_t)cc[i] * (uint64_t)tc.ldb + (uint32_t)tc.k0 : zrow;
    if constexpr (kUnaligned) {
      const Float4Unaligned u = *reinterpret_cast<const Float4Unaligned*>(src + tc.lb);
      b[i] = make_float4(u.x, u.y, u.z, u.w);
    } else {
      b[i] = *reinterpret_cast<const float4*>(src + tc.lb);
    }
  }
  s_val[tid] = c >= 0 ? v : 0.f;
  wave_lds_fence();
#pragma unroll
  for (int i = 0; i < S; ++i) fma4(acc, s_val[base + i * R + tc.sub], b[i]);
  wave_lds_fence();
}

// What a wavefront knows about its tile once the records are staged.
struct TileInfo {
  int32_t row;  // of this lane's slot (-1: padding slot)
  int depth;    // wavefront-uniform
  int lg;       // wavefront-uniform
};

// Stages the tile's records (e = this lane's) in LDS, issues the load of this lane's value
// (unconditionally: a padding entry reads val[0] and discards it) and gathers `depth` entries per
// slot; depth < 0 = take the tile's own.
template <bool kUnaligned, int kSub>
__device__ __forceinline__ TileInfo gather_tile(float4& acc, int2 e, int depth, int tid, int base, int l,
                                                const TileColumns& tc, int32_t* s_col, int32_t* s_x, float* s_val,
                                                const float* __restrict__ val, const float* __restrict__ B,
                                                const float* __restrict__ zrow) {
  s_col[tid] = e.x;
  s_x[tid] = e.y;
  wave_lds_fence();
  const int wbase = tid & ~63;
  TileInfo info;
  info.row = s_x[base];
  info.depth = depth >= 0 ? depth : __builtin_amdgcn_readfirstlane(s_x[wbase + 2]);
  info.lg = __builtin_amdgcn_readfirstlane(s_x[wbase + 3]);
  const float v = val[e.x >= 0 ? s_x[base + 1] + l : 0];
  switch (info.depth) {
    case 0: wave_lds_fence(); break;
    case 1: gather_n<1, kUnaligned, kSub>(acc, e.x, v, tid, base, tc, s_col, s_val, B, zrow); break;
    case 2: gather_n<2, kUnaligned, kSub>(acc, e.x, v, tid, base, tc, s_col, s_val, B, zrow); break;
    case 3: gather_n<3, kUnaligned, kSub>(acc, e.x, v, tid, base, tc, s_col, s_val, B, zrow); break;
    case 4: gather_n<4, kUnaligned, kSub>(acc, e.x, v, tid, base, tc, s_col, s_val, B, zrow); break;
    case 5: gather_n<5, kUnaligned, kSub>(acc, e.x, v, tid, base, tc, s_col, s_val, B, zrow); break;
    case 6: gather_n<6, kUnaligned, kSub>(acc, e.x, v, tid, base, tc, s_col, s_val, B, zrow); break;
    case 7: gather_n<7, kUnaligned, kSub>(acc, e.x, v, tid, base, tc, s_col, s_val, B, zrow); break;
    default: gather_n<8, kUnaligned, kSub>(acc, e.x, v, tid, base, tc, s_col, s_val, B, zrow); break;
  }
  return info;
}

// acc += the products of tiles [t0, t1) (t0 < t1) of one long row, worked through by one
// wavefront; returns the row.
template <bool kUnaligned, int kSub>
__device__ __forceinline__ int32_t gather_tiles(float4& acc, int32_t t0, int32_t t1, int lane, int l, int tid,
                                                int base, const TileColumns& tc, int32_t* s_col, int32_t* s_x,
                                                float* s_val,
                                                const int2* __restrict__ tent, const float* __restrict__ val,
                                                const float* __restrict__ B, const float* __restrict__ zrow) {
  int2 e = tent[(int64_t)t0 * kRowTile + lane];
  int32_t row = -1;
  for (int32_t t = t0; t < t1; ++t) {
    const int2 e_now = e;
    if (t + 1 < t1) e = tent[(int64_t)(t + 1) * kRowTile + lane];  // on its way while this tile is gathered
    row = gather_tile<kUnaligned, kSub>(acc, e_now, kSlot, tid, base, l, tc, s_col, s_x, s_val, val, B, zrow).row;
  }
  return row;
}

// Sum over the 2^lg adjacent slots of a row (xor shuffles, in a fixed order), then the row's
// first slot stores.
template <int kLd, int kSub>
__device__ __forceinline__ void reduce_and_store(float4 acc, int lg, int32_t row, int s, int l, const TileColumns& tc,
                                                 float* __restrict__ C) {
  reduce_slot<kSub>(acc);
#pragma unroll
  for (int step = 0; step < 3; ++step) {
    if (lg > step) {
      acc.x += __shfl_xor(acc.x, kSlot << step);
      acc.y += __shfl_xor(acc.y, kSlot << step);
      acc.z += __shfl_xor(acc.z, kSlot << step);
      acc.w += __shfl_xor(acc.w, kSlot << step);
    }
  }
  if ((s & ((1 << lg) - 1)) == 0 && row >= 0 && l < kSub) store_tile_row<kLd>(C, row, l, tc, acc);
}

// Wavefront w < n_loop works through the tiles of long row w (ldesc[w] = first
// tile, tile count); wavefront w >= n_loop owns tile loop_tiles + (w - n_loop).
template <int K, int WPB, int kLd = 0, int kSub = kSlot, bool kChunks = false>
__global__ __launch_bounds__(WPB * 64) void spmm_rowtiles_kernel(int32_t n_waves, int32_t n_loop, int32_t loop_tiles,
                                                               const int2* __restrict__ ldesc,
                                                               const int2* __restrict__ tent,
                                                               const float* __restrict__ val,
                                                               const float* __restrict__ B, float* __restrict__ C,
                                                               const float* __restrict__ zrow, uint32_t ldb,
                                                               uint32_t ldc, bool same_xcd, TileChunksArg<kChunks> chunks) {
  const int T = column_tiles<K, kLd>(ldc);
  __shared__ int32_t s_col[WPB * 64];
  __shared__ int32_t s_x[WPB * 64];
  __shared__ float s_val[WPB * 64];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int l = lane & (kSlot - 1);
  const int s = lane / kSlot;
  const int base = tid - l;
  int ctile;
  int32_t group;
  tile_of_workgroup<kLd>(blockIdx.x, T, same_xcd, chunks, ctile, group);
  const TileColumns tc = tile_columns<K, kLd, kSub>(ldb, ldc, ctile, l);
  const int32_t w = __builtin_amdgcn_readfirstlane(group * WPB + (tid >> 6));
  if (w >= n_waves) return;

  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  if (w >= n_loop) {
    const int32_t tile = loop_tiles + (w - n_loop);
    const int2 e = tent[(int64_t)tile * kRowTile + lane];
    const TileInfo info = gather_tile<kLd == 3, kSub>(acc, e, -1, tid, base, l, tc, s_col, s_x, s_val, val, B, zrow);
    reduce_and_store<kLd, kSub>(acc, info.lg, info.row, s, l, tc, C);
  } else {
    const int2 ld = ldesc[w];
    const int32_t row = gather_tiles<kLd == 3, kSub>(acc, ld.x, ld.x + ld.y, lane, l, tid, base, tc, s_col, s_x, s_val, tent, val,
                                        B, zrow);
    reduce_and_store<kLd, kSub>(acc, 3, row, s, l, tc, C);
  }
}

// The same with a whole workgroup of WPB wavefronts on each of the n_wg longest rows (the first
// n_wg entries of ldesc; workgroups [0, n_wg) of a column tile; the row's tiles dealt in contiguous
// shares, the shares' sums added in wavefront order through LDS), for matrices whose longest rows
// would otherwise be the critical path of the launch.  The wavefronts of the other workgroups take
// one remaining long row or one ordinary tile each, as above.
template <int K, int WPB, int kLd = 0, int kSub = kSlot, bool kChunks = false>
__global__ __launch_bounds__(WPB * 64) void spmm_rowtiles_wg_kernel(int32_t n_tiles, int32_t n_wg, int32_t n_loop,
                                                                    int32_t loop_tiles,
                                                                    const int2* __restrict__ ldesc,
                                                                    const int2* __restrict__ tent,
                                                                    const float* __restrict__ val,
                                                                    const float* __restrict__ B,
                                                                    float* __restrict__ C,
                                                                    const float* __restrict__ zrow,
                                                                    uint32_t ldb, uint32_t ldc, bool same_xcd,
                                                                    TileChunksArg<kChunks> chunks) {
  const int T = column_tiles<K, kLd>(ldc);
  __shared__ int32_t s_col[WPB * 64];
  __shared__ int32_t s_x[WPB * 64];
  __shared__ float s_val[WPB * 64];
  __shared__ float4 s_part[WPB][kSlot];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int l = lane & (kSlot - 1);
  const int s = lane / kSlot;
  const int base = tid - l;
  int ctile;
  int32_t blk;
  tile_of_workgroup<kLd>(blockIdx.x, T, same_xcd, chunks, ctile, blk);
  const TileColumns tc = tile_columns<K, kLd, kSub>(ldb, ldc, ctile, l);
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);

  if (blk < n_wg) {  // uniform over the workgroup: every wavefront reaches the barrier
    const int2 ld = ldesc[blk];
    const int32_t per = (ld.y + WPB - 1) / WPB;
    const int32_t t0 = ld.x + wave * per;
    const int32_t t1 = t0 + per < ld.x + ld.y ? t0 + per : ld.x + ld.y;
    int32_t row = -1;  // wavefront 0 always has tiles, the later ones may not
    if (t0 < t1) row = gather_tiles<kLd == 3, kSub>(acc, t0, t1, lane, l, tid, base, tc, s_col, s_x, s_val, tent, val, B, zrow);
    reduce_slot<kSub>(acc);
#pragma unroll
    for (int off = kSlot; off < 64; off <<= 1) {
      acc.x += __shfl_xor(acc.x, off);
      acc.y += __shfl_xor(acc.y, off);
      acc.z += __shfl_xor(acc.z, off);
      acc.w += __shfl_xor(acc.w, off);
    }
    if (lane < kSlot) s_part[wave][lane] = acc;
    __syncthreads();
    if (tid < kSub) {
      float4 sum = s_part[0][tid];
      for (int j = 1; j < WPB; ++j) {
        const float4 p = s_part[j][tid];
        sum.x += p.x;
        sum.y += p.y;
        sum.z += p.z;
        sum.w += p.w;
      }
      store_tile_row<kLd>(C, row, l, tc, sum);
    }
    return;
  }

  const int32_t w = __builtin_amdgcn_readfirstlane(n_wg + (blk - n_wg) * WPB + wave);
  if (w < n_loop) {
    const int2 ld = ldesc[w];
    const int32_t row = gather_tiles<kLd == 3, kSub>(acc, ld.x, ld.x + ld.y, lane, l, tid, base, tc, s_col, s_x, s_val, tent, val,
                                        B, zrow);
    reduce_and_store<kLd, kSub>(acc, 3, row, s, l, tc, C);
  } else {
    const int32_t tile = loop_tiles + (w - n_loop);
    if (tile >= n_tiles) return;
    const int2 e = tent[(int64_t)tile * kRowTile + lane];
    const TileInfo info = gather_tile<kLd == 3, kSub>(acc, e, -1, tid, base, l, tc, s_col, s_x, s_val, val, B, zrow);
    reduce_and_store<kLd, kSub>(acc, info.lg, info.row, s, l, tc, C);
  }
}

}  // namespace hpspmm
