// gfx950 device code for FP32 CSR SpMM, C = A * B (B, C row-major, leading
// dimension K).  Wave64 only.
//
// Work decomposition (K in {32, 64, 128}):
//   A row of B or C is K floats = K/4 float4.  A *sub-wave* is G = K/4
//   adjacent lanes of one wavefront; lane l of a sub-wave owns columns
//   [4l, 4l+4) and every B row is fetched by one coalesced float4 load per
//   lane.  A wavefront holds P = 64/G independent sub-waves (8 / 4 / 2).
//
//   rows kernel      each sub-wave owns one whole CSR row.
//   segments kernel  each sub-wave owns a fixed-length run of consecutive
//                    nonzeros (a segment), wherever row boundaries fall, so
//                    the load is balanced for any degree distribution.  Rows
//                    that lie inside one segment are stored directly; the
//                    partial sums of rows that cross a segment boundary go to
//                    a carry buffer and are added, in segment order, by the
//                    fix-up kernel, which also zeroes empty rows.  No atomics.
//
// In both, the (col, val[, row]) entries of the next G nonzeros are fetched
// with one coalesced load per lane, staged in LDS and read back as broadcasts;
// up to kBatch B-row fragments are in flight per lane.
//
// What this replaces in the reference: the row-per-warp kernels
// topoCacheSPMMKernel / topoCacheCoarsenSPMMKernel
// (spmm/mm/spmm_kernel.cu:247-370) and the equal-nnz-per-warp COO kernels
// LBSPMMKernel* (spmm/mm/spmm_kernel.cu:428-731).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

// A kernel that is not a template: defined in every translation unit that includes its header
// (internal linkage), emitted only where it is launched.
#define HPSPMM_KERNEL [[maybe_unused]] static __global__

namespace hpspmm {

constexpr int kBlock = 256;         // threads per workgroup = 4 wavefronts
constexpr int kWavesPerBlock = 4;
constexpr int kBatch = 8;           // B-row fragments in flight per lane
constexpr int kXcds = 8;            // accelerator complex dies, each with its own L2
constexpr int kLongChain = 32;      // fix-up: a row over this many segments is added up by a whole wavefront

// LDS written by some lanes of a wavefront and read by others: LDS operations
// of one wavefront complete in issue order, so only the compiler has to be
// kept from reordering them.
__device__ __forceinline__ void wave_lds_fence() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

__device__ __forceinline__ void fma4(float4& acc, float a, const float4& b) {
  acc.x = __builtin_fmaf(a, b.x, acc.x);
  acc.y = __builtin_fmaf(a, b.y, acc.y);
  acc.z = __builtin_fmaf(a, b.z, acc.z);
  acc.w = __builtin_fmaf(a, b.w, acc.w);
}

// Store a result fragment from a gather kernel: nontemporal, so that it does not displace rows of
// B from the L2 (four scalar stores - the compiler mis-lowered the vector form of the nontemporal
// builtins in an earlier experiment).  Measured: 20k-vertex citation graph K=128 11.5 -> 10.3 us,
// social graph K=128 3.85 -> 3.77 ms.  Not used by the kernels that only stream (final pass,
// value re-ordering): there it cost time (R-MAT 6.02 -> 6.26 ms).
__device__ __forceinline__ void store_result(float* __restrict__ dst, const float4& v) {
  __builtin_nontemporal_store(v.x, dst);
  __builtin_nontemporal_store(v.y, dst + 1);
  __builtin_nontemporal_store(v.z, dst + 2);
  __builtin_nontemporal_store(v.w, dst + 3);
}

template <int K>
__device__ __forceinline__ float4 load_b(const float* __restrict__ B, int32_t c, int l) {
  // 64-bit address: cols * K * 4 reaches 2^31 bytes at the largest benchmark size
  return *reinterpret_cast<const float4*>(B + (uint64_t)(uint32_t)c * (uint64_t)K + (uint32_t)(4 * l));
}

// The same with the row length of B given at run time: the operands of a tuned kernel may be K
// columns of a wider B and C (one column tile of a product whose row length is not K).  kLd = 0
// compiles to the fixed form; 1 = row lengths at run time, multiples of 4; 2 = the rows of C may be
// up to three floats shorter than those of B and start at any multiple of 4 bytes (B is then a
// padded copy of the caller's), and a lane may own fewer than four columns of C.
// ld_arg carries three things: in bits 0-21 the row length of B (a multiple of 4); in bits 22-23 by
// how much the rows of C are shorter (0 ... 3: the caller's row length need not be a multiple of 4
// - B is then a copy padded to one, C is the caller's own); in bits 24-31 how many of the tile's K
// columns exist (0 = all of them): the last tile of a row length that is not a multiple of K is
// narrower, and the lanes whose columns lie beyond it must not write C.
template <int K, int kLd>
__device__ __forceinline__ uint32_t row_length(uint32_t ld_arg) {
  return kLd ? (ld_arg & 0x3FFFFFu) : (uint32_t)K;
}
template <int K, int kLd>
__device__ __forceinline__ uint32_t c_row_length(uint32_t ld_arg) {
  return kLd == 2 ? (ld_arg & 0x3FFFFFu) - ((ld_arg >> 22) & 3u) : row_length<K, kLd>(ld_arg);
}
// C's rows start at multiples of 16 bytes (when C itself does).
template <int kLd>
__device__ __forceinline__ bool c_rows_aligned(uint32_t ld_arg) {
  return kLd < 2 || ((ld_arg >> 22) & 3u) == 0;
}
// How many of lane l's four columns exist in the tile (0 ... 4).
template <int K, int kLd>
__device__ __forceinline__ int lane_columns(uint32_t ld_arg, int l) {
  if constexpr (kLd == 0) return 4;
  const int cols = (int)(ld_arg >> 24);
  if (cols == 0) return 4;
  const int left = cols - 4 * l;
  return left < 0 ? 0 : left > 4 ? 4 : left;
}
// A lane's nv (1 ... 4) columns into a row of C: in the form the fixed kernels use when the rows are
// aligned and the lane owns all four, else float by float.
template <int kLd, bool kStream>
__device__ __forceinline__ void store_c_row(float* __restrict__ p, const float4& v, int nv, bool aligned) {
  if (kLd < 2 || (aligned && nv == 4)) {  // (kLd < 2: nv is 4 wherever this is called)
    if constexpr (kStream) store_result(p, v);
    else *reinterpret_cast<float4*>(p) = v;
  } else {
    p[0] = v.x;
    if (nv > 1) p[1] = v.y;
    if (nv > 2) p[2] = v.z;
    if (nv > 3) p[3] = v.w;
  }
}
// Four floats at a 4-byte aligned address.
struct __attribute__((packed, aligned(4))) Float4Unaligned {
  float x, y, z, w;
};

__device__ __forceinline__ float4 load_b_ld(const float* __restrict__ B, int32_t c, int l, uint32_t ld) {
  return *reinterpret_cast<const float4*>(B + (uint64_t)(uint32_t)c * (uint64_t)ld + (uint32_t)(4 * l));
}

// Fragment l of a KT-wide column tile starting at column k0 of row c (leading dimension K).
template <int K>
__device__ __forceinline__ float4 load_b_tile(const float* __restrict__ B, int32_t c, int k0, int l) {
  return *reinterpret_cast<const float4*>(B + (uint64_t)(uint32_t)c * (uint64_t)K + (uint32_t)(k0 + 4 * l));
}

// Hub cache: the plan may keep the most referenced rows of B in a compact
// buffer (refreshed at the start of every SpMM) and rewrite their column
// indices as ~slot (negative).  A negative index reads the compact buffer.
template <int K, bool kHub>
__device__ __forceinline__ float4 load_b_hub(const float* __restrict__ B, const float* __restrict__ Bhot, int32_t c,
                                             int l) {
  if constexpr (kHub) {
    const bool hot = c < 0;
    const float* base = hot ? Bhot : B;
    const uint32_t idx = hot ? (uint32_t)~c : (uint32_t)c;
    return *reinterpret_cast<const float4*>(base + (uint64_t)idx * (uint64_t)K + (uint32_t)(4 * l));
  } else {
    return load_b<K>(B, c, l);
  }
}

// The same with rows of B that are ld floats apart (the compact buffer's rows stay K apart).
template <int K, bool kHub>
__device__ __forceinline__ float4 load_b_hub_ld(const float* __restrict__ B, const float* __restrict__ Bhot, int32_t c,
                                                int l, uint32_t ld) {
  if constexpr (kHub) {
    const bool hot = c < 0;
    const float* base = hot ? Bhot : B;
    const uint32_t idx = hot ? (uint32_t)~c : (uint32_t)c;
    return *reinterpret_cast<const float4*>(base + (uint64_t)idx * (uint64_t)(hot ? (uint32_t)K : ld) + (uint32_t)(4 * l));
  } else {
    return load_b_ld(B, c, l, ld);
  }
}

// Workgroups are dealt to the XCDs round-robin (workgroup b runs on XCD
// b % 8).  Remapping so that XCD x receives the x-th contiguous eighth of the
// logical workgroups keeps neighbouring rows (similar column sets) behind one
// L2.  Returns -1 for the padding workgroups of the rounded-up grid.
__device__ __forceinline__ int64_t xcd_remap(int64_t b, int64_t nblocks, bool remap) {
  if (!remap) return b < nblocks ? b : -1;
  const int64_t per = (nblocks + kXcds - 1) / kXcds;
  const int64_t lb = (b % kXcds) * per + b / kXcds;
  return lb < nblocks ? lb : -1;
}

// ---------------------------------------------------------------------------
// rows kernel: one sub-wave per CSR row; rows longer than `long_threshold` are
// left to the wave-per-row part of the same launch.
// ---------------------------------------------------------------------------

// acc += sum over nonzeros [lb, hb) of val[j] * B[col[j], 4l .. 4l+4), executed by
// one sub-wave.  `base` is the LDS slot of the sub-wave's lane 0.
template <int K, int KT>
__device__ __forceinline__ void accumulate_range(float4& acc, int32_t lb, int32_t hb, int l, int tid, int base,
                                                 int32_t* s_col, float* s_val, const int32_t* __restrict__ col,
                                                 const float* __restrict__ val, const float* __restrict__ B,
                                                 int k0) {
  constexpr int G = KT / 4;
  constexpr int U = G < kBatch ? G : kBatch;
  for (int32_t jj = lb; jj < hb; jj += G) {
    const int32_t p = jj + l;
    if (p < hb) {
      s_col[tid] = col[p];
      s_val[tid] = val[p];
    }
    wave_lds_fence();
    const int cnt = (hb - jj) < G ? (hb - jj) : G;
    int u = 0;
    for (; u + U <= cnt; u += U) {
      int32_t c[U];
      float v[U];
      float4 b[U];
#pragma unroll
      for (int i = 0; i < U; ++i) {
        c[i] = s_col[base + u + i];
        v[i] = s_val[base + u + i];
      }
#pragma unroll
      for (int i = 0; i < U; ++i) b[i] = load_b_tile<K>(B, c[i], k0, l);
#pragma unroll
      for (int i = 0; i < U; ++i) fma4(acc, v[i], b[i]);
    }
    if constexpr (G == 8) {
      // Fewer than 8 entries left, narrow sub-waves: branch-free batches of 4.
      // Slots past the end re-read the last valid entry (a legal address) and
      // their FMA result is discarded by a select, so the loads of a short row
      // are in flight together and a non-finite B value cannot leak in through
      // 0 * inf.  (Measured on the 20k-vertex citation graph: 6.0 us against
      // 6.5 us for a one-at-a-time loop.  For G >= 16 the extra load
      // instructions cost more than the overlap gains: 7.7 vs 6.7 us at K=64.)
      constexpr int R = 4;
      for (; u < cnt; u += R) {
        float v[R];
        float4 b[R];
        bool ok[R];
#pragma unroll
        for (int i = 0; i < R; ++i) {
          ok[i] = u + i < cnt;
          const int slot = base + (ok[i] ? u + i : cnt - 1);
          v[i] = s_val[slot];
          b[i] = load_b_tile<K>(B, s_col[slot], k0, l);
        }
#pragma unroll
        for (int i = 0; i < R; ++i) {
          float4 t = acc;
          fma4(t, v[i], b[i]);
          acc.x = ok[i] ? t.x : acc.x;
          acc.y = ok[i] ? t.y : acc.y;
          acc.z = ok[i] ? t.z : acc.z;
          acc.w = ok[i] ? t.w : acc.w;
        }
      }
    } else {
      for (; u < cnt; ++u) {
        const float4 b = load_b_tile<K>(B, s_col[base + u], k0, l);
        fma4(acc, s_val[base + u], b);
      }
    }
    wave_lds_fence();
  }
}

// Workgroups come in groups of T = K / KT, one per KT-wide column tile of B
// and C (workgroup b serves tile b % T; T divides 8, so an XCD always sees the
// same tile and its L2 only has to hold cols * KT floats of B).  Within a tile:
// workgroup groups [0, short_blocks) run one sub-wave per row and skip rows
// longer than long_threshold; the remaining groups run one wavefront per entry
// of long_rows[], the row's nonzeros dealt in contiguous runs to the sub-waves
// and the partial sums combined with wavefront shuffles.
template <int K, int KT>
__global__ __launch_bounds__(kBlock) void spmm_rows_kernel(int64_t rows, const int32_t* __restrict__ rowptr,
                                                           const int32_t* __restrict__ col,
                                                           const float* __restrict__ val,
                                                           const float* __restrict__ B, float* __restrict__ C,
                                                           int64_t short_blocks, int32_t long_threshold,
                                                           const int32_t* __restrict__ long_rows,
                                                           int64_t n_long) {
  constexpr int T = K / KT;
  constexpr int G = KT / 4;
  constexpr int P = 64 / G;
  __shared__ int32_t s_col[kBlock];
  __shared__ float s_val[kBlock];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int l = lane % G;
  const int base = tid - l;
  const int k0 = (int)(blockIdx.x % T) * KT;
  const int64_t blk = blockIdx.x / T;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);

  if (blk < short_blocks) {
    const int64_t row = (blk * kWavesPerBlock + (tid >> 6)) * P + lane / G;
    if (row >= rows) return;
    const int32_t lb = rowptr[row];
    const int32_t hb = rowptr[row + 1];
    if (hb - lb > long_threshold) return;
    accumulate_range<K, KT>(acc, lb, hb, l, tid, base, s_col, s_val, col, val, B, k0);
    store_result(C + (uint64_t)row * K + k0 + 4 * l, acc);
  } else {
    const int64_t w = (blk - short_blocks) * kWavesPerBlock + (tid >> 6);
    if (w >= n_long) return;
    const int32_t row = long_rows[w];
    const int32_t lb = rowptr[row];
    const int32_t hb = rowptr[row + 1];
    // contiguous runs, each a multiple of G long so that the staging loads stay aligned to the run
    const int32_t per = ((hb - lb + P * G - 1) / (P * G)) * G;
    const int32_t my_lb = lb + (lane / G) * per;
    const int32_t my_hb = (my_lb + per) < hb ? (my_lb + per) : hb;
    accumulate_range<K, KT>(acc, my_lb, my_hb, l, tid, base, s_col, s_val, col, val, B, k0);
#pragma unroll
    for (int off = G; off < 64; off <<= 1) {
      acc.x += __shfl_xor(acc.x, off);
      acc.y += __shfl_xor(acc.y, off);
      acc.z += __shfl_xor(acc.z, off);
      acc.w += __shfl_xor(acc.w, off);
    }
    if (lane < G) store_result(C + (uint64_t)(uint32_t)row * K + k0 + 4 * l, acc);
  }
}

// ---------------------------------------------------------------------------
// Tile engine of the segment-type kernels.
//
// A sub-wave consumes its segment in tiles of kTile = 32 entries.  Lane l holds
// TL = 32 / G consecutive entries of the *next* tile in registers (one 16/8/4
// byte load per array), so that the metadata fetch of tile t+1 overlaps the B
// gathers of tile t (the role cp.async double buffering plays in the
// reference, spmm/mm/spmm_kernel.cu:650-702).  At the top of an iteration the
// registers are written to the sub-wave's LDS region and read back as
// broadcasts, 8 entries (8 B-row fragments in flight per lane) at a time.
// LDS regions are 36 entries apart: 16-byte aligned for the vector stores and
// on distinct banks for the broadcast reads of the P sub-waves.
// ---------------------------------------------------------------------------
constexpr int kTile = 32;
constexpr int kTileStride = 36;

template <int TL>
struct TileRegs {
  int32_t c[TL];
  float v[TL];
  int32_t r[TL];
};

// dst[0..TL) = src[q .. q+TL): one vector load when allowed and the tile is full, else guarded scalars.
template <int TL, typename T>
__device__ __forceinline__ void load_run(T (&dst)[TL], const T* __restrict__ src, int64_t q, int64_t e, bool vec_ok) {
  if (TL > 1 && vec_ok && q + TL <= e) {
    if constexpr (TL == 4) {
      const int4 w = *reinterpret_cast<const int4*>(src + q);
      dst[0] = __builtin_bit_cast(T, w.x);
      dst[1] = __builtin_bit_cast(T, w.y);
      dst[2] = __builtin_bit_cast(T, w.z);
      dst[3] = __builtin_bit_cast(T, w.w);
    } else if constexpr (TL == 2) {
      const int2 w = *reinterpret_cast<const int2*>(src + q);
      dst[0] = __builtin_bit_cast(T, w.x);
      dst[1] = __builtin_bit_cast(T, w.y);
    }
  } else {
#pragma unroll
    for (int i = 0; i < TL; ++i) dst[i] = q + i < e ? src[q + i] : T(0);
  }
}

template <int TL>
__device__ __forceinline__ void stage_tile(const TileRegs<TL>& m, int slot, int32_t* s_col, float* s_val,
                                           int32_t* s_row) {
  if constexpr (TL == 4) {
    *reinterpret_cast<int4*>(s_col + slot) = make_int4(m.c[0], m.c[1], m.c[2], m.c[3]);
    *reinterpret_cast<float4*>(s_val + slot) = make_float4(m.v[0], m.v[1], m.v[2], m.v[3]);
    *reinterpret_cast<int4*>(s_row + slot) = make_int4(m.r[0], m.r[1], m.r[2], m.r[3]);
  } else if constexpr (TL == 2) {
    *reinterpret_cast<int2*>(s_col + slot) = make_int2(m.c[0], m.c[1]);
    *reinterpret_cast<float2*>(s_val + slot) = make_float2(m.v[0], m.v[1]);
    *reinterpret_cast<int2*>(s_row + slot) = make_int2(m.r[0], m.r[1]);
  } else {
    s_col[slot] = m.c[0];
    s_val[slot] = m.v[0];
    s_row[slot] = m.r[0];
  }
}

// Accumulate the first `cnt` staged entries of a sub-wave's tile; a change of
// row calls flush() (which stores the finished row and is told nothing else).
template <class LoadB, class Flush>
__device__ __forceinline__ void consume_tile(int cnt, int sbase, const int32_t* s_col, const float* s_val,
                                             const int32_t* s_row, int32_t& cur, float4& acc, LoadB loadb,
                                             Flush flush) {
  constexpr int U = kBatch;
  int u = 0;
  for (; u + U <= cnt; u += U) {
    int32_t c[U], r[U];
    float v[U];
    float4 b[U];
#pragma unroll
    for (int i = 0; i < U; ++i) {
      c[i] = s_col[sbase + u + i];
      v[i] = s_val[sbase + u + i];
      r[i] = s_row[sbase + u + i];
    }
#pragma unroll
    for (int i = 0; i < U; ++i) b[i] = loadb(c[i]);
#pragma unroll
    for (int i = 0; i < U; ++i) {
      if (r[i] != cur) {
        flush();
        acc = make_float4(0.f, 0.f, 0.f, 0.f);
        cur = r[i];
      }
      fma4(acc, v[i], b[i]);
    }
  }
  for (; u < cnt; ++u) {
    const int32_t r = s_row[sbase + u];
    const float4 b = loadb(s_col[sbase + u]);
    if (r != cur) {
      flush();
      acc = make_float4(0.f, 0.f, 0.f, 0.f);
      cur = r;
    }
    fma4(acc, s_val[sbase + u], b);
  }
}

// ---------------------------------------------------------------------------
// segments kernel.
//
// Segment g covers nonzeros [g << shift, min((g+1) << shift, nnz)).  nnz_row[j]
// is the row of nonzero j.  Partial sums:
//   * the first row of a segment, if it began in an earlier segment, goes to
//     carry slot 2g   ("head");
//   * the last row of a segment, if it continues into the next one and is not
//     that head row, goes to carry slot 2g+1 ("tail");
//   * every other row is complete and is stored to C.
// A row spanning segments ga < gb is therefore tail[ga] + head[ga+1..gb].
// kAtomic = true is the COO "accumulate" form: no carry buffer, every flush is
// an FP32 atomic add into C, rows may come in any order.
// ---------------------------------------------------------------------------
template <int K, bool kAtomic, bool kHub>
__global__ __launch_bounds__(kBlock) void spmm_segments_kernel(
    const int32_t* __restrict__ rowptr, const int32_t* __restrict__ col, const float* __restrict__ val,
    const int32_t* __restrict__ nnz_row, const float* __restrict__ B, const float* __restrict__ Bhot,
    float* __restrict__ C, float* __restrict__ carry, int64_t nnz, int shift, int64_t nseg, int64_t nblocks,
    bool remap, bool vec_ok) {
  constexpr int G = K / 4;
  constexpr int P = 64 / G;
  constexpr int TL = kTile / G;
  __shared__ __attribute__((aligned(16))) int32_t s_col[kWavesPerBlock * P * kTileStride];
  __shared__ __attribute__((aligned(16))) float s_val[kWavesPerBlock * P * kTileStride];
  __shared__ __attribute__((aligned(16))) int32_t s_row[kWavesPerBlock * P * kTileStride];

  const int64_t blk = xcd_remap(blockIdx.x, nblocks, remap);
  if (blk < 0) return;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int l = lane % G;
  const int64_t g = (blk * kWavesPerBlock + (tid >> 6)) * P + lane / G;
  if (g >= nseg) return;

  const int64_t s = g << shift;
  const int64_t e = (s + ((int64_t)1 << shift)) < nnz ? (s + ((int64_t)1 << shift)) : nnz;
  const int sbase = ((tid >> 6) * P + lane / G) * kTileStride;

  int32_t cur = nnz_row[s];
  bool head_pending = false;
  if constexpr (!kAtomic) head_pending = (int64_t)rowptr[cur] < s;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);

  auto flush_to = [&](bool is_tail) {
    if constexpr (kAtomic) {
      float* dst = C + (uint64_t)(uint32_t)cur * K + 4 * l;
      unsafeAtomicAdd(dst + 0, acc.x);
      unsafeAtomicAdd(dst + 1, acc.y);
      unsafeAtomicAdd(dst + 2, acc.z);
      unsafeAtomicAdd(dst + 3, acc.w);
    } else {
      float* dst = head_pending ? carry + (uint64_t)(2 * g) * K
                                : (is_tail ? carry + (uint64_t)(2 * g + 1) * K
                                           : C + (uint64_t)(uint32_t)cur * K);
      head_pending = false;
      store_result(dst + 4 * l, acc);
    }
  };
  auto flush = [&]() { flush_to(false); };
  auto loadb = [&](int32_t c) { return load_b_hub<K, kHub>(B, Bhot, c, l); };
  auto fetch = [&](TileRegs<TL>& m, int64_t t) {
    const int64_t q = t + l * TL;
    load_run<TL>(m.c, col, q, e, vec_ok);
    load_run<TL>(m.v, val, q, e, vec_ok);
    load_run<TL>(m.r, nnz_row, q, e, vec_ok);
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
  bool continues = false;
  if constexpr (!kAtomic) continues = (int64_t)rowptr[cur + 1] > e;
  flush_to(continues);
}

// Fix-up after the segments kernel.  A wavefront scans `rpw` consecutive rows
// (one rowptr pair per lane, coalesced) and classifies them by ballot; its
// sub-waves then zero the empty rows and, for rows that cross a segment
// boundary, add the carry slots in segment order.  All other rows were already
// stored.  rpw = 64 when rows are plentiful; rpw = 64 / (K/4), one row per
// sub-wave, when they are few and long - 4,659 rows of 310 nonzeros on average
// left 73 wavefronts adding up eight chains each, one after the other (56 us,
// five times the segments kernel before it).
// `start` (may be NULL): first position of every row when the nonzeros were
// processed in an order of the plan's own; NULL = stored order (rowptr).
template <int K, int kLd = 0>
__global__ __launch_bounds__(kBlock) void spmm_fixup_kernel(int64_t rows, const int32_t* __restrict__ rowptr,
                                                            const int32_t* __restrict__ start,
                                                            const float* __restrict__ carry,
                                                            float* __restrict__ C, int shift, int rpw,
                                                            uint32_t ld_arg) {
  constexpr int G = K / 4;
  constexpr int P = 64 / G;
  const uint32_t ld = c_row_length<K, kLd>(ld_arg);  // floats between the rows of C
  const bool c_aligned = c_rows_aligned<kLd>(ld_arg);
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int l = lane % G;
  const int nv = lane_columns<K, kLd>(ld_arg, l);
  const bool in_tile = nv > 0;
  const int sub = lane / G;
  const int64_t r0 = ((int64_t)blockIdx.x * kWavesPerBlock + (tid >> 6)) * rpw;
  if (r0 >= rows) return;
  const int64_t r = r0 + lane;
  const bool valid = r < rows && lane < rpw;
  int32_t lb = valid ? rowptr[r] : 0;
  int32_t hb = valid ? rowptr[r + 1] : 0;
  if (start != nullptr && valid) {
    hb = start[r] + (hb - lb);
    lb = start[r];
  }
  const bool empty = valid && lb == hb;
  const bool split = valid && lb != hb && ((int64_t)lb >> shift) != ((int64_t)(hb - 1) >> shift);
  // a row over many segments is put together by the whole wavefront, see below
  const bool chain = split && (((int64_t)(hb - 1) >> shift) - ((int64_t)lb >> shift)) >= kLongChain;
  const uint64_t m_empty = __ballot(empty);
  const uint64_t m_split = __ballot(split && !chain);
  uint64_t m_chain = __ballot(chain);
  if ((m_empty | m_split | m_chain) == 0) return;

  auto add = [](float4& a, const float4& b) {
    a.x += b.x;
    a.y += b.y;
    a.z += b.z;
    a.w += b.w;
  };
  // acc += head[g0] + head[g0 + step] + ... (g <= gb), 8 slots in flight at a time, in that order
  auto add_heads = [&](float4& acc, int64_t g0, int64_t gb, int64_t step) {
    int64_t g = g0;
    for (; g + (kBatch - 1) * step <= gb; g += kBatch * step) {
      float4 part[kBatch];
#pragma unroll
      for (int q = 0; q < kBatch; ++q)
        part[q] = *reinterpret_cast<const float4*>(carry + (uint64_t)(2 * (g + q * step)) * K + 4 * l);
#pragma unroll
      for (int q = 0; q < kBatch; ++q) add(acc, part[q]);
    }
    for (; g <= gb; g += step) add(acc, *reinterpret_cast<const float4*>(carry + (uint64_t)(2 * g) * K + 4 * l));
  };

  for (int i = sub; i < rpw; i += P) {
    // every lane takes part in the shuffles; only then do the sub-waves diverge
    const int32_t lb_i = __shfl(lb, i);
    const int32_t hb_i = __shfl(hb, i);
    float* out = C + (uint64_t)(r0 + i) * ld + 4 * l;
    if ((m_empty >> i) & 1ull) {
      if (in_tile) store_c_row<kLd, false>(out, make_float4(0.f, 0.f, 0.f, 0.f), nv, c_aligned);
    } else if ((m_split >> i) & 1ull) {
      const int64_t ga = (int64_t)lb_i >> shift;
      const int64_t gb = (int64_t)(hb_i - 1) >> shift;
      float4 acc = *reinterpret_cast<const float4*>(carry + (uint64_t)(2 * ga + 1) * K + 4 * l);
      add_heads(acc, ga + 1, gb, 1);
      if (in_tile) store_c_row<kLd, false>(out, acc, nv, c_aligned);
    }
  }
  // Long chains, one row at a time, all P sub-waves together: sub-wave s adds the heads ga+1+s,
  // ga+1+s+P, ...; sub-wave 0 then adds tail[ga] and the P partial sums in the order of s.  (A
  // single dense row of 100k nonzeros cut into 1500 segments: 80 us for one sub-wave alone.)
  while (m_chain) {
    const int i = __ffsll((long long)m_chain) - 1;
    m_chain &= m_chain - 1;
    const int32_t lb_i = __shfl(lb, i);
    const int32_t hb_i = __shfl(hb, i);
    const int64_t ga = (int64_t)lb_i >> shift;
    const int64_t gb = (int64_t)(hb_i - 1) >> shift;
    float4 part = make_float4(0.f, 0.f, 0.f, 0.f);
    add_heads(part, ga + 1 + sub, gb, P);
    float4 acc = *reinterpret_cast<const float4*>(carry + (uint64_t)(2 * ga + 1) * K + 4 * l);
#pragma unroll
    for (int s = 0; s < P; ++s) {
      float4 t;
      t.x = __shfl(part.x, s * G + l);
      t.y = __shfl(part.y, s * G + l);
      t.z = __shfl(part.z, s * G + l);
      t.w = __shfl(part.w, s * G + l);
      add(acc, t);
    }
    if (sub == 0 && in_tile) store_c_row<kLd, false>(C + (uint64_t)(r0 + i) * ld + 4 * l, acc, nv, c_aligned);
  }
}

// ---------------------------------------------------------------------------
// Plan-time kernels.
// ---------------------------------------------------------------------------

// status[0] |= 1 rowptr[0] != 0, |= 2 rowptr decreases, |= 4 rowptr[rows] != nnz,
//           |= 8 column index out of [0, cols).
HPSPMM_KERNEL __launch_bounds__(kBlock) void validate_csr_kernel(int64_t rows, int64_t cols, int64_t nnz,
                                                              const int32_t* __restrict__ rowptr,
                                                              const int32_t* __restrict__ col,
                                                              int32_t* __restrict__ status) {
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  const int64_t i0 = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  int32_t bad = 0;
  if (i0 == 0) {
    if (rowptr[0] != 0) bad |= 1;
    if ((int64_t)rowptr[rows] != nnz) bad |= 4;
  }
  for (int64_t i = i0; i < rows; i += stride)
    if (rowptr[i + 1] < rowptr[i]) bad |= 2;
  for (int64_t j = i0; j < nnz; j += stride) {
    const int32_t c = col[j];
    if (c < 0 || (int64_t)c >= cols) bad |= 8;
  }
  if (bad) atomicOr(status, bad);
}

// stats[0] = max row length, stats[1] = number of empty rows.
HPSPMM_KERNEL __launch_bounds__(kBlock) void row_stats_kernel(int64_t rows, const int32_t* __restrict__ rowptr,
                                                           int32_t* __restrict__ stats) {
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  int32_t mx = 0, empty = 0;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < rows; i += stride) {
    const int32_t d = rowptr[i + 1] - rowptr[i];
    mx = d > mx ? d : mx;
    empty += (d == 0);
  }
  for (int off = 32; off > 0; off >>= 1) {
    const int32_t o = __shfl_down(mx, off);
    mx = o > mx ? o : mx;
    empty += __shfl_down(empty, off);
  }
  if ((threadIdx.x & 63) == 0) {
    atomicMax(&stats[0], mx);
    if (empty) atomicAdd(&stats[1], empty);
  }
}

// Appends every row longer than `threshold` to list[] (order unspecified);
// *count must be zero on entry.
HPSPMM_KERNEL __launch_bounds__(kBlock) void collect_long_rows_kernel(int64_t rows, const int32_t* __restrict__ rowptr,
                                                                   int32_t threshold, int32_t* __restrict__ list,
                                                                   int32_t* __restrict__ count) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  const bool is_long = i < rows && (rowptr[i + 1] - rowptr[i]) > threshold;
  const uint64_t mask = __ballot(is_long);
  if (mask == 0) return;
  const int lane = threadIdx.x & 63;
  int32_t base = 0;
  if (lane == 0) base = atomicAdd(count, (int32_t)__popcll(mask));
  base = __shfl(base, 0);
  if (is_long) list[base + __popcll(mask & ((1ull << lane) - 1ull))] = (int32_t)i;
}

// out[j] = ~slot if column col[j] is cached in slot colmap[col[j]] >= 0, else col[j].
HPSPMM_KERNEL __launch_bounds__(kBlock) void remap_columns_kernel(int64_t nnz, const int32_t* __restrict__ col,
                                                               const int32_t* __restrict__ colmap,
                                                               int32_t* __restrict__ out) {
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  for (int64_t j = (int64_t)blockIdx.x * kBlock + threadIdx.x; j < nnz; j += stride) {
    const int32_t c = col[j];
    const int32_t slot = colmap[c];
    out[j] = slot >= 0 ? ~slot : c;
  }
}

// Bhot[s, :] = B[hub_ids[s], :] for s in [0, n_hub): one sub-wave per row.
template <int K>
__global__ __launch_bounds__(kBlock) void gather_hub_rows_kernel(int64_t n_hub, const int32_t* __restrict__ hub_ids,
                                                                 const float* __restrict__ B,
                                                                 float* __restrict__ Bhot) {
  constexpr int G = K / 4;
  const int64_t t = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  const int64_t s = t / G;
  const int l = (int)(t % G);
  if (s >= n_hub) return;
  *reinterpret_cast<float4*>(Bhot + (uint64_t)s * K + 4 * l) = load_b<K>(B, hub_ids[s], l);
}

// Largest r in [lo, hi) with rowptr[r] <= j (rowptr[lo] <= j must hold): the row of nonzero j.
__device__ __forceinline__ int64_t row_of_nonzero(const int32_t* __restrict__ rowptr, int64_t lo, int64_t hi, int64_t j) {
  while (hi - lo > 1) {
    const int64_t mid = (lo + hi) >> 1;
    if ((int64_t)rowptr[mid] <= j) lo = mid; else hi = mid;
  }
  return lo;
}

// nnz_row[j] = the row r with rowptr[r] <= j < rowptr[r+1] (CSR -> COO row
// expansion, the device-side form of spmm/mm/spmm_common.cpp:210-216).  A workgroup takes
// kExpandPerBlock consecutive nonzeros: two threads bisect all of rowptr for its first and last
// one, the others only between those two rows (a handful of steps instead of log2(rows)).
constexpr int kExpandPerBlock = 4 * kBlock;
HPSPMM_KERNEL __launch_bounds__(kBlock) void expand_rows_kernel(int64_t rows, int64_t nnz,
                                                             const int32_t* __restrict__ rowptr,
                                                             int32_t* __restrict__ nnz_row) {
  __shared__ int64_t s_ends[2];
  const int64_t first = (int64_t)blockIdx.x * kExpandPerBlock;
  const int64_t last = first + kExpandPerBlock - 1 < nnz ? first + kExpandPerBlock - 1 : nnz - 1;
  if (threadIdx.x == 0) s_ends[0] = row_of_nonzero(rowptr, 0, rows, first);
  if (threadIdx.x == 64) s_ends[1] = row_of_nonzero(rowptr, 0, rows, last);
  __syncthreads();
  const int64_t lo = s_ends[0], hi = s_ends[1] + 1;
  for (int64_t j = first + threadIdx.x; j <= last; j += kBlock) nnz_row[j] = (int32_t)row_of_nonzero(rowptr, lo, hi, j);
}

// out[b] = id of the XCD that workgroup b runs on (hardware register XCC_ID, bits 3:0): lets the
// plan verify the dealing of workgroups to XCDs that the routed strategy and xcd_remap assume.
HPSPMM_KERNEL __launch_bounds__(64) void xcc_probe_kernel(int32_t* __restrict__ out) {
  const unsigned v = __builtin_amdgcn_s_getreg(((4 - 1) << 11) | (0 << 6) | 20);
  if (threadIdx.x == 0) out[blockIdx.x] = (int32_t)(v & 0xFu);
}

// dst[r, 0:kp) = src[r, 0:k) followed by zeros: B with its rows padded to a multiple of 4 floats.
HPSPMM_KERNEL __launch_bounds__(kBlock) void pad_rows_kernel(int64_t rows, int64_t k, int64_t kp,
                                                          const float* __restrict__ src, float* __restrict__ dst) {
  const int64_t total = rows * kp;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < total; i += (int64_t)gridDim.x * kBlock) {
    const int64_t r = i / kp, j = i - r * kp;
    dst[i] = j < k ? src[r * k + j] : 0.f;
  }
}

HPSPMM_KERNEL __launch_bounds__(kBlock) void fill_f32_kernel(float* __restrict__ x, int64_t n, float v) {
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) x[i] = v;
}

}  // namespace hpspmm
