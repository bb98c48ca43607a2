// gfx950 device code for FP32 CSR SpMM with a row length K of B and C that is not one of the tuned
// sizes 32 / 64 / 128 (K = 8, 16, 48, 100, 160, ... and, with kOdd, any K at all: 7, 41, 47, 173).
//
// The same work decomposition as the tuned kernels, with the row length at run time: a sub-wave is
// GP adjacent lanes (GP a power of two, 2 ... 32), lane l owns the four columns [k0 + 4l, k0 + 4l + 4)
// of a column tile that starts at k0 and is `kw` <= 4 GP floats wide; lanes whose columns lie beyond
// the tile idle (K = 48: 12 of 16 lanes work).  K <= 128 is one tile, a longer row is cut into
// tiles of 128 floats served by separate workgroups (workgroup b serves tile b % tiles).
//
// kOdd = K is not a multiple of 4: the rows of B and C then start at any multiple of 4 bytes, so
// their 16-byte accesses are declared 4-byte aligned, and the lane that owns the last columns of a
// row reads and writes only those that exist (K = 41: lane 10 owns column 40 alone).  The carry
// slots keep rows of K rounded up to 4 floats.  (The number of classes of a node classifier is such
// a K - 41, 47, 172 ...; one wavefront per row with scalar loads was 6 to 25 times slower.)
//
//   spmm_rows_anyk_kernel      one sub-wave per CSR row, rows beyond a threshold by a whole
//                              wavefront (the plan lists them) - small matrices, no plan
//   spmm_segments_anyk_kernel  one sub-wave per fixed-length run of nonzeros, carry slots for the
//   spmm_fixup_anyk_kernel     rows cut by a segment boundary - everything else
//
// What this replaces in the reference: the K < 32 row-per-warp kernel
// (spmm/mm/spmm_kernel.cu:372-387, dispatch :406-410), whose lanes beyond K idle in the same way, and
// the column-tile loop of the wider sizes (:412-421).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "spmm_kernels.hpp"

namespace hpspmm {

constexpr int kAnyKTile = 128;  // widest column tile, floats

// Column tile of a workgroup: tile index b % tiles (every tile kAnyKTile wide but the last).
struct ColumnTile {
  int k0;       // first column
  int nv;       // how many of this lane's four columns exist (0 ... 4)
  bool active;  // nv > 0
};
__device__ __forceinline__ ColumnTile column_tile(int tile, int K, int l) {
  ColumnTile t;
  t.k0 = tile * kAnyKTile;
  const int kw = K - t.k0 < kAnyKTile ? K - t.k0 : kAnyKTile;
  const int left = kw - 4 * l;
  t.nv = left < 0 ? 0 : left > 4 ? 4 : left;
  t.active = t.nv > 0;
  return t;
}

// The first nv (1 ... 4) of the four floats at p, zeros for the rest; kOdd = false: all four, p 16-byte aligned.
template <bool kOdd>
__device__ __forceinline__ float4 load_columns(const float* __restrict__ p, int nv) {
  if constexpr (!kOdd) {
    return *reinterpret_cast<const float4*>(p);
  } else {
    if (nv == 4) {
      const Float4Unaligned u = *reinterpret_cast<const Float4Unaligned*>(p);
      return make_float4(u.x, u.y, u.z, u.w);
    }
    float4 r = make_float4(p[0], 0.f, 0.f, 0.f);
    if (nv > 1) r.y = p[1];
    if (nv > 2) r.z = p[2];
    return r;
  }
}

// The first nv of v's components to p (a row of C); kOdd = false: all four.
template <bool kOdd>
__device__ __forceinline__ void store_columns(float* __restrict__ p, const float4& v, int nv) {
  if constexpr (!kOdd) {
    store_result(p, v);
  } else {
    __builtin_nontemporal_store(v.x, p);
    if (nv > 1) __builtin_nontemporal_store(v.y, p + 1);
    if (nv > 2) __builtin_nontemporal_store(v.z, p + 2);
    if (nv > 3) __builtin_nontemporal_store(v.w, p + 3);
  }
}

// dst[0..TL) = src[q .. q+TL) for the tile sizes of narrow sub-waves (TL = 8, 16); the tuned sizes
// go through load_run.
template <int TL, typename T>
__device__ __forceinline__ void load_run_wide(T (&dst)[TL], const T* __restrict__ src, int64_t q, int64_t e,
                                              bool vec_ok) {
  if constexpr (TL <= 4) {
    load_run<TL>(dst, src, q, e, vec_ok);
  } else {
    if (vec_ok && q + TL <= e) {
#pragma unroll
      for (int i = 0; i < TL; i += 4) {
        const int4 w = *reinterpret_cast<const int4*>(src + q + i);
        dst[i] = __builtin_bit_cast(T, w.x);
        dst[i + 1] = __builtin_bit_cast(T, w.y);
        dst[i + 2] = __builtin_bit_cast(T, w.z);
        dst[i + 3] = __builtin_bit_cast(T, w.w);
      }
    } else {
#pragma unroll
      for (int i = 0; i < TL; ++i) dst[i] = q + i < e ? src[q + i] : T(0);
    }
  }
}

template <int TL>
__device__ __forceinline__ void stage_tile_wide(const TileRegs<TL>& m, int slot, int32_t* s_col, float* s_val,
                                                int32_t* s_row) {
  if constexpr (TL <= 4) {
    stage_tile<TL>(m, slot, s_col, s_val, s_row);
  } else {
#pragma unroll
    for (int i = 0; i < TL; i += 4) {
      *reinterpret_cast<int4*>(s_col + slot + i) = make_int4(m.c[i], m.c[i + 1], m.c[i + 2], m.c[i + 3]);
      *reinterpret_cast<float4*>(s_val + slot + i) = make_float4(m.v[i], m.v[i + 1], m.v[i + 2], m.v[i + 3]);
      *reinterpret_cast<int4*>(s_row + slot + i) = make_int4(m.r[i], m.r[i + 1], m.r[i + 2], m.r[i + 3]);
    }
  }
}

// acc += sum over nonzeros [lb, hb) of val[j] * B[col[j], k0 + 4l ...), by the lanes of one sub-wave
// together.  Every lane reads the column and the value itself (the lanes of a sub-wave read the
// same address, which the memory pipeline serves as one request), eight nonzeros in flight.
template <bool kOdd>
__device__ __forceinline__ void accumulate_range_anyk(float4& acc, int32_t lb, int32_t hb,
                                                      const int32_t* __restrict__ col,
                                                      const float* __restrict__ val, const float* __restrict__ Bl,
                                                      int64_t K, bool active, int nv) {
  int32_t j = lb;
  for (; j + kBatch <= hb; j += kBatch) {
    int32_t c[kBatch];
    float v[kBatch];
    float4 b[kBatch];
#pragma unroll
    for (int i = 0; i < kBatch; ++i) {
      c[i] = col[j + i];
      v[i] = val[j + i];
    }
#pragma unroll
    for (int i = 0; i < kBatch; ++i)
      b[i] = active ? load_columns<kOdd>(Bl + (uint64_t)(uint32_t)c[i] * (uint64_t)K, nv)
                    : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int i = 0; i < kBatch; ++i) fma4(acc, v[i], b[i]);
  }
  for (; j < hb; ++j) {
    const float4 b = active ? load_columns<kOdd>(Bl + (uint64_t)(uint32_t)col[j] * (uint64_t)K, nv)
                            : make_float4(0.f, 0.f, 0.f, 0.f);
    fma4(acc, val[j], b);
  }
}

// Workgroup b serves column tile b % tiles.  Within a tile: workgroups [0, short_blocks) run one
// sub-wave per row and skip rows longer than long_threshold; the remaining ones run one wavefront per
// entry of long_rows[], the row's nonzeros dealt in contiguous runs to the sub-waves and the partial
// sums combined with wavefront shuffles.
template <int GP, bool kOdd>
__global__ __launch_bounds__(kBlock) void spmm_rows_anyk_kernel(int64_t rows, int K, int tiles,
                                                                const int32_t* __restrict__ rowptr,
                                                                const int32_t* __restrict__ col,
                                                                const float* __restrict__ val,
                                                                const float* __restrict__ B, float* __restrict__ C,
                                                                int64_t short_blocks, int32_t long_threshold,
                                                                const int32_t* __restrict__ long_rows,
                                                                int64_t n_long) {
  constexpr int P = 64 / GP;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int l = lane % GP;
  const ColumnTile ct = column_tile((int)(blockIdx.x % tiles), K, l);
  const int64_t blk = blockIdx.x / tiles;
  const float* Bl = B + ct.k0 + 4 * l;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);

  if (blk < short_blocks) {
    const int64_t row = (blk * kWavesPerBlock + (tid >> 6)) * P + lane / GP;
    if (row >= rows) return;
    const int32_t lb = rowptr[row];
    const int32_t hb = rowptr[row + 1];
    if (hb - lb > long_threshold) return;
    accumulate_range_anyk<kOdd>(acc, lb, hb, col, val, Bl, K, ct.active, ct.nv);
    if (ct.active) store_columns<kOdd>(C + (uint64_t)row * K + ct.k0 + 4 * l, acc, ct.nv);
  } else {
    const int64_t w = (blk - short_blocks) * kWavesPerBlock + (tid >> 6);
    if (w >= n_long) return;
    const int32_t row = long_rows[w];
    const int32_t lb = rowptr[row];
    const int32_t hb = rowptr[row + 1];
    const int32_t per = (hb - lb + P - 1) / P;
    const int32_t my_lb = lb + (lane / GP) * per < hb ? lb + (lane / GP) * per : hb;
    const int32_t my_hb = (my_lb + per) < hb ? (my_lb + per) : hb;
    accumulate_range_anyk<kOdd>(acc, my_lb, my_hb, col, val, Bl, K, ct.active, ct.nv);
#pragma unroll
    for (int off = GP; off < 64; off <<= 1) {
      acc.x += __shfl_xor(acc.x, off);
      acc.y += __shfl_xor(acc.y, off);
      acc.z += __shfl_xor(acc.z, off);
      acc.w += __shfl_xor(acc.w, off);
    }
    if (lane < GP && ct.active) store_columns<kOdd>(C + (uint64_t)(uint32_t)row * K + ct.k0 + 4 * l, acc, ct.nv);
  }
}

// The segments kernel (see spmm_segments_kernel for the carry rule) with the row length at run time.
// Workgroup b serves column tile b % tiles of segment group b / tiles.  kAtomic = the COO
// "accumulate" form: nnz_row is the caller's row array (any order), no carry slots, every flush an
// FP32 atomic add into C.
template <int GP, bool kAtomic, bool kOdd>
__global__ __launch_bounds__(kBlock) void spmm_segments_anyk_kernel(
    const int32_t* __restrict__ rowptr, const int32_t* __restrict__ col, const float* __restrict__ val,
    const int32_t* __restrict__ nnz_row, const float* __restrict__ B, float* __restrict__ C,
    float* __restrict__ carry, int64_t nnz, int shift, int64_t nseg, int K, int tiles, bool vec_ok) {
  const int64_t Kc = (K + 3) & ~3;  // floats of a carry slot
  constexpr int G = GP;
  constexpr int P = 64 / G;
  constexpr int TL = kTile / G;
  __shared__ __attribute__((aligned(16))) int32_t s_col[kWavesPerBlock * P * kTileStride];
  __shared__ __attribute__((aligned(16))) float s_val[kWavesPerBlock * P * kTileStride];
  __shared__ __attribute__((aligned(16))) int32_t s_row[kWavesPerBlock * P * kTileStride];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int l = lane % G;
  const ColumnTile ct = column_tile((int)(blockIdx.x % tiles), K, l);
  const int64_t blk = blockIdx.x / tiles;
  const int64_t g = (blk * kWavesPerBlock + (tid >> 6)) * P + lane / G;
  if (g >= nseg) return;

  const int64_t s = g << shift;
  const int64_t e = (s + ((int64_t)1 << shift)) < nnz ? (s + ((int64_t)1 << shift)) : nnz;
  const int sbase = ((tid >> 6) * P + lane / G) * kTileStride;
  const float* Bl = B + ct.k0 + 4 * l;
  const int64_t off = ct.k0 + 4 * l;

  int32_t cur = nnz_row[s];
  bool head_pending = false;
  if constexpr (!kAtomic) head_pending = (int64_t)rowptr[cur] < s;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);

  auto flush_to = [&](bool is_tail) {
    if constexpr (kAtomic) {
      if (ct.active) {
        float* dst = C + (uint64_t)(uint32_t)cur * K + off;
        unsafeAtomicAdd(dst + 0, acc.x);
        if (!kOdd || ct.nv > 1) unsafeAtomicAdd(dst + 1, acc.y);
        if (!kOdd || ct.nv > 2) unsafeAtomicAdd(dst + 2, acc.z);
        if (!kOdd || ct.nv > 3) unsafeAtomicAdd(dst + 3, acc.w);
      }
    } else {
      const bool to_carry = head_pending || is_tail;
      float* dst = head_pending ? carry + (uint64_t)(2 * g) * Kc
                                : (is_tail ? carry + (uint64_t)(2 * g + 1) * Kc : C + (uint64_t)(uint32_t)cur * K);
      head_pending = false;
      if (ct.active) {
        if (to_carry) store_result(dst + off, acc);  // a carry slot has room for all four
        else store_columns<kOdd>(dst + off, acc, ct.nv);
      }
    }
  };
  auto flush = [&]() { flush_to(false); };
  auto loadb = [&](int32_t c) {
    return ct.active ? load_columns<kOdd>(Bl + (uint64_t)(uint32_t)c * (uint64_t)K, ct.nv)
                     : make_float4(0.f, 0.f, 0.f, 0.f);
  };
  auto fetch = [&](TileRegs<TL>& m, int64_t t) {
    const int64_t q = t + l * TL;
    load_run_wide<TL>(m.c, col, q, e, vec_ok);
    load_run_wide<TL>(m.v, val, q, e, vec_ok);
    load_run_wide<TL>(m.r, nnz_row, q, e, vec_ok);
  };

  TileRegs<TL> m;
  fetch(m, s);
  for (int64_t t = s; t < e; t += kTile) {
    stage_tile_wide<TL>(m, sbase + l * TL, s_col, s_val, s_row);
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

// Fix-up after the segments kernel (see spmm_fixup_kernel): one row per lane is classified, the
// sub-waves then zero the empty rows and add the carry slots of the split ones in segment order, one
// column tile after the other.
template <int GP, bool kOdd>
__global__ __launch_bounds__(kBlock) void spmm_fixup_anyk_kernel(int64_t rows, const int32_t* __restrict__ rowptr,
                                                                 const float* __restrict__ carry,
                                                                 float* __restrict__ C, int shift, int K) {
  constexpr int P = 64 / GP;
  const int64_t Kc = (K + 3) & ~3;  // floats of a carry slot
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int l = lane % GP;
  const int sub = lane / GP;
  const int64_t r0 = ((int64_t)blockIdx.x * kWavesPerBlock + (tid >> 6)) * 64;
  if (r0 >= rows) return;
  const int64_t r = r0 + lane;
  const bool valid = r < rows;
  const int32_t lb = valid ? rowptr[r] : 0;
  const int32_t hb = valid ? rowptr[r + 1] : 0;
  const bool empty = valid && lb == hb;
  const bool split = valid && lb != hb && ((int64_t)lb >> shift) != ((int64_t)(hb - 1) >> shift);
  const uint64_t m_empty = __ballot(empty);
  const uint64_t m_split = __ballot(split);
  if ((m_empty | m_split) == 0) return;
  for (int i = sub; i < 64; i += P) {
    const int32_t lb_i = __shfl(lb, i);
    const int32_t hb_i = __shfl(hb, i);
    const bool is_empty = (m_empty >> i) & 1ull, is_split = (m_split >> i) & 1ull;
    if (!is_empty && !is_split) continue;
    for (int k0 = 4 * l; k0 < K; k0 += 4 * GP) {
      float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
      if (is_split) {
        const int64_t ga = (int64_t)lb_i >> shift;
        const int64_t gb = (int64_t)(hb_i - 1) >> shift;
        acc = *reinterpret_cast<const float4*>(carry + (uint64_t)(2 * ga + 1) * Kc + k0);
        for (int64_t g = ga + 1; g <= gb; ++g) {
          const float4 h = *reinterpret_cast<const float4*>(carry + (uint64_t)(2 * g) * Kc + k0);
          acc.x += h.x;
          acc.y += h.y;
          acc.z += h.z;
          acc.w += h.w;
        }
      }
      if constexpr (kOdd) {
        float* out = C + (uint64_t)(r0 + i) * K + k0;
        const int nv = K - k0 < 4 ? K - k0 : 4;
        out[0] = acc.x;
        if (nv > 1) out[1] = acc.y;
        if (nv > 2) out[2] = acc.z;
        if (nv > 3) out[3] = acc.w;
      } else {
        *reinterpret_cast<float4*>(C + (uint64_t)(r0 + i) * K + k0) = acc;
      }
    }
  }
}

}  // namespace hpspmm
