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

namespace hpspmm {

constexpr int kBlock = 256;         // threads per workgroup = 4 wavefronts
constexpr int kWavesPerBlock = 4;
constexpr int kBatch = 8;           // B-row fragments in flight per lane
constexpr int kXcds = 8;            // accelerator complex dies, each with its own L2

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

template <int K>
__device__ __forceinline__ float4 load_b(const float* __restrict__ B, int32_t c, int l) {
  // 64-bit address: cols * K * 4 reaches 2^31 bytes at the largest benchmark size
  return *reinterpret_cast<const float4*>(B + (uint64_t)(uint32_t)c * (uint64_t)K + (uint32_t)(4 * l));
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
// rows kernel: one sub-wave per CSR row.
// ---------------------------------------------------------------------------
template <int K>
__global__ __launch_bounds__(kBlock) void spmm_rows_kernel(int64_t rows, const int32_t* __restrict__ rowptr,
                                                           const int32_t* __restrict__ col,
                                                           const float* __restrict__ val,
                                                           const float* __restrict__ B, float* __restrict__ C) {
  constexpr int G = K / 4;
  constexpr int P = 64 / G;
  constexpr int U = G < kBatch ? G : kBatch;
  __shared__ int32_t s_col[kBlock];
  __shared__ float s_val[kBlock];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int l = lane % G;
  const int64_t row = ((int64_t)blockIdx.x * kWavesPerBlock + (tid >> 6)) * P + lane / G;
  if (row >= rows) return;

  const int32_t lb = rowptr[row];
  const int32_t hb = rowptr[row + 1];
  const int base = tid - l;  // LDS slot of this sub-wave's lane 0
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);

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
      for (int i = 0; i < U; ++i) b[i] = load_b<K>(B, c[i], l);
#pragma unroll
      for (int i = 0; i < U; ++i) fma4(acc, v[i], b[i]);
    }
    for (; u < cnt; ++u) {
      const float4 b = load_b<K>(B, s_col[base + u], l);
      fma4(acc, s_val[base + u], b);
    }
    wave_lds_fence();
  }
  *reinterpret_cast<float4*>(C + (uint64_t)row * K + 4 * l) = acc;
}

// Any K: one wavefront per row, lanes stride over columns.
__global__ __launch_bounds__(kBlock) void spmm_rows_generic_kernel(int64_t rows, int64_t K,
                                                                   const int32_t* __restrict__ rowptr,
                                                                   const int32_t* __restrict__ col,
                                                                   const float* __restrict__ val,
                                                                   const float* __restrict__ B,
                                                                   float* __restrict__ C) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int32_t lb = rowptr[row];
  const int32_t hb = rowptr[row + 1];
  for (int64_t k0 = lane; k0 < K; k0 += 64) {
    float acc = 0.f;
    for (int32_t j = lb; j < hb; ++j)
      acc = __builtin_fmaf(val[j], B[(uint64_t)(uint32_t)col[j] * (uint64_t)K + (uint64_t)k0], acc);
    C[(uint64_t)row * (uint64_t)K + (uint64_t)k0] = acc;
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
template <int K, bool kAtomic>
__global__ __launch_bounds__(kBlock) void spmm_segments_kernel(
    const int32_t* __restrict__ rowptr, const int32_t* __restrict__ col, const float* __restrict__ val,
    const int32_t* __restrict__ nnz_row, const float* __restrict__ B, float* __restrict__ C,
    float* __restrict__ carry, int64_t nnz, int shift, int64_t nseg, int64_t nblocks, bool remap) {
  constexpr int G = K / 4;
  constexpr int P = 64 / G;
  constexpr int U = G < kBatch ? G : kBatch;
  __shared__ int32_t s_col[kBlock];
  __shared__ float s_val[kBlock];
  __shared__ int32_t s_row[kBlock];

  const int64_t blk = xcd_remap(blockIdx.x, nblocks, remap);
  if (blk < 0) return;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int l = lane % G;
  const int64_t g = (blk * kWavesPerBlock + (tid >> 6)) * P + lane / G;
  if (g >= nseg) return;

  const int64_t s = g << shift;
  const int64_t e = (s + ((int64_t)1 << shift)) < nnz ? (s + ((int64_t)1 << shift)) : nnz;
  const int base = tid - l;

  int32_t cur = nnz_row[s];
  bool head_pending = false;
  if constexpr (!kAtomic) head_pending = (int64_t)rowptr[cur] < s;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);

  auto flush = [&](bool is_tail) {
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
      *reinterpret_cast<float4*>(dst + 4 * l) = acc;
    }
  };

  for (int64_t t = s; t < e; t += G) {
    const int64_t p = t + l;
    if (p < e) {
      s_col[tid] = col[p];
      s_val[tid] = val[p];
      s_row[tid] = nnz_row[p];
    }
    wave_lds_fence();
    const int cnt = (e - t) < G ? (int)(e - t) : G;
    int u = 0;
    for (; u + U <= cnt; u += U) {
      int32_t c[U], r[U];
      float v[U];
      float4 b[U];
#pragma unroll
      for (int i = 0; i < U; ++i) {
        c[i] = s_col[base + u + i];
        v[i] = s_val[base + u + i];
        r[i] = s_row[base + u + i];
      }
#pragma unroll
      for (int i = 0; i < U; ++i) b[i] = load_b<K>(B, c[i], l);
#pragma unroll
      for (int i = 0; i < U; ++i) {
        if (r[i] != cur) {
          flush(false);
          acc = make_float4(0.f, 0.f, 0.f, 0.f);
          cur = r[i];
        }
        fma4(acc, v[i], b[i]);
      }
    }
    for (; u < cnt; ++u) {
      const int32_t r = s_row[base + u];
      const float4 b = load_b<K>(B, s_col[base + u], l);
      if (r != cur) {
        flush(false);
        acc = make_float4(0.f, 0.f, 0.f, 0.f);
        cur = r;
      }
      fma4(acc, s_val[base + u], b);
    }
    wave_lds_fence();
  }
  bool continues = false;
  if constexpr (!kAtomic) continues = (int64_t)rowptr[cur + 1] > e;
  flush(continues);
}

// Fix-up after the segments kernel: one sub-wave per row.  Empty rows are
// zeroed; rows that cross a segment boundary are summed from the carry buffer
// in segment order; all other rows were already stored.
template <int K>
__global__ __launch_bounds__(kBlock) void spmm_fixup_kernel(int64_t rows, const int32_t* __restrict__ rowptr,
                                                            const float* __restrict__ carry,
                                                            float* __restrict__ C, int shift) {
  constexpr int G = K / 4;
  constexpr int P = 64 / G;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int l = lane % G;
  const int64_t row = ((int64_t)blockIdx.x * kWavesPerBlock + (tid >> 6)) * P + lane / G;
  if (row >= rows) return;
  const int64_t lb = rowptr[row];
  const int64_t hb = rowptr[row + 1];
  float4* out = reinterpret_cast<float4*>(C + (uint64_t)row * K + 4 * l);
  if (lb == hb) {
    *out = make_float4(0.f, 0.f, 0.f, 0.f);
    return;
  }
  const int64_t ga = lb >> shift;
  const int64_t gb = (hb - 1) >> shift;
  if (ga == gb) return;
  float4 acc = *reinterpret_cast<const float4*>(carry + (uint64_t)(2 * ga + 1) * K + 4 * l);
  int64_t g = ga + 1;
  for (; g + kBatch <= gb + 1; g += kBatch) {
    float4 part[kBatch];
#pragma unroll
    for (int i = 0; i < kBatch; ++i)
      part[i] = *reinterpret_cast<const float4*>(carry + (uint64_t)(2 * (g + i)) * K + 4 * l);
#pragma unroll
    for (int i = 0; i < kBatch; ++i) {
      acc.x += part[i].x;
      acc.y += part[i].y;
      acc.z += part[i].z;
      acc.w += part[i].w;
    }
  }
  for (; g <= gb; ++g) {
    const float4 part = *reinterpret_cast<const float4*>(carry + (uint64_t)(2 * g) * K + 4 * l);
    acc.x += part.x;
    acc.y += part.y;
    acc.z += part.z;
    acc.w += part.w;
  }
  *out = acc;
}

// COO accumulate for any K: one thread per (entry, column).
__global__ __launch_bounds__(kBlock) void spmm_coo_generic_kernel(int64_t nnz, int64_t K,
                                                                  const int32_t* __restrict__ row,
                                                                  const int32_t* __restrict__ col,
                                                                  const float* __restrict__ val,
                                                                  const float* __restrict__ B,
                                                                  float* __restrict__ C) {
  const int64_t total = nnz * K;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < total; i += (int64_t)gridDim.x * kBlock) {
    const int64_t j = i / K;
    const int64_t k0 = i - j * K;
    unsafeAtomicAdd(C + (uint64_t)(uint32_t)row[j] * (uint64_t)K + (uint64_t)k0,
                    val[j] * B[(uint64_t)(uint32_t)col[j] * (uint64_t)K + (uint64_t)k0]);
  }
}

// ---------------------------------------------------------------------------
// Plan-time kernels.
// ---------------------------------------------------------------------------

// status[0] |= 1 rowptr[0] != 0, |= 2 rowptr decreases, |= 4 rowptr[rows] != nnz,
//           |= 8 column index out of [0, cols).
__global__ __launch_bounds__(kBlock) void validate_csr_kernel(int64_t rows, int64_t cols, int64_t nnz,
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
__global__ __launch_bounds__(kBlock) void row_stats_kernel(int64_t rows, const int32_t* __restrict__ rowptr,
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

// nnz_row[j] = the row r with rowptr[r] <= j < rowptr[r+1] (CSR -> COO row
// expansion, the device-side form of spmm/mm/spmm_common.cpp:210-216).
__global__ __launch_bounds__(kBlock) void expand_rows_kernel(int64_t rows, int64_t nnz,
                                                             const int32_t* __restrict__ rowptr,
                                                             int32_t* __restrict__ nnz_row) {
  const int64_t j = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (j >= nnz) return;
  // largest r in [0, rows) with rowptr[r] <= j
  int64_t lo = 0, hi = rows;  // invariant: rowptr[lo] <= j, answer in [lo, hi)
  while (hi - lo > 1) {
    const int64_t mid = (lo + hi) >> 1;
    if ((int64_t)rowptr[mid] <= j) lo = mid; else hi = mid;
  }
  nnz_row[j] = (int32_t)lo;
}

__global__ __launch_bounds__(kBlock) void fill_f32_kernel(float* __restrict__ x, int64_t n, float v) {
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) x[i] = v;
}

}  // namespace hpspmm
