// Device-wide exclusive scan of 32-bit counters (three launches: tile sums, scan of the tile
// sums by one workgroup, apply) and the workgroup-wide scan it is built on.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "spmm_kernels.hpp"

namespace hpspmm {

// Three-pass exclusive scan of uint32 (n up to 2^32, total < 2^32).
constexpr int kScanItems = 16;  // per thread
constexpr int kScanTile = kBlock * kScanItems;

__device__ __forceinline__ uint32_t block_exclusive_scan(uint32_t v, uint32_t* s_wave, uint32_t& block_total) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  uint32_t incl = v;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const uint32_t o = __shfl_up(incl, off);
    if (lane >= off) incl += o;
  }
  if (lane == 63) s_wave[wave] = incl;
  __syncthreads();
  uint32_t wave_off = 0;
  uint32_t total = 0;
#pragma unroll
  for (int w = 0; w < kWavesPerBlock; ++w) {
    if (w < wave) wave_off += s_wave[w];
    total += s_wave[w];
  }
  __syncthreads();
  block_total = total;
  return wave_off + incl - v;
}

HPSPMM_KERNEL __launch_bounds__(kBlock) void scan_tile_sums_kernel(int64_t n, const uint32_t* __restrict__ in,
                                                                uint32_t* __restrict__ tile_sums) {
  __shared__ uint32_t s_wave[kWavesPerBlock];
  const int64_t base = (int64_t)blockIdx.x * kScanTile + (int64_t)threadIdx.x * kScanItems;
  uint32_t sum = 0;
#pragma unroll
  for (int i = 0; i < kScanItems; ++i)
    if (base + i < n) sum += in[base + i];
  uint32_t total;
  (void)block_exclusive_scan(sum, s_wave, total);
  if (threadIdx.x == 0) tile_sums[blockIdx.x] = total;
}

// Exclusive scan of the tile sums in place, by one workgroup.
HPSPMM_KERNEL __launch_bounds__(kBlock) void scan_tile_offsets_kernel(int64_t ntiles, uint32_t* __restrict__ tile_sums) {
  __shared__ uint32_t s_wave[kWavesPerBlock];
  uint32_t carry = 0;
  for (int64_t base = 0; base < ntiles; base += kBlock) {
    const int64_t i = base + threadIdx.x;
    const uint32_t v = i < ntiles ? tile_sums[i] : 0u;
    uint32_t total;
    const uint32_t ex = block_exclusive_scan(v, s_wave, total);
    if (i < ntiles) tile_sums[i] = carry + ex;
    carry += total;
  }
}

// (`out` may be `in`: every thread reads its items before it writes them.)
HPSPMM_KERNEL __launch_bounds__(kBlock) void scan_apply_kernel(int64_t n, const uint32_t* in,
                                                            const uint32_t* __restrict__ tile_offsets,
                                                            uint32_t* out) {
  __shared__ uint32_t s_wave[kWavesPerBlock];
  const int64_t base = (int64_t)blockIdx.x * kScanTile + (int64_t)threadIdx.x * kScanItems;
  uint32_t v[kScanItems];
  uint32_t sum = 0;
#pragma unroll
  for (int i = 0; i < kScanItems; ++i) {
    v[i] = base + i < n ? in[base + i] : 0u;
    sum += v[i];
  }
  uint32_t total;
  uint32_t run = tile_offsets[blockIdx.x] + block_exclusive_scan(sum, s_wave, total);
#pragma unroll
  for (int i = 0; i < kScanItems; ++i) {
    if (base + i < n) out[base + i] = run;
    run += v[i];
  }
}

}  // namespace hpspmm
