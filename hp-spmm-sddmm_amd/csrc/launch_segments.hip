// Segments (with or without the hub cache), the ordered strategy, COO accumulate, and the segments
// strategy from a workspace the caller brings: the launches of one SpMM.
#include "host.hpp"

#include "anyk_kernels.hpp"
#include "ordered_kernels.hpp"

namespace hpspmm_host {

namespace {

template <int GP, bool kOdd>
int launch_segments_anyk_g(const hpspmm_plan* p, const int32_t* rp, const int32_t* ci, const float* v, const float* B,
                           float* C, hipStream_t st) {
  const int tiles = anyk_tiles(p->k);
  const int64_t blocks = ceil_div(ceil_div(p->nseg, 64 / GP), hpspmm::kWavesPerBlock) * tiles;
  if (blocks > INT32_MAX) return fail(HPSPMM_ERR_INVALID_ARG, "grid too large");
  if (p->nnz > 0) {
    hipLaunchKernelGGL((hpspmm::spmm_segments_anyk_kernel<GP, false, kOdd>), dim3((unsigned)blocks), dim3(hpspmm::kBlock), 0, st, rp,
                       ci, v, p->d_nnz_row, B, C, p->d_carry, p->nnz, p->shift, p->nseg, (int)p->k, tiles,
                       aligned16(ci, v, p->d_nnz_row));
    mark_launch(st, "spmm_segments_anyk_kernel");
  }
  const int64_t fix_blocks = ceil_div(ceil_div(p->rows, 64), hpspmm::kWavesPerBlock);
  hipLaunchKernelGGL((hpspmm::spmm_fixup_anyk_kernel<GP, kOdd>), dim3((unsigned)fix_blocks), dim3(hpspmm::kBlock), 0, st,
                     p->rows, rp, (const float*)p->d_carry, C, p->shift, (int)p->k);
  mark_launch(st, "spmm_fixup_anyk_kernel");
  return HPSPMM_OK;
}

int launch_segments_anyk(const hpspmm_plan* p, const int32_t* rp, const int32_t* ci, const float* v, const float* B,
                         float* C, hipStream_t st) {
  return dispatch_anyk_lanes(p->k, [&](auto GP) {
    constexpr int gp = decltype(GP)::value;
    return odd_k(p->k) ? launch_segments_anyk_g<gp, true>(p, rp, ci, v, B, C, st)
                       : launch_segments_anyk_g<gp, false>(p, rp, ci, v, B, C, st);
  });
}

template <int GP, bool kOdd>
int launch_coo_anyk_g(int64_t nnz, int64_t k, const int32_t* ri, const int32_t* ci, const float* v, const float* B,
                      float* C, hipStream_t st) {
  constexpr int P = 64 / GP;
  const int tiles = anyk_tiles(k);
  int shift = 4;  // as launch_coo: 16 nonzeros per sub-wave, doubled while that leaves 4096 wavefronts, up to 512
  while (shift < 9 && (nnz >> (shift + 1)) / P >= 4096) ++shift;
  const int64_t nseg = ceil_div(nnz, (int64_t)1 << shift);
  const int64_t blocks = ceil_div(ceil_div(nseg, P), hpspmm::kWavesPerBlock) * tiles;
  if (blocks > INT32_MAX) return fail(HPSPMM_ERR_INVALID_ARG, "grid too large");
  hipLaunchKernelGGL((hpspmm::spmm_segments_anyk_kernel<GP, true, kOdd>), dim3((unsigned)blocks), dim3(hpspmm::kBlock), 0, st,
                     (const int32_t*)nullptr, ci, v, ri, B, C, (float*)nullptr, nnz, shift, nseg, (int)k, tiles,
                     aligned16(ci, v, ri));
  return HPSPMM_OK;
}

int launch_coo_anyk(int64_t nnz, int64_t k, const int32_t* ri, const int32_t* ci, const float* v, const float* B,
                    float* C, hipStream_t st) {
  return dispatch_anyk_lanes(k, [&](auto GP) {
    constexpr int gp = decltype(GP)::value;
    return odd_k(k) ? launch_coo_anyk_g<gp, true>(nnz, k, ri, ci, v, B, C, st)
                    : launch_coo_anyk_g<gp, false>(nnz, k, ri, ci, v, B, C, st);
  });
}

// Rows scanned by one wavefront of the fix-up kernel: 64, or one per sub-wave while that still
// leaves the grid small.
inline int fixup_rows_per_wave(int64_t rows, int k) { return rows <= (1 << 18) ? 64 / (k / 4) : 64; }

template <int K>
int launch_segments(const hpspmm_plan* p, const int32_t* rp, const int32_t* ci, const float* v,
                    const float* B, float* C, hipStream_t st) {
  constexpr int P = 64 / (K / 4);
  const int64_t nblocks = ceil_div(ceil_div(p->nseg, P), hpspmm::kWavesPerBlock);
  const int64_t grid = p->xcd_remap ? ceil_div(nblocks, hpspmm::kXcds) * hpspmm::kXcds : nblocks;
  if (grid > INT32_MAX) return fail(HPSPMM_ERR_INVALID_ARG, "grid too large");
  if (p->nnz > 0) {
    if (p->n_hub > 0) {
      const int64_t threads = p->n_hub * (K / 4);
      hipLaunchKernelGGL(hpspmm::gather_hub_rows_kernel<K>, dim3((unsigned)ceil_div(threads, hpspmm::kBlock)),
                         dim3(hpspmm::kBlock), 0, st, p->n_hub, p->d_hub_ids, B, p->d_bhot);
      mark_launch(st, "gather_hub_rows_kernel");
      hipLaunchKernelGGL((hpspmm::spmm_segments_kernel<K, false, true>), dim3((unsigned)grid), dim3(hpspmm::kBlock),
                         0, st, rp, p->d_hub_col, v, p->d_nnz_row, B, p->d_bhot, C, p->d_carry, p->nnz, p->shift,
                         p->nseg, nblocks, p->xcd_remap, aligned16(p->d_hub_col, v, p->d_nnz_row));
    } else {
      hipLaunchKernelGGL((hpspmm::spmm_segments_kernel<K, false, false>), dim3((unsigned)grid),
                         dim3(hpspmm::kBlock), 0, st, rp, ci, v, p->d_nnz_row, B, (const float*)nullptr, C,
                         p->d_carry, p->nnz, p->shift, p->nseg, nblocks, p->xcd_remap,
                         aligned16(ci, v, p->d_nnz_row));
    }
    mark_launch(st, "spmm_segments_kernel");
  }
  const int rpw = fixup_rows_per_wave(p->rows, K);
  const int64_t fix_blocks = ceil_div(ceil_div(p->rows, rpw), hpspmm::kWavesPerBlock);
  hipLaunchKernelGGL(hpspmm::spmm_fixup_kernel<K>, dim3((unsigned)fix_blocks), dim3(hpspmm::kBlock), 0, st, p->rows,
                     rp, (const int32_t*)nullptr, p->d_carry, C, p->shift, rpw, (uint32_t)K);
  mark_launch(st, "spmm_fixup_kernel");
  return HPSPMM_OK;
}

// kLd: B and C are K columns of wider arrays whose rows are `ld` floats apart (one column tile).
template <int K, int kLd = 0>
int launch_ordered(const hpspmm_plan* p, const int32_t* rp, const float* v, const float* B, float* C,
                   hipStream_t st, uint32_t ld = K) {
  const int64_t nblocks = p->owindows;
  const int64_t grid = p->xcd_remap ? ceil_div(nblocks, hpspmm::kXcds) * hpspmm::kXcds : nblocks;
  if (grid > INT32_MAX) return fail(HPSPMM_ERR_INVALID_ARG, "grid too large");
  if (p->nnz > 0) {
    hipLaunchKernelGGL((hpspmm::spmm_ordered_kernel<K, kLd>), dim3((unsigned)grid), dim3(hpspmm::kBlock),
                       (size_t)p->ocap * K * sizeof(float), st, rp, p->d_ostart, p->d_ocol, p->d_run_row, p->d_run_delta,
                       p->d_seg_run, v, p->d_wcols, p->ocap, B, C, p->d_carry, p->nnz, p->shift, nblocks, p->xcd_remap,
                       ld);
    mark_launch(st, "spmm_ordered_kernel");
  }
  const int64_t cross_blocks = row_blocks(p->n_cross, K);
  const int64_t fix_blocks = cross_blocks + row_blocks(p->n_zero, K);
  if (fix_blocks > 0) {
    hipLaunchKernelGGL((hpspmm::spmm_ordered_fixup_kernel<K, kLd>), dim3((unsigned)fix_blocks), dim3(hpspmm::kBlock), 0,
                       st, rp, p->d_ostart, p->d_cross_rows, p->n_cross, cross_blocks, p->d_zero_rows, p->n_zero,
                       p->d_carry, C, p->shift, ld);
    mark_launch(st, "spmm_ordered_fixup_kernel");
  }
  return HPSPMM_OK;
}

template <int K>
int launch_coo(int64_t nnz, const int32_t* ri, const int32_t* ci, const float* v, const float* B, float* C,
               hipStream_t st) {
  constexpr int P = 64 / (K / 4);
  // 16 nonzeros per sub-wave, and twice that as long as this leaves 4096 wavefronts, up to 512: the
  // one flush per segment end is the better amortised the longer the segment, and every SIMD still
  // has several wavefronts (social graph, K = 32: 2.16 ms at 64 nonzeros, 1.44 ms at 512; K = 128:
  // 8.33 -> 7.06; R-MAT K = 128: 14.3 -> 13.3; the 20k-vertex citation graph stays at 16)
  int shift = 4;
  while (shift < 9 && (nnz >> (shift + 1)) / P >= 4096) ++shift;
  const int64_t nseg = ceil_div(nnz, (int64_t)1 << shift);
  const int64_t nblocks = ceil_div(ceil_div(nseg, P), hpspmm::kWavesPerBlock);
  if (nblocks > INT32_MAX) return fail(HPSPMM_ERR_INVALID_ARG, "grid too large");
  hipLaunchKernelGGL((hpspmm::spmm_segments_kernel<K, true, false>), dim3((unsigned)nblocks), dim3(hpspmm::kBlock),
                     0, st, (const int32_t*)nullptr, ci, v, ri, B, (const float*)nullptr, C, (float*)nullptr, nnz,
                     shift, nseg, nblocks, false, aligned16(ci, v, ri));
  return HPSPMM_OK;
}

template <int K>
int launch_workspace(int64_t rows, int64_t nnz, const int32_t* rp, const int32_t* ci, const float* v, const float* B,
                     float* C, int32_t* nnz_row, float* carry, int64_t carry_floats, hipStream_t st) {
  constexpr int P = 64 / (K / 4);
  // segment length as a plan would choose it, then doubled until the carry slots fit the workspace
  int shift = 5;
  const int64_t target_waves = 256 * 4 * 16;
  while (shift < 9 && (nnz >> (shift + 1)) / P >= target_waves) ++shift;
  while (2 * ceil_div(nnz, (int64_t)1 << shift) * K > carry_floats) ++shift;
  const int64_t nseg = ceil_div(nnz, (int64_t)1 << shift);
  if (nnz > 0) {
    hipLaunchKernelGGL(hpspmm::expand_rows_kernel, dim3((unsigned)ceil_div(nnz, hpspmm::kExpandPerBlock)), dim3(hpspmm::kBlock),
                       0, st, rows, nnz, rp, nnz_row);
    const int64_t nblocks = ceil_div(ceil_div(nseg, P), hpspmm::kWavesPerBlock);
    hipLaunchKernelGGL((hpspmm::spmm_segments_kernel<K, false, false>), dim3((unsigned)nblocks), dim3(hpspmm::kBlock),
                       0, st, rp, ci, v, (const int32_t*)nnz_row, B, (const float*)nullptr, C, carry, nnz, shift, nseg,
                       nblocks, false, aligned16(ci, v, nnz_row));
  }
  const int rpw = fixup_rows_per_wave(rows, K);
  const int64_t fix_blocks = ceil_div(ceil_div(rows, rpw), hpspmm::kWavesPerBlock);
  hipLaunchKernelGGL(hpspmm::spmm_fixup_kernel<K>, dim3((unsigned)fix_blocks), dim3(hpspmm::kBlock), 0, st, rows, rp,
                     (const int32_t*)nullptr, (const float*)carry, C, shift, rpw, (uint32_t)K);
  return HPSPMM_OK;
}

}  // namespace

int launch_segments_plan(const hpspmm_plan* p, const int32_t* rp, const int32_t* ci, const float* v, const float* B,
                         float* C, hipStream_t st) {
  if (!fast_k(p->k)) return launch_segments_anyk(p, rp, ci, v, B, C, st);
  return dispatch_k(p->k, [&](auto K) { return launch_segments<decltype(K)::value>(p, rp, ci, v, B, C, st); });
}

int launch_ordered_plan(const hpspmm_plan* p, const int32_t* rp, const float* v, const float* B, float* C,
                        hipStream_t st, int ld_mode, uint32_t ld) {
  return dispatch_k_ld(p->k, ld_mode, [&](auto K, auto L) {
    return launch_ordered<decltype(K)::value, decltype(L)::value>(p, rp, v, B, C, st, ld);
  });
}

int launch_coo_any(int64_t nnz, int64_t k, const int32_t* ri, const int32_t* ci, const float* v, const float* B,
                   float* C, hipStream_t st) {
  if (!fast_k(k)) return launch_coo_anyk(nnz, k, ri, ci, v, B, C, st);  // segments reduced in registers, one atomic per flush
  return dispatch_k(k, [&](auto K) { return launch_coo<decltype(K)::value>(nnz, ri, ci, v, B, C, st); });
}

int launch_segments_workspace(int64_t rows, int64_t nnz, int64_t k, const int32_t* rp, const int32_t* ci,
                              const float* v, const float* B, float* C, int32_t* nnz_row, float* carry,
                              int64_t carry_floats, hipStream_t st) {
  return dispatch_k(k, [&](auto K) {
    return launch_workspace<decltype(K)::value>(rows, nnz, rp, ci, v, B, C, nnz_row, carry, carry_floats, st);
  });
}

}  // namespace hpspmm_host
