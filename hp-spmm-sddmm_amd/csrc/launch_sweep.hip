// Sweep strategy: the launches of one SpMM, and the values bound to a plan.
#include "host.hpp"

namespace hpspmm_host {

namespace {

// Lets the sweep kernels have their LDS; *out = workgroups of them that one CU holds (1 is what the
// layout is made for).
template <int K>
int sweep_prepare_kernels_k(int* out) {
  const size_t lds = hpspmm::sweep_lds_bytes<K>();
  HPSPMM_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&hpspmm::spmm_sweep_kernel<K, true>),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  HPSPMM_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&hpspmm::spmm_sweep_kernel<K, false>),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  HPSPMM_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&hpspmm::spmm_sweep_kernel<K, true, 1>),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  HPSPMM_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&hpspmm::spmm_sweep_kernel<K, false, 1>),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  HPSPMM_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&hpspmm::spmm_sweep_kernel<K, true, 2>),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  HPSPMM_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&hpspmm::spmm_sweep_kernel<K, false, 2>),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  HPSPMM_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(out, hpspmm::spmm_sweep_kernel<K, true>,
                                                          hpspmm::sweep_waves<K>() * 64, lds));
  return HPSPMM_OK;
}

// kLd: B and C are K columns of wider arrays whose rows are `ld` floats apart (one column tile).
template <int K, int kLd = 0>
int launch_sweep(const hpspmm_plan* p, const int32_t* rp, const float* v, const float* B, float* C, hipStream_t st,
                 uint32_t ld = K) {
  const bool bound = p->bound_val && p->bound_val == v && p->d_vval;
  constexpr int wpb = hpspmm::sweep_waves<K>();
  const dim3 grid((unsigned)(p->sw.n_waves / wpb));
  const size_t lds = hpspmm::sweep_lds_bytes<K>();
  if (bound)
    hipLaunchKernelGGL((hpspmm::spmm_sweep_kernel<K, false, kLd>), grid, dim3(wpb * 64), lds, st, p->sw, p->d_sw_base,
                       p->d_sw_len, p->d_sw_ends, p->d_vcol, p->d_vval, (const int32_t*)nullptr, p->d_sw_slot_row, B,
                       p->d_sw_zrow, p->d_partial, C, ld);
  else
    hipLaunchKernelGGL((hpspmm::spmm_sweep_kernel<K, true, kLd>), grid, dim3(wpb * 64), lds, st, p->sw, p->d_sw_base,
                       p->d_sw_len, p->d_sw_ends, p->d_vcol, v, p->d_vsrc, p->d_sw_slot_row, B, p->d_sw_zrow,
                       p->d_partial, C, ld);
  mark_launch(st, "spmm_sweep_kernel");
  const int64_t split_blocks = row_blocks(p->n_split, K);
  const int64_t fin_blocks = split_blocks + row_blocks(p->n_zero, K);
  if (fin_blocks > 0) {
    hipLaunchKernelGGL((hpspmm::spmm_sweep_final_kernel<K, kLd>), dim3((unsigned)fin_blocks), dim3(hpspmm::kBlock), 0, st,
                       rp, p->sw_limit, p->d_sw_split_rows, p->n_split, split_blocks, p->d_sw_part_base, p->d_zero_rows,
                       p->n_zero, p->d_partial, C, ld);
    mark_launch(st, "spmm_sweep_final_kernel");
  }
  return HPSPMM_OK;
}

}  // namespace

int sweep_prepare_kernels(int64_t k, int* per_cu) {
  return dispatch_k(k, [&](auto K) { return sweep_prepare_kernels_k<decltype(K)::value>(per_cu); });
}

int sweep_waves_for(int64_t k) {
  return dispatch_k(k, [](auto K) { return hpspmm::sweep_waves<decltype(K)::value>(); });
}

int launch_sweep_plan(const hpspmm_plan* p, const int32_t* rp, const float* v, const float* B, float* C,
                      hipStream_t st, int ld_mode, uint32_t ld) {
  return dispatch_k_ld(p->k, ld_mode, [&](auto K, auto L) {
    return launch_sweep<decltype(K)::value, decltype(L)::value>(p, rp, v, B, C, st, ld);
  });
}

int bind_values_sweep(hpspmm_plan* plan, const float* d_val, hipStream_t st) {
  if (!plan->d_vval) {
    if (hipMalloc(&plan->d_vval, (size_t)std::max<int64_t>(plan->sw_total, 1) * sizeof(float)) != hipSuccess) {
      (void)hipGetLastError();
      plan->d_vval = nullptr;
      return fail(HPSPMM_ERR_ALLOC, "device allocation for the bound values failed");
    }
    plan->workspace_bytes += plan->sw_total * (int64_t)sizeof(float);
  }
  hipLaunchKernelGGL(hpspmm::sweep_gather_values_kernel, dim3(grid_for(plan->sw_total, 1 << 16)), dim3(hpspmm::kBlock),
                     0, st, plan->sw_total, plan->d_vsrc, d_val, plan->d_vval);
  HPSPMM_HIP(hipGetLastError());
  return HPSPMM_OK;
}

}  // namespace hpspmm_host
