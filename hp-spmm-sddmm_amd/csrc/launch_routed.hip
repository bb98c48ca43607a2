// Routed strategy: the launches of one SpMM, and the values bound to a plan.
#include "host.hpp"

namespace hpspmm_host {

namespace {

// kLd: B and C are K columns of wider arrays whose rows are `ld` floats apart (one column tile);
// values_ready: an earlier tile of the same product has already brought the values into the plan's order.
template <int K, int kLd = 0>
int launch_routed(const hpspmm_plan* p, const float* v, const float* B, float* C, hipStream_t st, uint32_t ld = K,
                  bool values_ready = false) {
  // values bound to the plan are already in class-major order: only the hub rows of B are refreshed
  const bool bound = p->bound_val && p->bound_val == v;
  const bool inplace = p->d_vsrc && !(bound && p->d_vval);
  const int64_t permute_nnz = (p->d_vsrc || bound || values_ready) ? 0 : p->nnz;
  const int64_t gather_blocks = ceil_div(p->n_bhot * (K / 4), hpspmm::kBlock);
  const int64_t prep_blocks = gather_blocks + ceil_div(permute_nnz, hpspmm::kPermChunk);
  if (prep_blocks > INT32_MAX) return fail(HPSPMM_ERR_INVALID_ARG, "grid too large");
  if (prep_blocks > 0) {
    hipLaunchKernelGGL((hpspmm::routed_prepare_kernel<K, kLd>), dim3((unsigned)prep_blocks), dim3(hpspmm::kBlock), 0, st,
                       p->n_bhot, gather_blocks, p->d_bhot_src, B, p->d_bhot, p->nnz, p->lay.nhub + 1, v, p->d_lslot,
                       p->d_chunk_base, p->d_chunk_pref, p->d_vval, ld, p->lay.tile_width);
    mark_launch(st, "routed_prepare_kernel");
  }
  if (p->lay.tile_width > 0 && p->routed_grid > 0) {
    // Column-tile phases: one launch over all tiles; with routed_split_launch one per tile and part
    // (hub classes, cold class).
    if constexpr (kLd == 0) {
      const bool split = p->routed_split_launch;
      const int parts = split ? 2 * p->lay.tiles : 1;
      for (int part = 0; part < parts; ++part) {
        const int64_t tile0 = (int64_t)(part / 2) * p->lay.tile_grid;
        const int64_t first = !split ? 0 : part % 2 ? tile0 + p->lay.hub_grid : tile0;
        const int64_t last = !split ? p->routed_grid : part % 2 ? tile0 + p->lay.tile_grid : tile0 + p->lay.hub_grid;
        if (last <= first) continue;
        const dim3 grid((unsigned)(last - first));
        constexpr int WPB = hpspmm::kRoutedTileWaves;
        auto launch = [&](auto kernel, size_t lds) {
          hipLaunchKernelGGL(kernel, grid, dim3(WPB * 64), lds, st, p->lay, p->d_rvptr, p->d_coldptr, p->d_vcol,
                             p->d_vval, p->d_run_row, p->d_seg_run, p->d_zero_rows, B, p->d_bhot, p->d_partial,
                             p->d_carry, C, first, (uint32_t)K, p->n_bhot);
        };
        if (p->lay.tile_width == 32)
          launch(hpspmm::spmm_routed_tiles_kernel<32, WPB>, hpspmm::routed_tiles_lds_bytes<32, WPB>(p->lay.lds_rows));
        else
          launch(hpspmm::spmm_routed_tiles_kernel<64, WPB>, hpspmm::routed_tiles_lds_bytes<64, WPB>(p->lay.lds_rows));
        mark_launch(st, !split ? "spmm_routed_tiles_kernel" : part % 2 ? "spmm_routed_tiles_kernel(cold class)"
                                                                       : "spmm_routed_tiles_kernel(hub classes)");
      }
    } else {
      return fail(HPSPMM_ERR_INVALID_ARG, "a plan of column-tile phases serves whole rows only");
    }
  } else if (p->routed_grid > 0) {
    // One launch; a plan created with hpspmm_plan_options.routed_split_launch (diagnostics: per-class
    // times and counters) issues one per phase of the hub classes and one for the cold class, each
    // from its first workgroup on.
    const bool split = p->routed_split_launch;
    const int parts = split ? p->lay.nsub + 1 : 1;
    for (int part = 0; part < parts; ++part) {
      const int64_t first = split ? p->lay.phase_begin[part] : 0;
      const int64_t last = split ? (part < p->lay.nsub ? p->lay.phase_begin[part + 1] : p->routed_grid) : p->routed_grid;
      if (last <= first) continue;
      const dim3 grid((unsigned)(last - first));
      if (inplace)
        hipLaunchKernelGGL((hpspmm::spmm_routed_kernel<K, true, false, kLd>), grid, dim3(hpspmm::kBlock), 0, st, p->lay,
                           p->d_rvptr, p->d_coldptr, p->d_vcol, v, p->d_vsrc, p->d_vrow, B, p->d_bhot, p->d_partial,
                           p->d_carry, C, first, ld);
      else if (p->d_vsrc)  // column-range slices, values bound: the plan's own copy of them, still no compact buffer
        hipLaunchKernelGGL((hpspmm::spmm_routed_kernel<K, false, false, kLd>), grid, dim3(hpspmm::kBlock), 0, st, p->lay,
                           p->d_rvptr, p->d_coldptr, p->d_vcol, p->d_vval, (const int32_t*)nullptr, p->d_vrow, B,
                           p->d_bhot, p->d_partial, p->d_carry, C, first, ld);
      else
        hipLaunchKernelGGL((hpspmm::spmm_routed_kernel<K, false, true, kLd>), grid, dim3(hpspmm::kBlock), 0, st, p->lay,
                           p->d_rvptr, p->d_coldptr, p->d_vcol, p->d_vval, (const int32_t*)nullptr, p->d_vrow, B,
                           p->d_bhot, p->d_partial, p->d_carry, C, first, ld);
      mark_launch(st, !split ? "spmm_routed_kernel" : part < p->lay.nsub ? "spmm_routed_kernel(hub phase)"
                                                                          : "spmm_routed_kernel(cold class)");
    }
  }
  const int64_t routed_blocks = row_blocks(p->lay.n_routed, K);
  const int64_t cross_blocks = row_blocks(p->n_cross, K);
  // (under column-tile phases the main kernel has written the rows without nonzeros)
  const int64_t n_zero = p->lay.tile_width > 0 ? 0 : p->n_zero;
  const int64_t fin_blocks = routed_blocks + cross_blocks + row_blocks(n_zero, K);
  if (fin_blocks > 0) {
    hipLaunchKernelGGL((hpspmm::spmm_routed_final_kernel<K, kLd>), dim3((unsigned)fin_blocks), dim3(hpspmm::kBlock), 0, st,
                       p->lay, p->d_rvptr, p->d_coldptr, p->d_routed_rows, routed_blocks, p->d_cross_rows, p->n_cross,
                       cross_blocks, p->d_zero_rows, n_zero, p->d_partial, p->d_carry, C, ld);
    mark_launch(st, "spmm_routed_final_kernel");
  }
  return HPSPMM_OK;
}

}  // namespace

namespace {
// LDS one workgroup of the column-tile kernel may use at most (of the CU's 160 KB).
constexpr int kRoutedTilesLdsBudget = 152 << 10;
template <int W>
int routed_tiles_prepare_w(int* lds_rows) {
  constexpr int WPB = hpspmm::kRoutedTileWaves;
  const int rows = (int)((kRoutedTilesLdsBudget - hpspmm::routed_tiles_lds_bytes<W, WPB>(0)) / ((W + hpspmm::kTileLdsPad) * 4));
  HPSPMM_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&hpspmm::spmm_routed_tiles_kernel<W, WPB>),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, kRoutedTilesLdsBudget));
  *lds_rows = rows;
  return HPSPMM_OK;
}
}  // namespace

int routed_tiles_prepare(int tile_width, int* lds_rows) {
  return tile_width == 32 ? routed_tiles_prepare_w<32>(lds_rows) : routed_tiles_prepare_w<64>(lds_rows);
}

int launch_routed_plan(const hpspmm_plan* p, const float* v, const float* B, float* C, hipStream_t st, int ld_mode,
                       uint32_t ld, bool values_ready) {
  return dispatch_k_ld(p->k, ld_mode, [&](auto K, auto L) {
    return launch_routed<decltype(K)::value, decltype(L)::value>(p, v, B, C, st, ld, values_ready);
  });
}

int bind_values_routed(hpspmm_plan* plan, const float* d_val, hipStream_t st) {
  if (plan->d_vsrc) {
    // column-range slices: constant values are worth a copy in the plan's order after all (reading them
    // in place costs the main kernel what a bound plan no longer pays in re-ordering)
    const int64_t vtotal = plan->lay.cls_end[plan->lay.nhub];
    if (!plan->d_vval) {
      if (hipMalloc(&plan->d_vval, (size_t)std::max<int64_t>(vtotal, 1) * sizeof(float)) != hipSuccess) {
        (void)hipGetLastError();
        plan->d_vval = nullptr;
        return fail(HPSPMM_ERR_ALLOC, "device allocation for the bound values failed");
      }
      plan->workspace_bytes += vtotal * (int64_t)sizeof(float);
    }
    hipLaunchKernelGGL(hpspmm::routed_gather_values_kernel, dim3(grid_for(vtotal, 1 << 16)), dim3(hpspmm::kBlock), 0,
                       st, vtotal, plan->d_vsrc, d_val, plan->d_vval);
    HPSPMM_HIP(hipGetLastError());
  } else {
    // the value half of routed_prepare_kernel alone (its template argument only shapes the other half)
    const int64_t blocks = ceil_div(plan->nnz, hpspmm::kPermChunk);
    if (blocks > INT32_MAX) return fail(HPSPMM_ERR_INVALID_ARG, "grid too large");
    hipLaunchKernelGGL(hpspmm::routed_prepare_kernel<32>, dim3((unsigned)blocks), dim3(hpspmm::kBlock), 0, st,
                       (int64_t)0, (int64_t)0, (const int32_t*)nullptr, (const float*)nullptr, (float*)nullptr,
                       plan->nnz, plan->lay.nhub + 1, d_val, plan->d_lslot, plan->d_chunk_base, plan->d_chunk_pref,
                       plan->d_vval, 32u);
    HPSPMM_HIP(hipGetLastError());
  }
  return HPSPMM_OK;
}

}  // namespace hpspmm_host
