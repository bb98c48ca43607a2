// Entry points of the C ABI (include/hpspmm.h) other than those about plans: one SpMM with a plan,
// without one, from the static workspace; COO accumulate; fill; the timing protocols.
#include "host.hpp"

#include <mutex>

using namespace hpspmm_host;

HPSPMM_API int hpspmm_version(void) { return 201; }

HPSPMM_API const char* hpspmm_last_error(void) { return last_error_message(); }

HPSPMM_API int hpspmm_get_device_info(hpspmm_device_info* out) {
  if (!out) return fail(HPSPMM_ERR_INVALID_ARG, "info_out is NULL");
  std::memset(out, 0, sizeof *out);
  int dev = 0;
  hipDeviceProp_t prop;
  HPSPMM_HIP(hipGetDevice(&dev));
  HPSPMM_HIP(hipGetDeviceProperties(&prop, dev));
  out->device = dev;
  out->compute_units = prop.multiProcessorCount;
  out->clock_khz = prop.clockRate;
  out->memory_clock_khz = prop.memoryClockRate;
  out->l2_bytes = prop.l2CacheSize;
  out->lds_bytes_per_cu = (int64_t)prop.maxSharedMemoryPerMultiProcessor;
  out->global_bytes = (int64_t)prop.totalGlobalMem;
  out->xcd_dealing = xcd_dealing_holds((hipStream_t) nullptr, -1) ? 1 : 0;
  std::snprintf(out->arch, sizeof out->arch, "%s", prop.gcnArchName);
  return HPSPMM_OK;
}

namespace {

// One SpMM through the plan's strategy, with operands of the form ld_mode (0: rows of B and C are
// plan->k floats; 1 / 2: one column tile of wider arrays, see row_length() in spmm_kernels.hpp).
int launch_strategy(const hpspmm_plan* plan, const int32_t* d_rowptr, const int32_t* d_col, const float* d_val,
                    const float* B, float* C, hipStream_t st, int ld_mode, uint32_t ld, bool values_ready) {
  switch (plan->strategy) {
    case HPSPMM_STRATEGY_ORDERED: return launch_ordered_plan(plan, d_rowptr, d_val, B, C, st, ld_mode, ld);
    case HPSPMM_STRATEGY_SWEEP: return launch_sweep_plan(plan, d_rowptr, d_val, B, C, st, ld_mode, ld);
    case HPSPMM_STRATEGY_ROUTED: return launch_routed_plan(plan, d_val, B, C, st, ld_mode, ld, values_ready);
    default: break;
  }
  if (ld_mode != 0) return fail(HPSPMM_ERR_INVALID_ARG, "plan of column tiles without a tiled strategy");
  if (plan->strategy == HPSPMM_STRATEGY_SEGMENTS) return launch_segments_plan(plan, d_rowptr, d_col, d_val, B, C, st);
  if (plan->d_tent) return launch_row_tiles_plan(plan, d_val, B, C, st);
  return launch_rows_any(plan->rows, plan->cols, plan->k, d_rowptr, d_col, d_val, B, C, plan->long_threshold,
                         plan->d_long_rows, plan->n_long, st);
}

}  // namespace

HPSPMM_API int hpspmm_csr_spmm(hpspmm_plan* plan, const int32_t* d_rowptr, const int32_t* d_col, const float* d_val,
                               const float* d_B, float* d_C, void* stream) {
  if (!plan) return fail(HPSPMM_ERR_INVALID_ARG, "plan is NULL");
  if (plan->rows == 0) return HPSPMM_OK;
  if (!d_rowptr || !d_C) return fail(HPSPMM_ERR_INVALID_ARG, "d_rowptr or d_C is NULL");
  if (plan->nnz > 0 && (!d_col || !d_val || !d_B))
    return fail(HPSPMM_ERR_INVALID_ARG, "d_col, d_val or d_B is NULL with nnz > 0");
  // The plan holds the structure of the arrays it was built from (some strategies run entirely
  // from its own copy): other addresses most likely mean another matrix, whose product would
  // silently be that of the old one.
  if (!plan->allow_moved && (d_rowptr != plan->src_rowptr || (plan->nnz > 0 && d_col != plan->src_col)))
    return fail(HPSPMM_ERR_INVALID_ARG,
                "d_rowptr / d_col are not the arrays this plan was built from (build a new plan for another "
                "structure, or create the plan with HPSPMM_PLAN_ALLOW_MOVED_CSR if the same structure has moved)");
  hipStream_t st = (hipStream_t)stream;
  int rc = HPSPMM_OK;
  // another value array overwrites the plan's copy of the bound one
  if (plan->bound_val && plan->bound_val != d_val) plan->bound_val = nullptr;
  if (plan->k_full != plan->k || plan->k_user != plan->k_full) {
    // one column tile after the other through the layout built for the tile width; the operands of
    // tile t are columns [t * k, (t + 1) * k) of B and C.  The rows of B are k_full floats apart -
    // the caller's B, or its padded copy when the caller's row length is not a multiple of 4 -,
    // those of C k_user floats.
    const float* Bsrc = d_B;
    if (plan->k_user != plan->k_full) {
      if ((rc = launch_pad_rows(plan->cols, plan->k_user, plan->k_full, d_B, plan->d_bpad, st))) return rc;
      Bsrc = plan->d_bpad;
    }
    const uint32_t shorter = (uint32_t)(plan->k_full - plan->k_user);  // 0 ... 3
    for (int t = 0; t < plan->tiles && rc == HPSPMM_OK; ++t) {
      const float* Bt = Bsrc + (int64_t)t * plan->k;
      float* Ct = d_C + (int64_t)t * plan->k;
      // the row length of B; how much shorter C's rows are; the columns of the tile that exist when
      // the last one is narrower than the layout
      const int64_t left = plan->k_user - (int64_t)t * plan->k;
      const uint32_t ld = (uint32_t)plan->k_full | shorter << 22 | (left < plan->k ? (uint32_t)left << 24 : 0u);
      // (shorter != 0: rows of C shorter than those of B, at any 4-byte alignment)
      rc = launch_strategy(plan, d_rowptr, d_col, d_val, Bt, Ct, st, shorter == 0 ? 1 : 2, ld, t > 0);
    }
  } else {
    rc = launch_strategy(plan, d_rowptr, d_col, d_val, d_B, d_C, st, 0, (uint32_t)plan->k, false);
  }
  if (rc) return rc;
  HPSPMM_HIP(hipGetLastError());
  return HPSPMM_OK;
}

HPSPMM_API int hpspmm_csr_spmm_noplan(int64_t rows, int64_t cols, int64_t nnz, const int32_t* d_rowptr,
                                      const int32_t* d_col, const float* d_val, const float* d_B, int64_t k,
                                      float* d_C, void* stream) {
  if (int rc = check_dims(rows, cols, nnz, k)) return rc;
  if (rows == 0) return HPSPMM_OK;
  if (!d_rowptr || !d_C) return fail(HPSPMM_ERR_INVALID_ARG, "d_rowptr or d_C is NULL");
  if (nnz > 0 && (!d_col || !d_val || !d_B))
    return fail(HPSPMM_ERR_INVALID_ARG, "d_col, d_val or d_B is NULL with nnz > 0");
  if (int rc = launch_rows_any(rows, cols, k, d_rowptr, d_col, d_val, d_B, d_C, INT32_MAX, nullptr, 0,
                               (hipStream_t)stream))
    return rc;
  HPSPMM_HIP(hipGetLastError());
  return HPSPMM_OK;
}

// ---------------------------------------------------------------------------------------------
// hpspmm_csr_spmm_static: the segments strategy without a plan and without any allocation.  What a
// plan would hold in its workspace lives in one file-scope device array: the row of every nonzero
// (kStaticMaxNnz int32) followed by the carry slots (kStaticCarryFloats floats).  Every device the
// library is loaded on holds its own copy of the array; its address there is looked up once per
// device (hipGetSymbolAddress) and only that pointer is ever handed to kernels.
// ---------------------------------------------------------------------------------------------
namespace {
constexpr int64_t kStaticMaxNnz = (int64_t)1 << 22;
constexpr int64_t kStaticCarryFloats = (int64_t)1 << 22;
constexpr size_t kStaticScratchBytes = (size_t)kStaticMaxNnz * sizeof(int32_t) + (size_t)kStaticCarryFloats * sizeof(float);
}  // namespace
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
namespace {
constexpr int kMaxDevices = 64;
std::mutex g_static_mutex;
void* g_static_ptr[kMaxDevices] = {nullptr};

// Device address of `scratch` on the current device (looked up on the first call per device).
int static_scratch(void** out) {
  int dev = 0;
  HPSPMM_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return fail(HPSPMM_ERR_INVALID_ARG, "device index %d not supported", dev);
  std::lock_guard<std::mutex> lock(g_static_mutex);
  if (!g_static_ptr[dev]) {
    void* ptr = nullptr;
    HPSPMM_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (!ptr) return fail(HPSPMM_ERR_HIP, "hipGetSymbolAddress returned a null address for the static workspace");
    g_static_ptr[dev] = ptr;
  }
  *out = g_static_ptr[dev];
  return HPSPMM_OK;
}
}  // namespace

HPSPMM_API int hpspmm_static_workspace_init(void) {
  void* base = nullptr;
  return static_scratch(&base);
}

HPSPMM_API int hpspmm_csr_spmm_static(int64_t rows, int64_t cols, int64_t nnz, const int32_t* d_rowptr,
                                      const int32_t* d_col, const float* d_val, const float* d_B, int64_t k,
                                      float* d_C, void* stream) {
  if (int rc = check_dims(rows, cols, nnz, k)) return rc;
  if (!fast_k(k)) return fail(HPSPMM_ERR_INVALID_ARG, "hpspmm_csr_spmm_static: k must be 32, 64 or 128, got %lld", (long long)k);
  if (nnz > kStaticMaxNnz)
    return fail(HPSPMM_ERR_INVALID_ARG,
                "hpspmm_csr_spmm_static: nnz = %lld exceeds the static workspace (at most %lld nonzeros); use a plan",
                (long long)nnz, (long long)kStaticMaxNnz);
  if (rows == 0) return HPSPMM_OK;
  if (!d_rowptr || !d_C) return fail(HPSPMM_ERR_INVALID_ARG, "d_rowptr or d_C is NULL");
  if (nnz > 0 && (!d_col || !d_val || !d_B))
    return fail(HPSPMM_ERR_INVALID_ARG, "d_col, d_val or d_B is NULL with nnz > 0");
  void* base = nullptr;
  if (int rc = static_scratch(&base)) return rc;
  int32_t* nnz_row = static_cast<int32_t*>(base);
  float* carry = reinterpret_cast<float*>(static_cast<unsigned char*>(base) + (size_t)kStaticMaxNnz * sizeof(int32_t));
  if (int rc = launch_segments_workspace(rows, nnz, k, d_rowptr, d_col, d_val, d_B, d_C, nnz_row, carry,
                                         kStaticCarryFloats, (hipStream_t)stream))
    return rc;
  HPSPMM_HIP(hipGetLastError());
  return HPSPMM_OK;
}

HPSPMM_API int hpspmm_coo_spmm_accumulate(int64_t rows, int64_t cols, int64_t nnz, const int32_t* d_row,
                                          const int32_t* d_col, const float* d_val, const float* d_B, int64_t k,
                                          float* d_C, void* stream) {
  if (int rc = check_dims(rows, cols, nnz, k)) return rc;
  if (nnz == 0) return HPSPMM_OK;
  if (rows == 0) return fail(HPSPMM_ERR_INVALID_ARG, "nnz > 0 with rows == 0");
  if (!d_row || !d_col || !d_val || !d_B || !d_C) return fail(HPSPMM_ERR_INVALID_ARG, "NULL device pointer");
  if (int rc = launch_coo_any(nnz, k, d_row, d_col, d_val, d_B, d_C, (hipStream_t)stream)) return rc;
  HPSPMM_HIP(hipGetLastError());
  return HPSPMM_OK;
}

HPSPMM_API int hpspmm_fill_f32(float* d_x, int64_t n, float value, void* stream) {
  if (n < 0) return fail(HPSPMM_ERR_INVALID_ARG, "negative length");
  if (n == 0) return HPSPMM_OK;
  if (!d_x) return fail(HPSPMM_ERR_INVALID_ARG, "d_x is NULL");
  hipLaunchKernelGGL(hpspmm::fill_f32_kernel, dim3(grid_for(n, 1 << 16)), dim3(hpspmm::kBlock), 0,
                     (hipStream_t)stream, d_x, n, value);
  HPSPMM_HIP(hipGetLastError());
  return HPSPMM_OK;
}

namespace {

// Mean milliseconds of `iters` back-to-back SpMMs between two events on the stream.
int time_region(hpspmm_plan* plan, const int32_t* d_rowptr, const int32_t* d_col, const float* d_val, const float* d_B,
                float* d_C, void* stream, int64_t iters, hipEvent_t t0, hipEvent_t t1, double* total_ms) {
  hipStream_t st = (hipStream_t)stream;
  int rc = HPSPMM_OK;
  hipError_t e = hipEventRecord(t0, st);
  for (int64_t i = 0; i < iters && rc == HPSPMM_OK && e == hipSuccess; ++i)
    rc = hpspmm_csr_spmm(plan, d_rowptr, d_col, d_val, d_B, d_C, stream);
  if (e == hipSuccess) e = hipEventRecord(t1, st);
  if (e == hipSuccess) e = hipEventSynchronize(t1);
  float ms = 0.f;
  if (e == hipSuccess && rc == HPSPMM_OK) e = hipEventElapsedTime(&ms, t0, t1);
  if (rc) return rc;
  if (e != hipSuccess) return fail(HPSPMM_ERR_HIP, "timing failed: %s", hipGetErrorString(e));
  *total_ms = ms;
  return HPSPMM_OK;
}

}  // namespace

HPSPMM_API int hpspmm_csr_spmm_timed_min(hpspmm_plan* plan, const int32_t* d_rowptr, const int32_t* d_col,
                                         const float* d_val, const float* d_B, float* d_C, void* stream, int warmup,
                                         int iters, float min_total_ms, float* mean_ms_out, int64_t* iters_done_out) {
  if (!mean_ms_out || iters <= 0 || warmup < 0 || !(min_total_ms >= 0.f))
    return fail(HPSPMM_ERR_INVALID_ARG, "bad timing arguments");
  for (int i = 0; i < warmup; ++i)
    if (int rc = hpspmm_csr_spmm(plan, d_rowptr, d_col, d_val, d_B, d_C, stream)) return rc;
  hipEvent_t t0, t1;
  HPSPMM_HIP(hipEventCreate(&t0));
  if (hipEventCreate(&t1) != hipSuccess) {
    (void)hipEventDestroy(t0);
    return fail(HPSPMM_ERR_HIP, "hipEventCreate failed");
  }
  double total = 0.0;
  int64_t done = iters;
  int rc = time_region(plan, d_rowptr, d_col, d_val, d_B, d_C, stream, done, t0, t1, &total);
  // A region shorter than min_total_ms says little (a 4 us SpMM timed over 20 launches is 80 us of
  // clock ramps and launch jitter): time a second region of as many launches as fill that time at
  // the rate just seen, and report that one.
  if (rc == HPSPMM_OK && total < (double)min_total_ms && total > 0.0) {
    const double per = total / (double)done;
    done = std::min<int64_t>((int64_t)1 << 20, std::max<int64_t>(iters, (int64_t)((double)min_total_ms / per) + 1));
    rc = time_region(plan, d_rowptr, d_col, d_val, d_B, d_C, stream, done, t0, t1, &total);
  }
  (void)hipEventDestroy(t0);
  (void)hipEventDestroy(t1);
  if (rc) return rc;
  *mean_ms_out = (float)(total / (double)done);
  if (iters_done_out) *iters_done_out = done;
  return HPSPMM_OK;
}

HPSPMM_API int hpspmm_csr_spmm_timed(hpspmm_plan* plan, const int32_t* d_rowptr, const int32_t* d_col,
                                     const float* d_val, const float* d_B, float* d_C, void* stream, int warmup,
                                     int iters, float* mean_ms_out) {
  return hpspmm_csr_spmm_timed_min(plan, d_rowptr, d_col, d_val, d_B, d_C, stream, warmup, iters, 0.f, mean_ms_out,
                                   nullptr);
}

HPSPMM_API int hpspmm_csr_spmm_timed_launches(hpspmm_plan* plan, const int32_t* d_rowptr, const int32_t* d_col,
                                              const float* d_val, const float* d_B, float* d_C, void* stream,
                                              int warmup, int iters, int max_launches, float* mean_ms_out,
                                              const char** names_out, int* n_launches_out) {
  if (!mean_ms_out || !names_out || !n_launches_out || iters <= 0 || warmup < 0 || max_launches <= 0)
    return fail(HPSPMM_ERR_INVALID_ARG, "bad timing arguments");
  *n_launches_out = 0;
  hipStream_t st = (hipStream_t)stream;
  for (int i = 0; i < warmup; ++i)
    if (int rc = hpspmm_csr_spmm(plan, d_rowptr, d_col, d_val, d_B, d_C, stream)) return rc;
  LaunchTrace trace;
  hipEvent_t begin = nullptr, end = nullptr;
  int created = 0;
  hipError_t e = hipEventCreate(&begin);
  if (e == hipSuccess) e = hipEventCreate(&end);
  for (; created < kMaxTracedLaunches && e == hipSuccess; ++created) e = hipEventCreate(&trace.ev[created]);
  auto destroy_events = [&]() {
    if (begin) (void)hipEventDestroy(begin);
    if (end) (void)hipEventDestroy(end);
    for (int q = 0; q < created - (e == hipSuccess ? 0 : 1); ++q) (void)hipEventDestroy(trace.ev[q]);
  };
  if (e != hipSuccess) {
    destroy_events();
    return fail(HPSPMM_ERR_HIP, "hipEventCreate: %s", hipGetErrorString(e));
  }
  // sum[q]: launch q; sum[kMaxTracedLaunches]: the launches beyond the trace's capacity, together
  double sum[kMaxTracedLaunches + 1] = {0};
  int rc = HPSPMM_OK, n = 0, seen = 0;
  for (int i = 0; i < iters && rc == HPSPMM_OK && e == hipSuccess; ++i) {
    trace.n = 0;
    trace.launches = 0;
    e = hipEventRecord(begin, st);
    set_launch_trace(&trace);
    rc = hpspmm_csr_spmm(plan, d_rowptr, d_col, d_val, d_B, d_C, stream);
    set_launch_trace(nullptr);
    if (rc != HPSPMM_OK || e != hipSuccess) break;
    n = trace.n;
    seen = trace.launches;
    if (n == 0) break;
    // the end event closes the iteration: nothing of it runs into the next one's first interval
    e = hipEventRecord(end, st);
    if (e == hipSuccess) e = hipEventSynchronize(end);
    for (int q = 0; q < n && e == hipSuccess; ++q) {
      float ms = 0.f;
      e = hipEventElapsedTime(&ms, q == 0 ? begin : trace.ev[q - 1], trace.ev[q]);
      sum[q] += ms;
    }
    if (seen > n && e == hipSuccess) {
      float ms = 0.f;
      e = hipEventElapsedTime(&ms, trace.ev[n - 1], end);
      sum[kMaxTracedLaunches] += ms;
    }
  }
  destroy_events();
  if (rc) return rc;
  if (e != hipSuccess) return fail(HPSPMM_ERR_HIP, "timing failed: %s", hipGetErrorString(e));
  // what does not fit the caller's arrays, or the trace, is reported as one last entry
  const bool overflow = seen > n || n > max_launches;
  const int own = overflow ? std::min(n, max_launches - 1) : n;
  for (int q = 0; q < own; ++q) {
    mean_ms_out[q] = (float)(sum[q] / iters);
    names_out[q] = trace.name[q];
  }
  int out = own;
  if (overflow) {
    double rest = sum[kMaxTracedLaunches];
    for (int q = own; q < n; ++q) rest += sum[q];
    mean_ms_out[out] = (float)(rest / iters);
    names_out[out] = "(remaining launches)";
    ++out;
  }
  *n_launches_out = out;
  return HPSPMM_OK;
}
