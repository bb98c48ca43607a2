#include "spmm/spmm_kernel.h"

#include <hip/hip_runtime_api.h>
#include <rocsparse/rocsparse.h>

#include <cstddef>
#include <cstring>
#include <iostream>

#include "hpspmm.h"

using starml::Error;

namespace {

struct Dims {
  int64_t m, n, k, nnz;
};

// Operand checks the reference leaves to its dtype assertions and to luck:
// shapes must agree and everything must already be in device memory.
Dims check_operands(int64_t rows, int64_t cols, const Matrix& idx_a, const Matrix& idx_b, const Matrix& values,
                    const Matrix& mat2, const Matrix& result, const char* who) {
  if (mat2.ndims() != 2 || result.ndims() != 2) throw Error(std::string(who) + ": B and C must be 2-D");
  Dims d{rows, cols, mat2.dim(1), values.size()};
  if (mat2.dim(0) != cols) throw Error(std::string(who) + ": B must have num_cols rows");
  if (result.dim(0) != rows || result.dim(1) != d.k) throw Error(std::string(who) + ": C must be num_rows x K");
  for (const Matrix* m : {&idx_a, &idx_b, &values, &mat2, &result})
    if (!m->is_cuda()) throw Error(std::string(who) + ": operands must be in device memory");
  return d;
}

// Plan options of GESpMM / HPSpMM (set_spmm_plan_option); all zero = the library's own choices.
hpspmm_plan_options g_plan_options{};
bool g_have_plan_options = false;

void check_status(int rc, const char* who) {
  if (rc != HPSPMM_OK) throw Error(std::string(who) + ": " + hpspmm_last_error());
}

void csr_spmm_timed(const CSR_Matrix& a, const Matrix& mat2, Matrix& result, float& time, const char* who,
                    bool bind_values) {
  const Matrix rp = a.row_offsets(), ci = a.column_indices(), va = a.values();
  if (rp.size() != a.num_rows() + 1) throw Error(std::string(who) + ": row_offsets must have num_rows + 1 entries");
  const Dims d = check_operands(a.num_rows(), a.num_cols(), rp, ci, va, mat2, result, who);
  hpspmm_plan* plan = nullptr;
  if (g_have_plan_options) {
    g_plan_options.struct_size = sizeof(hpspmm_plan_options);
    check_status(hpspmm_plan_create_ex(d.m, d.n, d.nnz, rp.data<int32_t>(), ci.data<int32_t>(), d.k, &g_plan_options,
                                       nullptr, &plan),
                 who);
  } else {
    check_status(hpspmm_plan_create(d.m, d.n, d.nnz, rp.data<int32_t>(), ci.data<int32_t>(), d.k, HPSPMM_PLAN_DEFAULT,
                                    nullptr, &plan),
                 who);
  }
  if (bind_values) {
    const int rb = hpspmm_plan_bind_values(plan, va.data<float>(), nullptr);
    if (rb != HPSPMM_OK) {
      hpspmm_plan_destroy(plan);
      check_status(rb, who);
    }
  }
  const int rc = hpspmm_csr_spmm_timed(plan, rp.data<int32_t>(), ci.data<int32_t>(), va.data<float>(),
                                       mat2.data<float>(), result.mutable_data<float>(), nullptr, WARMUP_NUM_CUDA,
                                       EXE_NUM_CUDA, &time);
  hpspmm_plan_destroy(plan);
  check_status(rc, who);
  std::cout << who << " time: " << time << " ms " << std::endl;
}

}  // namespace

bool set_spmm_plan_option(const std::string& field, long value) {
  struct Field {
    const char* name;
    size_t offset;
    bool is_unsigned;
  };
#define HPSPMM_OPTION(f) {#f, offsetof(hpspmm_plan_options, f), false}
  static const Field fields[] = {
      {"flags", offsetof(hpspmm_plan_options, flags), true},
      HPSPMM_OPTION(segment_shift), HPSPMM_OPTION(hub_log2), HPSPMM_OPTION(routed_row_log2),
      HPSPMM_OPTION(routed_phases), HPSPMM_OPTION(routed_tile_width), HPSPMM_OPTION(routed_split_launch),
      HPSPMM_OPTION(routed_lds_rows), HPSPMM_OPTION(xcd_dealing), HPSPMM_OPTION(no_column_tiles),
      HPSPMM_OPTION(row_tiles_min_k), HPSPMM_OPTION(row_tiles_pad), HPSPMM_OPTION(row_tiles_wide),
      HPSPMM_OPTION(row_tiles_round_robin), HPSPMM_OPTION(sweep_window_log2), HPSPMM_OPTION(sweep_lead),
      HPSPMM_OPTION(sweep_spin), HPSPMM_OPTION(sweep_limit), HPSPMM_OPTION(sweep_no_priorities),
      HPSPMM_OPTION(cluster_sweeps), HPSPMM_OPTION(report), HPSPMM_OPTION(row_tiles_chunk_log2)};
#undef HPSPMM_OPTION
  for (const Field& f : fields) {
    if (field != f.name) continue;
    char* at = reinterpret_cast<char*>(&g_plan_options) + f.offset;
    if (f.is_unsigned) {
      const uint32_t v = (uint32_t)value;
      std::memcpy(at, &v, sizeof v);
    } else {
      const int32_t v = (int32_t)value;
      std::memcpy(at, &v, sizeof v);
    }
    g_have_plan_options = true;
    return true;
  }
  return false;
}

void GESpMM(const CSR_Matrix& mat1, const Matrix& mat2, Matrix& result, float& time) {
  csr_spmm_timed(mat1, mat2, result, time, "GESpMM", false);
}

void HPSpMM(const CSR_Matrix& mat1, const Matrix& mat2, Matrix& result, float& time) {
  csr_spmm_timed(mat1, mat2, result, time, "HPSpMM", true);
}

void LBSpMM(const COO_Matrix& mat1, const Matrix& mat2, Matrix& result, float& time) {
  const Matrix ri = mat1.row_indices(), ci = mat1.column_indices(), va = mat1.values();
  if (ri.size() != va.size() || ci.size() != va.size()) throw Error("LBSpMM: COO arrays differ in length");
  const Dims d = check_operands(mat1.num_rows(), mat1.num_cols(), ri, ci, va, mat2, result, "LBSpMM");
  GpuTimer timer;
  timer.Start();
  for (int i = 0; i < EXE_NUM_CUDA; ++i)
    check_status(hpspmm_coo_spmm_accumulate(d.m, d.n, d.nnz, ri.data<int32_t>(), ci.data<int32_t>(), va.data<float>(),
                                            mat2.data<float>(), d.k, result.mutable_data<float>(), nullptr),
                 "LBSpMM");
  timer.Stop();
  time = timer.Elapsed() / EXE_NUM_CUDA;
  std::cout << "LBSpMM time: " << time << " ms " << std::endl;
}

void fill_matrix(starml::Matrix& a, float val) {
  if (!a.is_cuda()) throw Error("fill_matrix: matrix must be in device memory");
  check_status(hpspmm_fill_f32(a.mutable_data<float>(), a.size(), val, nullptr), "fill_matrix");
}

namespace {

// Shared body of the two vendor comparators: descriptors for B and C, buffer,
// preprocess, WARMUP_NUM_CUDA + EXE_NUM_CUDA timed compute calls.
bool rocsparse_spmm_timed(rocsparse_spmat_descr A, const Dims& d, const Matrix& mat2, Matrix& result,
                          rocsparse_spmm_alg alg, rocsparse_handle handle, float& time) {
  rocsparse_dnmat_descr B = nullptr, C = nullptr;
  void* buffer = nullptr;
  bool ok = rocsparse_create_dnmat_descr(&B, d.n, d.k, d.k, mat2.raw_mutable_data(), rocsparse_datatype_f32_r,
                                         rocsparse_order_row) == rocsparse_status_success;
  ok = ok && rocsparse_create_dnmat_descr(&C, d.m, d.k, d.k, result.raw_mutable_data(), rocsparse_datatype_f32_r,
                                          rocsparse_order_row) == rocsparse_status_success;
  const float alpha = 1.0f, beta = 0.0f;
  size_t bytes = 0;
  auto stage = [&](rocsparse_spmm_stage s) {
    return rocsparse_spmm(handle, rocsparse_operation_none, rocsparse_operation_none, &alpha, A, B, &beta, C,
                          rocsparse_datatype_f32_r, alg, s, &bytes, buffer) == rocsparse_status_success;
  };
  ok = ok && stage(rocsparse_spmm_stage_buffer_size);
  ok = ok && hipMalloc(&buffer, bytes ? bytes : 4) == hipSuccess;
  ok = ok && stage(rocsparse_spmm_stage_preprocess);
  if (ok) {
    for (int i = 0; i < WARMUP_NUM_CUDA && ok; ++i) ok = stage(rocsparse_spmm_stage_compute);
    GpuTimer timer;
    timer.Start();
    for (int i = 0; i < EXE_NUM_CUDA && ok; ++i) ok = stage(rocsparse_spmm_stage_compute);
    timer.Stop();
    time = ok ? timer.Elapsed() / EXE_NUM_CUDA : 0.f;
  }
  if (buffer) (void)hipFree(buffer);
  if (C) rocsparse_destroy_dnmat_descr(C);
  if (B) rocsparse_destroy_dnmat_descr(B);
  return ok;
}

}  // namespace

bool rocsparseCSRSpMM(const CSR_Matrix& mat1, const Matrix& mat2, Matrix& result, int algid, float& time) {
  time = 0.f;
  const Matrix rp = mat1.row_offsets(), ci = mat1.column_indices(), va = mat1.values();
  const Dims d = check_operands(mat1.num_rows(), mat1.num_cols(), rp, ci, va, mat2, result, "rocsparseCSRSpMM");
  rocsparse_spmm_alg alg = rocsparse_spmm_alg_default;
  if (algid == 2) alg = rocsparse_spmm_alg_csr_row_split;
  if (algid == 3) alg = rocsparse_spmm_alg_csr_nnz_split;
  if (algid == 4) alg = rocsparse_spmm_alg_csr_merge_path;
  rocsparse_handle handle = nullptr;
  rocsparse_spmat_descr A = nullptr;
  bool ok = rocsparse_create_handle(&handle) == rocsparse_status_success;
  ok = ok && rocsparse_create_csr_descr(&A, d.m, d.n, d.nnz, rp.raw_mutable_data(), ci.raw_mutable_data(),
                                        va.raw_mutable_data(), rocsparse_indextype_i32, rocsparse_indextype_i32,
                                        rocsparse_index_base_zero, rocsparse_datatype_f32_r) == rocsparse_status_success;
  ok = ok && rocsparse_spmm_timed(A, d, mat2, result, alg, handle, time);
  if (A) rocsparse_destroy_spmat_descr(A);
  if (handle) rocsparse_destroy_handle(handle);
  if (ok) std::cout << "rocSPARSE CSR SpMM (alg " << algid << ") time: " << time << " ms " << std::endl;
  return ok;
}

bool rocsparseCOOSpMM(const COO_Matrix& mat1, const Matrix& mat2, Matrix& result, float& time) {
  time = 0.f;
  const Matrix ri = mat1.row_indices(), ci = mat1.column_indices(), va = mat1.values();
  const Dims d = check_operands(mat1.num_rows(), mat1.num_cols(), ri, ci, va, mat2, result, "rocsparseCOOSpMM");
  rocsparse_handle handle = nullptr;
  rocsparse_spmat_descr A = nullptr;
  bool ok = rocsparse_create_handle(&handle) == rocsparse_status_success;
  ok = ok && rocsparse_create_coo_descr(&A, d.m, d.n, d.nnz, ri.raw_mutable_data(), ci.raw_mutable_data(),
                                        va.raw_mutable_data(), rocsparse_indextype_i32, rocsparse_index_base_zero,
                                        rocsparse_datatype_f32_r) == rocsparse_status_success;
  ok = ok && rocsparse_spmm_timed(A, d, mat2, result, rocsparse_spmm_alg_coo_segmented, handle, time);
  if (A) rocsparse_destroy_spmat_descr(A);
  if (handle) rocsparse_destroy_handle(handle);
  if (ok) std::cout << "rocSPARSE COO SpMM time: " << time << " ms " << std::endl;
  return ok;
}
