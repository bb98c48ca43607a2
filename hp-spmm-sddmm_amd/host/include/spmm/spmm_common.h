// Sparse containers, .smtx readers, row-length statistics and the result-file
// writer of the SpMM drivers.  Names and member meaning follow
// include/spmm/mm/spmm_common.h:58-164 of the reference so that its drivers'
// call sequences carry over; sizes handed back to the caller are 64-bit.
#pragma once

#include <cstdint>
#include <string>
#include <vector>

#include "starml/matrix.h"

using starml::Matrix;

// CSR container (reference: spmm_common.h:58-82): zero-based int32
// row_offsets_[rows+1] / column_indices_[nnz], float values_[nnz], each a 1-D Matrix.
class CSR_Matrix {
 public:
  int64_t num_rows_ = 0, num_cols_ = 0, num_nonzeros_ = 0;
  Matrix row_offsets_, column_indices_, values_;
  Matrix row_offsets() const { return row_offsets_; }
  Matrix column_indices() const { return column_indices_; }
  Matrix values() const { return values_; }
  int64_t num_rows() const { return num_rows_; }
  int64_t num_cols() const { return num_cols_; }
  int64_t num_nonzeros() const { return num_nonzeros_; }
};

// COO container (reference: spmm_common.h:84-108).  values_.size() may exceed the
// true nonzero count when the arrays are zero-padded.
class COO_Matrix {
 public:
  int64_t num_rows_ = 0, num_cols_ = 0, num_nonzeros_ = 0;
  Matrix row_indices_, column_indices_, values_;
  Matrix row_indices() const { return row_indices_; }
  Matrix column_indices() const { return column_indices_; }
  Matrix values() const { return values_; }
  int64_t num_rows() const { return num_rows_; }
  int64_t num_cols() const { return num_cols_; }
  int64_t num_nonzeros() const { return num_nonzeros_; }
};

// One result record = one CSV line (reference: spmm_common.h:111-141).  The
// vendor-library slots hold the rocSPARSE comparator here.
struct ResInfo {
  std::string filename_;
  float spmm_cs_csralg2_time_ = 0.f, spmm_cs_csralg2_throughput_ = 0.f;
  float spmm_cs_csralg3_time_ = 0.f, spmm_cs_csralg3_throughput_ = 0.f;
  float spmm_cs_csrdef_time_ = 0.f, spmm_cs_csrdef_throughput_ = 0.f;
  float spmm_cs_coo_time_ = 0.f, spmm_cs_coo_throughput_ = 0.f;
  float spmm_ge_time_ = 0.f, spmm_ge_throughput_ = 0.f;
  float spmm_hp_time_ = 0.f, spmm_hp_throughput_ = 0.f;
  int64_t num_rows_ = 0, num_cols_ = 0, num_nnz_ = 0, dense_dim_ = 0;
  double stdv = 0.0;
};

// GFLOPS = 2 * nnz * K / ms / 1e6 with the unpadded nnz (spmm_common.cpp:24-31);
// 0 when the time is 0 (method not run).
double spmm_gflops(int64_t nnz, int64_t k, double ms);
// Fills the *_throughput_ fields and appends one comma-separated line
// (spmm_common.cpp:22-44).
void write_info_to_file(const std::string& filename, ResInfo& info);

// .smtx text format (spmm_common.cpp:125-174): line 1 "rows,cols,nnz", line 2
// rows+1 row offsets, line 3 nnz column indices, whitespace separated.  Files
// carry no values: every value is 1.0 (spmm_common.cpp:154).
CSR_Matrix get_csr_mat_from_smtx(const std::string& filename, int64_t& num, int64_t& dim,
                                 int64_t& real_nonzero_num);
// Same file expanded to COO and zero-padded to a multiple of `padding`;
// num_nonzeros_ is the padded count (spmm_common.cpp:185-235).
COO_Matrix get_coo_mat_from_smtx(const std::string& filename, int64_t& num, int64_t& dim,
                                 int64_t& real_nonzero_num, int padding);
// COO with rows emitted in the order listed by the reorder file (one line of
// row ids); row ids stay the original ones, so C is not permuted, and
// num_nonzeros_ is the unpadded count (spmm_common.cpp:237-296).
COO_Matrix get_coo_mat_from_smtx_reorder(const std::string& filename, const std::string& reorder_filename,
                                         int64_t& num, int64_t& dim, int64_t& real_nonzero_num, int padding);
void write_smtx(const std::string& filename, const CSR_Matrix& host_csr);

// Host-side conversions used by the loaders, exposed for synthetic inputs.
COO_Matrix csr_to_coo(const CSR_Matrix& host_csr, int padding);
COO_Matrix csr_to_coo_reorder(const CSR_Matrix& host_csr, const std::vector<int32_t>& row_order, int padding);
int64_t roundUpToNextMultiple(int64_t num, int64_t multiple);

// Row-length statistics (population sigma and sigma/mean; spmm_common.cpp:300-321).
double calVarStdev(const std::vector<int>& v);
double calCV(const std::vector<int>& v);
double get_standard_CV(const std::string& filename);
double csr_row_length_cv(const CSR_Matrix& host_csr);

// Host <-> device moves of the three arrays (spmm_common.cpp:377-416).
CSR_Matrix csr_to_cuda(const CSR_Matrix& mat_cpu);
CSR_Matrix csr_to_host(const CSR_Matrix& mat_cuda);
COO_Matrix coo_to_cuda(const COO_Matrix& mat_cpu);
COO_Matrix coo_to_host(const COO_Matrix& mat_cuda);

// Dense row-major copy of a host CSR; a later duplicate overwrites an earlier
// one (spmm_common.cpp:417-449).  Small inputs only.
Matrix csrtodense_cpu(const CSR_Matrix& host_csr);

// A named synthetic benchmark graph ("c0_uniform" ... "c4_rmat") at the given
// scale, as a host CSR (the reference has no generators).
CSR_Matrix make_synthetic_csr(const std::string& name, double scale);
