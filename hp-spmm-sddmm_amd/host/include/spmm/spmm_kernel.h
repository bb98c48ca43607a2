// SpMM entry points of the host layer, with the signatures of
// include/spmm/mm/spmm_kernel.h:17-21 of the reference.  Operands live in device
// memory (Matrix on kHIP); `time` receives the mean milliseconds per launch over
// EXE_NUM_CUDA back-to-back launches (spmm/mm/spmm_kernel.cu:404-424).
#pragma once

#include <string>

#include "spmm/spmm_common.h"
#include "spmm/timer.h"

// A field of hpspmm_plan_options (by its name in include/hpspmm.h) for every plan GESpMM and HPSpMM
// build from here on; false if there is no such field.  Diagnostics and comparisons: no counterpart
// in the reference, whose launchers have no plan.
bool set_spmm_plan_option(const std::string& field, long value);

// C = A * B for CSR A.  Stands in for GESpMM (spmm_kernel.cu:389-426): same
// arguments, C overwritten.  Builds a plan (untimed, like the reference's host
// preprocessing), runs WARMUP_NUM_CUDA + EXE_NUM_CUDA launches, frees the plan.
void GESpMM(const CSR_Matrix& mat1, const Matrix& mat2, Matrix& result, float& time);
// The same operation under the name of this library's own method, with the
// values bound to the plan before the timed loop: the reference's HP-SpMM also
// lays its values out during preprocessing (spmm/mm/spmm_common.cpp:269-277),
// while GESpMM above is handed the CSR arrays as they are on every launch.
void HPSpMM(const CSR_Matrix& mat1, const Matrix& mat2, Matrix& result, float& time);
// C += A * B for COO A, EXE_NUM_CUDA launches without re-zeroing, i.e. C ends up
// as C0 + EXE_NUM_CUDA * A * B exactly like LBSpMM (spmm_kernel.cu:733-768).
void LBSpMM(const COO_Matrix& mat1, const Matrix& mat2, Matrix& result, float& time);
// Vendor comparator in the role of cusparseCSRSpMM (spmm_kernel.cu:36-151):
// rocSPARSE CSR SpMM, alpha = 1, beta = 0, row-major B and C.  algid as in the
// reference: 2, 3 or -1 (default).  Returns false (time = 0) when the library
// call is not available.
bool rocsparseCSRSpMM(const CSR_Matrix& mat1, const Matrix& mat2, Matrix& result, int algid, float& time);
// Vendor comparator in the role of cusparseCOOSpMM (spmm_kernel.cu:154-238): rocSPARSE COO SpMM
// (segmented algorithm), alpha = 1, beta = 0, row-major.  The COO arrays must hold the rows in
// ascending order (the plain loader's output, not the reordered one).
bool rocsparseCOOSpMM(const COO_Matrix& mat1, const Matrix& mat2, Matrix& result, float& time);
// x[i] = val on the device (spmm_kernel.cu:23-34).
void fill_matrix(starml::Matrix& a, float val);
