/*
 * CPU oracle for FP32 CSR SpMM  C = A * B.   TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker the GPU path is compared against.  Nothing that
 * ships (the HIP library, its C++ host layer, the Python binding) may link,
 * load or call it; only the test-suite, the smoke check and the CPU-baseline
 * leg of the benchmark do.
 *
 * The reference repository has no CPU SpMM of its own (its only CPU numeric
 * routine is the CSR->dense scatter, spmm/mm/spmm_common.cpp:417-449, and its
 * correctness check compares GPU kernels against cuSPARSE,
 * test/main.cpp:94-96).  The functions below therefore restate the *semantics*
 * the reference's CSR kernels and its cuSPARSE call define:
 *
 *   - alpha = 1, beta = 0, A not transposed, B and C dense row-major with
 *     leading dimension K, 32-bit zero-based indices
 *     (spmm/mm/spmm_kernel.cu:46-47, 82-108);
 *   - one output row per CSR row, nonzeros visited in stored order, one FP32
 *     multiply and one FP32 add per term, accumulator starts at 0
 *     (spmm/mm/spmm_kernel.cu:239-245, 338-346);
 *   - the COO entry point accumulates into C instead of overwriting it
 *     (spmm/mm/spmm_kernel.cu:463-476);
 *   - result comparison is max |x - y| over all elements, optionally with x
 *     divided by a launch count first (spmm/utils/compare.cpp:2-28);
 *   - row-length statistics are population sigma / mean
 *     (spmm/mm/spmm_common.cpp:311-321).
 *
 * Parity status of each function (what pins it, in tests/test_oracle.py):
 *   oracle_csr_spmm_f32      pinned: scipy float64 golden (tests/golden),
 *                            dense brute force, closed forms (identity,
 *                            permutation, all-ones values, row-normalised A
 *                            times ones, single hub row vs numpy sum).
 *   oracle_csr_spmm_f64      pinned: same checks at float64 tolerance; the
 *                            abs-sum output against numpy |A| @ |B|.
 *   oracle_coo_spmm_acc_f32  pinned: equals C0 + csr result on expanded COO,
 *                            brute force on tiny inputs, padded-tail no-op.
 *   oracle_csr_to_dense      pinned: against scipy .toarray() (no duplicates)
 *                            and the last-duplicate-wins rule by hand.
 *   oracle_max_abs_err       pinned: against numpy.
 *   oracle_row_length_cv     pinned: against numpy std/mean.
 *
 * Build: see oracle/Makefile (gcc -O2 -fopenmp -ffp-contract=off).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

int oracle_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* C[i, :] = sum_j val[j] * B[col[j], :] for j in [rowptr[i], rowptr[i+1]).
 * FP32 multiply then FP32 add, stored nnz order (spmm_kernel.cu:338-346).
 * Rows [row_begin, row_end) only; C is indexed by absolute row. */
void oracle_csr_spmm_f32_rows(int64_t row_begin, int64_t row_end, int64_t K,
                              const int32_t *rowptr, const int32_t *col,
                              const float *val, const float *B, float *C) {
#pragma omp parallel for schedule(dynamic, 64)
  for (int64_t i = row_begin; i < row_end; ++i) {
    float *c = C + (size_t)i * (size_t)K;
    for (int64_t k = 0; k < K; ++k) c[k] = 0.0f;
    for (int64_t j = rowptr[i]; j < rowptr[i + 1]; ++j) {
      const float a = val[j];
      const float *b = B + (size_t)col[j] * (size_t)K;
      for (int64_t k = 0; k < K; ++k) {
        const float p = a * b[k];
        c[k] = c[k] + p;
      }
    }
  }
}

void oracle_csr_spmm_f32(int64_t M, int64_t K, const int32_t *rowptr,
                         const int32_t *col, const float *val, const float *B,
                         float *C) {
  oracle_csr_spmm_f32_rows(0, M, K, rowptr, col, val, B, C);
}

/* Float64 accumulation of the same sum, plus S[i,k] = sum_j |a_ij| |b_jk|,
 * the denominator of the normalised error metric.  S may be NULL. */
void oracle_csr_spmm_f64_rows(int64_t row_begin, int64_t row_end, int64_t K,
                              const int32_t *rowptr, const int32_t *col,
                              const float *val, const float *B, double *C,
                              double *S) {
#pragma omp parallel for schedule(dynamic, 64)
  for (int64_t i = row_begin; i < row_end; ++i) {
    double *c = C + (size_t)i * (size_t)K;
    double *s = S ? S + (size_t)i * (size_t)K : NULL;
    for (int64_t k = 0; k < K; ++k) c[k] = 0.0;
    if (s)
      for (int64_t k = 0; k < K; ++k) s[k] = 0.0;
    for (int64_t j = rowptr[i]; j < rowptr[i + 1]; ++j) {
      const double a = (double)val[j];
      const float *b = B + (size_t)col[j] * (size_t)K;
      for (int64_t k = 0; k < K; ++k) {
        const double p = a * (double)b[k];
        c[k] += p;
        if (s) s[k] += fabs(p);
      }
    }
  }
}

void oracle_csr_spmm_f64(int64_t M, int64_t K, const int32_t *rowptr,
                         const int32_t *col, const float *val, const float *B,
                         double *C, double *S) {
  oracle_csr_spmm_f64_rows(0, M, K, rowptr, col, val, B, C, S);
}

/* COO SpMM that ACCUMULATES into C: C[row[j], :] += val[j] * B[col[j], :],
 * entries visited in stored order (spmm_kernel.cu:463-476).  Sequential on
 * purpose: entry order defines the FP32 result and rows may repeat anywhere. */
void oracle_coo_spmm_acc_f32(int64_t nnz, int64_t K, const int32_t *row,
                             const int32_t *col, const float *val,
                             const float *B, float *C) {
  for (int64_t j = 0; j < nnz; ++j) {
    const float a = val[j];
    const float *b = B + (size_t)col[j] * (size_t)K;
    float *c = C + (size_t)row[j] * (size_t)K;
    for (int64_t k = 0; k < K; ++k) {
      const float p = a * b[k];
      c[k] = c[k] + p;
    }
  }
}

/* CSR -> dense row-major scatter; a later duplicate overwrites an earlier one
 * (spmm_common.cpp:430-447). */
void oracle_csr_to_dense(int64_t M, int64_t N, const int32_t *rowptr,
                         const int32_t *col, const float *val, float *dense) {
#pragma omp parallel for
  for (int64_t i = 0; i < M; ++i)
    for (int64_t j = 0; j < N; ++j) dense[(size_t)i * (size_t)N + j] = 0.0f;
  for (int64_t i = 0; i < M; ++i)
    for (int64_t j = rowptr[i]; j < rowptr[i + 1]; ++j)
      dense[(size_t)i * (size_t)N + col[j]] = val[j];
}

/* max_i |x[i] / div - y[i]|  (compare.cpp:11-19; div = 1 for the plain form,
 * the launch count for the accumulate-then-divide form). */
float oracle_max_abs_err(int64_t n, const float *x, const float *y, float div) {
  float err_max = 0.0f;
  for (int64_t i = 0; i < n; ++i) {
    const float xi = (div == 1.0f) ? x[i] : x[i] / div;
    const float e = fabsf(xi - y[i]);
    if (e > err_max || e != e) err_max = e;
  }
  return err_max;
}

/* Normalised error of a FP32 result against the float64 oracle:
 *   max_ik |got - C64| / S   where S > 0, and, where S == 0, got must be
 * exactly 0 (returns +inf otherwise).  Also reports the arg-max position. */
double oracle_max_norm_err(int64_t n, const float *got, const double *C64,
                           const double *S, int64_t *argmax) {
  double worst = 0.0;
  int64_t pos = -1;
  for (int64_t i = 0; i < n; ++i) {
    double e;
    const double g = (double)got[i];
    if (S[i] > 0.0) {
      e = fabs(g - C64[i]) / S[i];
    } else {
      e = (g == 0.0) ? 0.0 : INFINITY;
    }
    if (!(e <= worst)) { /* also catches NaN */
      worst = (e != e) ? INFINITY : e;
      pos = i;
    }
  }
  if (argmax) *argmax = pos;
  return worst;
}

/* Coefficient of variation of row lengths, population sigma / mean
 * (spmm_common.cpp:311-321). */
double oracle_row_length_cv(int64_t M, const int32_t *rowptr) {
  if (M <= 0) return 0.0;
  double sum = 0.0;
  for (int64_t i = 0; i < M; ++i) sum += (double)(rowptr[i + 1] - rowptr[i]);
  const double mean = sum / (double)M;
  double acc = 0.0;
  for (int64_t i = 0; i < M; ++i) {
    const double d = (double)(rowptr[i + 1] - rowptr[i]) - mean;
    acc += d * d;
  }
  return sqrt(acc / (double)M) / mean;
}
