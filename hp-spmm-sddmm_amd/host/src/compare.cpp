#include "spmm/compare.h"

#include <cmath>
#include <iostream>

#include "spmm/timer.h"

using starml::Error;
using starml::Matrix;

float MaxAbsError(const Matrix& mat1, const Matrix& mat2, const std::string& ktype, int64_t* pos_out) {
  if (mat1.size() != mat2.size()) throw Error("compare: sizes differ");
  if (!(mat1.data_type() == mat2.data_type())) throw Error("compare: data types differ");
  if (mat1.ndims() != mat2.ndims()) throw Error("compare: ranks differ");
  const Matrix a = mat1.to(starml::kCPU), b = mat2.to(starml::kCPU);
  const float* x = a.data<float>();
  const float* y = b.data<float>();
  const float div = ktype == "div" ? (float)EXE_NUM_CUDA : 1.0f;
  float worst = 0.f;
  int64_t pos = -1;
  for (int64_t i = 0; i < a.size(); ++i) {
    const float e = std::fabs((div == 1.0f ? x[i] : x[i] / div) - y[i]);
    if (e != e) {  // a NaN on either side is the worst possible error and ends the search
      worst = INFINITY;
      pos = i;
      break;
    }
    if (e > worst) {
      worst = e;
      pos = i;
    }
  }
  if (pos_out) *pos_out = pos;
  return worst;
}

void ExpectEqualDenseWithError(const Matrix& mat1, const Matrix& mat2, const std::string& ktype) {
  int64_t pos = -1;
  const float err = MaxAbsError(mat1, mat2, ktype, &pos);
  const bool passed = err < 0.1f;
  if (passed)
    std::cout << "PASSed!! max_err = " << err << " < 0.1 " << std::endl;
  else
    std::cout << "Wrong!! max_err = " << err << " > 0.1 at pos: " << pos << std::endl;
  if (!passed) throw Error("ExpectEqualDenseWithError: results differ");
}
