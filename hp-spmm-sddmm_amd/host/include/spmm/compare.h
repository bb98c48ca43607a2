// Result check of the SpMM drivers (spmm/utils/compare.cpp:2-28).
#pragma once

#include <string>

#include "starml/matrix.h"

// max_i |mat1[i] (/ EXE_NUM_CUDA when ktype == "div") - mat2[i]| over FP32
// matrices of equal size; both are brought to the host first.  Returns the
// maximum error and the flat index where it occurs.
float MaxAbsError(const starml::Matrix& mat1, const starml::Matrix& mat2, const std::string& ktype = "",
                  int64_t* pos = nullptr);
// Prints PASSed / Wrong and throws starml::Error when the error is not below
// 0.1 - the reference's acceptance bar (compare.cpp:21-27; it aborts there).
void ExpectEqualDenseWithError(const starml::Matrix& mat1, const starml::Matrix& mat2,
                               const std::string& ktype = "");
