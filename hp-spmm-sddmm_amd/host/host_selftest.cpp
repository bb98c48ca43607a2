// CPU-only self-test of the host layer (no GPU call is made):
//   spmm_host_selftest <scratch-dir>
// Exercises the .smtx reader/writer, COO expansion with padding, the reorder
// loader, the row-length statistics, CSR->dense, the CSV writer and the host
// Matrix.  Exit status 0 = all checks passed.
#include <cmath>
#include <cstdio>
#include <fstream>
#include <iostream>
#include <sstream>
#include <string>
#include <vector>

#include "spmm/compare.h"
#include "spmm/spmm_common.h"

using namespace starml;

static int g_failed = 0;
#define CHECK(cond)                                                              \
  do {                                                                           \
    if (!(cond)) {                                                               \
      std::cerr << "FAILED " << __FILE__ << ":" << __LINE__ << ": " #cond "\n";  \
      ++g_failed;                                                                \
    }                                                                            \
  } while (0)

template <class F>
static bool throws(F f) {
  try {
    f();
  } catch (const Error&) {
    return true;
  }
  return false;
}

int main(int argc, char** argv) {
  if (argc != 2) {
    std::cerr << "usage: " << argv[0] << " <scratch-dir>\n";
    return 2;
  }
  const std::string dir = argv[1];

  // 4 x 5 matrix: rows of length 2, 0, 3, 1
  const std::string smtx = dir + "/tiny.smtx";
  {
    std::ofstream f(smtx);
    f << "4, 5,6\n0 2 2 5 6 \n0 3 1 2 4 0 \n";
  }
  int64_t num = -1, dim = -1, nnz = -1;
  CSR_Matrix a = get_csr_mat_from_smtx(smtx, num, dim, nnz);
  CHECK(num == 4 && dim == 5 && nnz == 6);
  CHECK(a.num_rows() == 4 && a.num_cols() == 5 && a.num_nonzeros() == 6);
  CHECK(a.row_offsets().size() == 5 && a.column_indices().size() == 6 && a.values().size() == 6);
  const int32_t want_rp[] = {0, 2, 2, 5, 6}, want_ci[] = {0, 3, 1, 2, 4, 0};
  for (int i = 0; i < 5; ++i) CHECK(a.row_offsets().data<int32_t>()[i] == want_rp[i]);
  for (int i = 0; i < 6; ++i) CHECK(a.column_indices().data<int32_t>()[i] == want_ci[i]);
  for (int i = 0; i < 6; ++i) CHECK(a.values().data<float>()[i] == 1.0f);  // files carry no values
  CHECK(throws([&] { (void)a.values().data<int32_t>(); }));                 // dtype is checked

  // COO expansion, zero padded to a multiple of 4; padded count reported
  COO_Matrix coo = get_coo_mat_from_smtx(smtx, num, dim, nnz, 4);
  CHECK(nnz == 6 && coo.num_nonzeros() == 8 && coo.values().size() == 8);
  const int32_t want_ri[] = {0, 0, 2, 2, 2, 3, 0, 0};
  for (int i = 0; i < 8; ++i) CHECK(coo.row_indices().data<int32_t>()[i] == want_ri[i]);
  CHECK(coo.values().data<float>()[5] == 1.0f && coo.values().data<float>()[6] == 0.0f &&
        coo.values().data<float>()[7] == 0.0f);
  CHECK(coo.column_indices().data<int32_t>()[6] == 0);
  CHECK(roundUpToNextMultiple(6, 4) == 8 && roundUpToNextMultiple(8, 4) == 8 && roundUpToNextMultiple(5, 0) == 5 &&
        roundUpToNextMultiple(0, 32) == 0);

  // reorder file: rows emitted in the listed order, ids kept, true count reported
  const std::string reorder = dir + "/tiny.reorder";
  {
    std::ofstream f(reorder);
    f << "2 3 1 0\n";
  }
  COO_Matrix cr = get_coo_mat_from_smtx_reorder(smtx, reorder, num, dim, nnz, 32);
  CHECK(cr.num_nonzeros() == 6 && cr.values().size() == 32);
  const int32_t want_rr[] = {2, 2, 2, 3, 0, 0}, want_cr[] = {1, 2, 4, 0, 0, 3};
  for (int i = 0; i < 6; ++i) {
    CHECK(cr.row_indices().data<int32_t>()[i] == want_rr[i]);
    CHECK(cr.column_indices().data<int32_t>()[i] == want_cr[i]);
  }
  {
    std::ofstream f(dir + "/bad.reorder");
    f << "2 2 1 0\n";
  }
  CHECK(throws([&] { get_coo_mat_from_smtx_reorder(smtx, dir + "/bad.reorder", num, dim, nnz, 32); }));

  // row-length statistics: lengths 2,0,3,1 -> mean 1.5, population sigma sqrt(1.25)
  CHECK(std::fabs(get_standard_CV(smtx) - std::sqrt(1.25) / 1.5) < 1e-12);
  CHECK(std::fabs(csr_row_length_cv(a) - std::sqrt(1.25) / 1.5) < 1e-12);
  CHECK(std::fabs(calVarStdev({2, 0, 3, 1}) - std::sqrt(1.25)) < 1e-12);

  // CSR -> dense, with a duplicate entry: the later one wins
  a.values().mutable_data<float>()[0] = 5.f;
  Matrix dense = csrtodense_cpu(a);
  CHECK(dense.dim(0) == 4 && dense.dim(1) == 5);
  const float* d = dense.data<float>();
  CHECK(d[0] == 5.f && d[3] == 1.f && d[1] == 0.f && d[5] == 0.f && d[2 * 5 + 4] == 1.f && d[3 * 5] == 1.f);
  CSR_Matrix dup = a;
  dup.column_indices_ = full({6}, Device(kCPU), kInt32, 0);  // every entry in column 0
  for (int i = 0; i < 6; ++i) dup.values().mutable_data<float>()[i] = (float)(i + 1);
  CHECK(csrtodense_cpu(dup).data<float>()[0] == 2.f && csrtodense_cpu(dup).data<float>()[2 * 5] == 5.f);

  // writer -> reader round trip on a generated graph
  CSR_Matrix g = make_synthetic_csr("c1_citation", 0.02);
  write_smtx(dir + "/gen.smtx", g);
  CSR_Matrix g2 = get_csr_mat_from_smtx(dir + "/gen.smtx", num, dim, nnz);
  CHECK(num == g.num_rows() && dim == g.num_cols() && nnz == g.num_nonzeros());
  bool same = true;
  for (int64_t i = 0; i <= num; ++i) same &= g.row_offsets().data<int32_t>()[i] == g2.row_offsets().data<int32_t>()[i];
  for (int64_t j = 0; j < nnz; ++j)
    same &= g.column_indices().data<int32_t>()[j] == g2.column_indices().data<int32_t>()[j];
  CHECK(same);
  CHECK(throws([&] { make_synthetic_csr("no_such_graph", 1.0); }));

  // malformed files are errors, not crashes
  {
    std::ofstream f(dir + "/short.smtx");
    f << "3,3,2\n0 1 2\n0 1\n";  // rows+1 offsets missing one
  }
  CHECK(throws([&] { get_csr_mat_from_smtx(dir + "/short.smtx", num, dim, nnz); }));
  {
    std::ofstream f(dir + "/range.smtx");
    f << "2,2,2\n0 1 2\n0 2\n";  // column 2 of 2
  }
  CHECK(throws([&] { get_csr_mat_from_smtx(dir + "/range.smtx", num, dim, nnz); }));
  CHECK(throws([&] { get_csr_mat_from_smtx(dir + "/missing.smtx", num, dim, nnz); }));

  // CSV line: GFLOPS = 2 nnz K / ms / 1e6, unpadded nnz, zero when not run
  ResInfo info;
  info.filename_ = "tiny.smtx";
  info.num_rows_ = 4;
  info.num_cols_ = 5;
  info.num_nnz_ = 1000000;
  info.dense_dim_ = 64;
  info.stdv = 0.5;
  info.spmm_ge_time_ = 2.0f;
  info.spmm_hp_time_ = 0.5f;
  const std::string csv = dir + "/res.csv";
  std::remove(csv.c_str());
  write_info_to_file(csv, info);
  write_info_to_file(csv, info);  // appends
  CHECK(std::fabs(info.spmm_ge_throughput_ - 64.0f) < 1e-3 && std::fabs(info.spmm_hp_throughput_ - 256.0f) < 1e-3);
  CHECK(info.spmm_cs_csralg2_throughput_ == 0.0f);
  CHECK(std::fabs(spmm_gflops(1000000, 64, 2.0) - 64.0) < 1e-9);
  std::ifstream in(csv);
  std::string line;
  int lines = 0;
  while (std::getline(in, line)) {
    ++lines;
    CHECK(line.rfind("tiny.smtx,4,5,1000000,64,0.5,cuSPARSE(CSR, ALG2): ,0,0,", 0) == 0);
    CHECK(line.find("GE-SpMM: ,2,64") != std::string::npos && line.find("HP-SpMM ,0.5,256") != std::string::npos);
    int commas = 0;
    for (char c : line) commas += c == ',';
    CHECK(commas == 5 + 6 * 3 + 3);  // three of the labels contain a comma themselves
  }
  CHECK(lines == 2);

  // host Matrix: shallow copies share storage, to(kCPU) is a deep copy, seeded rand
  Matrix m = full({3, 4}, Device(kCPU), kFloat, 2.5);
  Matrix alias = m;
  alias.mutable_data<float>()[5] = -1.f;
  CHECK(m.data<float>()[5] == -1.f && m.size() == 12 && m.dim(0) == 3 && m.dim(1) == 4 && m.ndims() == 2);
  Matrix deep = m.to(kCPU);
  deep.mutable_data<float>()[5] = 9.f;
  CHECK(m.data<float>()[5] == -1.f);
  set_rand_seed(7);
  Matrix r1 = rand({1000}, Device(kCPU), kFloat, -1.0, 1.0);
  set_rand_seed(7);
  Matrix r2 = rand({1000}, Device(kCPU), kFloat, -1.0, 1.0);
  bool eq = true, in_range = true;
  for (int i = 0; i < 1000; ++i) {
    eq &= r1.data<float>()[i] == r2.data<float>()[i];
    in_range &= r1.data<float>()[i] >= -1.f && r1.data<float>()[i] < 1.f;
  }
  CHECK(eq && in_range);
  CHECK(throws([&] { Matrix bad({-1}, Device(kCPU), kFloat); }));

  // result check: a NaN anywhere (not only in the last position) fails it, on either side
  {
    Matrix x = full({8}, Device(kCPU), kFloat, 1.0), y = full({8}, Device(kCPU), kFloat, 1.0);
    int64_t at = -1;
    CHECK(MaxAbsError(x, y, "", &at) == 0.f && at == -1);
    y.mutable_data<float>()[6] = 1.05f;
    CHECK(std::fabs(MaxAbsError(x, y, "", &at) - 0.05f) < 1e-6f && at == 6);
    x.mutable_data<float>()[3] = NAN;  // followed by finite, smaller errors
    CHECK(std::isinf(MaxAbsError(x, y, "", &at)) && at == 3);
    CHECK(throws([&] { ExpectEqualDenseWithError(x, y); }));
    x.mutable_data<float>()[3] = 1.0f;
    y.mutable_data<float>()[0] = NAN;
    CHECK(std::isinf(MaxAbsError(x, y, "", &at)) && at == 0);
    Matrix z = full({8}, Device(kCPU), kFloat, 200.0), w = full({8}, Device(kCPU), kFloat, 1.0);
    CHECK(MaxAbsError(z, w, "div", &at) == 0.f);  // "div": x / 200 launches against y
  }

  if (g_failed) {
    std::cerr << g_failed << " check(s) failed\n";
    return 1;
  }
  std::cout << "host selftest OK\n";
  return 0;
}
