// Command-line driver with the argv of the reference's test/test_all.cpp:27-109:
//
//   spmm_test_all <graph.smtx> <graph.reorder | -> <K> [--check] [--csv file] [--dump-c prefix]
//   spmm_test_all --synthetic <name> <scale> <K> [--check] [--csv file] [--dump-c prefix]
//   (either form: [--vendor-algs 2,3,-1,coo] [--plan-option FIELD=VALUE]..., a field of
//   hpspmm_plan_options for the plans of GESpMM and HPSpMM, for comparisons)
//
// It loads (or generates) the graph, moves it to the GPU, times the vendor
// comparator (rocSPARSE, in the slots the reference gives cuSPARSE), the CSR
// entry point and the COO accumulate entry point, optionally checks each
// against the comparator with the reference's 0.1 absolute bar, and appends one
// line in the reference's CSV format.  --check without a comparator result is an
// error (exit status 3), not a silent pass.  --dump-c writes the dense operand
// and the three results as raw little-endian FP32 files (prefix.B.f32,
// prefix.gespmm.f32, prefix.lbspmm.f32 - the accumulated sum of EXE_NUM_CUDA
// launches -, prefix.hpspmm.f32) for a checker outside this program.
// --vendor-algs takes a comma list out of 2,3,-1,coo (default: all four, the
// reference's set) for runs that only need one comparator result.
#include <hip/hip_runtime_api.h>

#include <cstring>
#include <fstream>
#include <iostream>
#include <numeric>
#include <string>
#include <vector>

#include "spmm/compare.h"
#include "spmm/spmm_common.h"
#include "spmm/spmm_kernel.h"

using namespace starml;

static void dump_f32(const std::string& path, const Matrix& m) {
  const Matrix h = m.to(kCPU);
  std::ofstream f(path, std::ios::binary);
  f.write(reinterpret_cast<const char*>(h.data<float>()), (std::streamsize)h.nbytes());
  if (!f) throw Error("cannot write " + path);
}

int main(int argc, char** argv) {
  try {
    std::vector<std::string> pos;
    bool check = false, synthetic = false;
    std::string csv, dump, vendor = "2,3,-1,coo";
    for (int i = 1; i < argc; ++i) {
      const std::string a = argv[i];
      if (a == "--check") check = true;
      else if (a == "--synthetic") synthetic = true;
      else if (a == "--csv" && i + 1 < argc) csv = argv[++i];
      else if (a == "--plan-option" && i + 1 < argc) {
        const std::string kv = argv[++i];
        const size_t eq = kv.find('=');
        if (eq == std::string::npos || !set_spmm_plan_option(kv.substr(0, eq), std::stol(kv.substr(eq + 1)))) {
          std::cerr << "error: --plan-option wants FIELD=VALUE with a field of hpspmm_plan_options, got '" << kv << "'\n";
          return 2;
        }
      }
      else if (a == "--dump-c" && i + 1 < argc) dump = argv[++i];
      else if (a == "--vendor-algs" && i + 1 < argc) vendor = argv[++i];
      else pos.push_back(a);
    }
    if (pos.size() != 3) {
      std::cerr << "usage: " << argv[0] << " <graph.smtx> <graph.reorder|-> <K> [--check] [--csv file] [--dump-c prefix] [--vendor-algs 2,3,-1,coo] [--plan-option FIELD=VALUE]\n"
                << "       " << argv[0] << " --synthetic <name> <scale> <K> [--check] [--csv file] [--dump-c prefix]\n";
      return 2;
    }
    const int64_t k = std::stoll(pos[2]);
    ResInfo info;
    int64_t num = 0, dim = 0, nnz = 0;
    CSR_Matrix h_csr;
    COO_Matrix h_coo_reorder, h_coo;
    // default result file: that of the reference driver whose input this is - test/main.cpp:112 without
    // a reorder file, test/test_all.cpp:108 with one
    if (csv.empty()) csv = !synthetic && pos[1] == "-" ? "./full_graph_res.csv" : "./full_graph_res_reorder.csv";
    if (synthetic) {
      info.filename_ = pos[0] + "@" + pos[1];
      h_csr = make_synthetic_csr(pos[0], std::stod(pos[1]));
      num = h_csr.num_rows();
      dim = h_csr.num_cols();
      nnz = h_csr.num_nonzeros();
      info.stdv = csr_row_length_cv(h_csr);
      std::vector<int32_t> order((size_t)num);
      std::iota(order.begin(), order.end(), 0);
      h_coo_reorder = csr_to_coo_reorder(h_csr, order, 32);
      h_coo = csr_to_coo(h_csr, 1);
    } else {
      info.filename_ = pos[0];
      info.stdv = get_standard_CV(pos[0]);
      h_csr = get_csr_mat_from_smtx(pos[0], num, dim, nnz);
      h_coo = get_coo_mat_from_smtx(pos[0], num, dim, nnz, 1);  // unpadded: the vendor routine wants sorted rows
      h_coo_reorder = pos[1] == "-" ? get_coo_mat_from_smtx(pos[0], num, dim, nnz, 32)
                                    : get_coo_mat_from_smtx_reorder(pos[0], pos[1], num, dim, nnz, 32);
    }
    std::cout << "row_num: " << num << "\ncol_num: " << dim << "\nk: " << k << "\nnonzero_num: " << nnz
              << "\nrow length stdv: " << info.stdv << "\ndensity: " << (double)nnz / ((double)num * (double)dim) << '\n';
    info.num_rows_ = num;
    info.num_cols_ = dim;
    info.dense_dim_ = k;
    info.num_nnz_ = nnz;

    Matrix d_B = rand({dim, k}, Device(kCPU), DataType(kFloat), -1.0, 1.0).to(kHIP);
    CSR_Matrix d_csr = csr_to_cuda(h_csr);
    COO_Matrix d_coo = coo_to_cuda(h_coo_reorder);
    Matrix d_ref = full({num, k}, Device(kHIP), DataType(kFloat), 0.0);
    Matrix d_csr_out = full({num, k}, Device(kHIP), DataType(kFloat), 0.0);
    Matrix d_coo_out = full({num, k}, Device(kHIP), DataType(kFloat), 0.0);

    auto wanted = [&](const std::string& alg) { return ("," + vendor + ",").find("," + alg + ",") != std::string::npos; };
    bool have_ref = false;
    if (wanted("2")) have_ref = rocsparseCSRSpMM(d_csr, d_B, d_ref, 2, info.spmm_cs_csralg2_time_) || have_ref;
    if (wanted("3")) have_ref = rocsparseCSRSpMM(d_csr, d_B, d_ref, 3, info.spmm_cs_csralg3_time_) || have_ref;
    if (wanted("-1")) have_ref = rocsparseCSRSpMM(d_csr, d_B, d_ref, -1, info.spmm_cs_csrdef_time_) || have_ref;
    if (wanted("coo")) {
      // vendor COO baseline on the row-ordered, unpadded COO
      COO_Matrix d_coo_plain = coo_to_cuda(h_coo);
      Matrix d_tmp = full({num, k}, Device(kHIP), DataType(kFloat), 0.0);
      rocsparseCOOSpMM(d_coo_plain, d_B, d_tmp, info.spmm_cs_coo_time_);
    }
    (void)hipDeviceSynchronize();
    if (check && !have_ref) {
      std::cerr << "error: --check asked for, but the rocSPARSE comparator produced no result" << std::endl;
      return 3;
    }
    if (!dump.empty()) dump_f32(dump + ".B.f32", d_B);

    fill_matrix(d_csr_out, 0.0f);
    GESpMM(d_csr, d_B, d_csr_out, info.spmm_ge_time_);
    if (check) ExpectEqualDenseWithError(d_csr_out, d_ref);
    if (!dump.empty()) dump_f32(dump + ".gespmm.f32", d_csr_out);

    fill_matrix(d_coo_out, 0.0f);
    LBSpMM(d_coo, d_B, d_coo_out, info.spmm_hp_time_);
    if (check) ExpectEqualDenseWithError(d_coo_out, d_ref, "div");
    if (!dump.empty()) dump_f32(dump + ".lbspmm.f32", d_coo_out);

    // this library's own method: the CSR path with the values bound before the timed loop.
    // It takes the HP slot of the result line when it is faster than the COO accumulate form.
    float hp_csr_time = 0.f;
    fill_matrix(d_csr_out, 0.0f);
    HPSpMM(d_csr, d_B, d_csr_out, hp_csr_time);
    if (check) ExpectEqualDenseWithError(d_csr_out, d_ref);
    if (!dump.empty()) dump_f32(dump + ".hpspmm.f32", d_csr_out);
    if (hp_csr_time > 0 && hp_csr_time < info.spmm_hp_time_) info.spmm_hp_time_ = hp_csr_time;
    write_info_to_file(csv, info);
    return 0;
  } catch (const std::exception& e) {
    std::cerr << "error: " << e.what() << std::endl;
    return 1;
  }
}
