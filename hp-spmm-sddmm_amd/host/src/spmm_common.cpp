#include "spmm/spmm_common.h"

#include <algorithm>
#include <cerrno>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <iostream>
#include <numeric>

using starml::Device;
using starml::Error;
using starml::kCPU;
using starml::kFloat;
using starml::kHIP;
using starml::kInt32;

extern "C" {
typedef struct hpspmm_graph hpspmm_graph;
const char* hpspmm_gen_last_error(void);
int64_t hpspmm_graph_rows(const hpspmm_graph*);
int64_t hpspmm_graph_cols(const hpspmm_graph*);
int64_t hpspmm_graph_nnz(const hpspmm_graph*);
const int32_t* hpspmm_graph_rowptr(const hpspmm_graph*);
const int32_t* hpspmm_graph_col(const hpspmm_graph*);
const float* hpspmm_graph_val(const hpspmm_graph*);
void hpspmm_graph_free(hpspmm_graph*);
hpspmm_graph* hpspmm_gen_named(const char* name, double scale);
}

namespace {

// Whole file in memory, then strtol over it: the three-line format can hold
// hundreds of MB on one line.
struct SmtxFile {
  int64_t rows = 0, cols = 0, nnz = 0;
  std::vector<int32_t> rowptr, col;
};

std::string slurp(const std::string& filename) {
  std::ifstream in(filename, std::ios::binary);
  if (!in) throw Error("cannot open " + filename);
  in.seekg(0, std::ios::end);
  const std::streamoff n = in.tellg();
  in.seekg(0, std::ios::beg);
  std::string buf((size_t)n, '\0');
  in.read(buf.data(), n);
  return buf;
}

// Parses whitespace-separated integers from [p, line end); returns the position
// after the newline.
const char* parse_int_line(const char* p, const char* end, std::vector<int32_t>& out, const std::string& what) {
  while (p < end) {
    while (p < end && (*p == ' ' || *p == '\t' || *p == '\r')) ++p;
    if (p >= end) break;
    if (*p == '\n') return p + 1;
    char* q = nullptr;
    errno = 0;
    const long v = std::strtol(p, &q, 10);
    if (q == p || errno != 0 || v < INT32_MIN || v > INT32_MAX) throw Error("bad integer in " + what);
    out.push_back((int32_t)v);
    p = q;
  }
  return p;
}

SmtxFile read_smtx(const std::string& filename, bool want_cols) {
  const std::string buf = slurp(filename);
  const char* p = buf.data();
  const char* end = p + buf.size();
  SmtxFile f;
  int r = 0, c = 0, n = 0;
  if (std::sscanf(p, "%d,%d,%d", &r, &c, &n) != 3 || r < 0 || c < 0 || n < 0)
    throw Error(filename + ": first line must be rows,cols,nnz");
  f.rows = r;
  f.cols = c;
  f.nnz = n;
  while (p < end && *p != '\n') ++p;
  if (p < end) ++p;
  f.rowptr.reserve((size_t)f.rows + 1);
  p = parse_int_line(p, end, f.rowptr, filename + " (row offsets)");
  if ((int64_t)f.rowptr.size() != f.rows + 1) throw Error(filename + ": expected rows+1 row offsets");
  if (f.rowptr.front() != 0 || f.rowptr.back() != f.nnz) throw Error(filename + ": row offsets do not span [0, nnz]");
  for (int64_t i = 0; i < f.rows; ++i)
    if (f.rowptr[i + 1] < f.rowptr[i]) throw Error(filename + ": row offsets decrease");
  if (want_cols) {
    f.col.reserve((size_t)f.nnz);
    parse_int_line(p, end, f.col, filename + " (column indices)");
    if ((int64_t)f.col.size() != f.nnz) throw Error(filename + ": expected nnz column indices");
    for (int32_t cc : f.col)
      if (cc < 0 || cc >= f.cols) throw Error(filename + ": column index out of range");
  }
  return f;
}

template <typename T>
Matrix host_vector(const std::vector<T>& v, starml::DataTypeKind kind, int64_t padded = -1) {
  const int64_t n = padded < 0 ? (int64_t)v.size() : padded;
  Matrix m({n}, Device(kCPU), starml::DataType(kind));
  T* d = m.mutable_data<T>();
  std::copy(v.begin(), v.end(), d);
  std::fill(d + v.size(), d + n, T(0));
  return m;
}

CSR_Matrix csr_from_arrays(int64_t rows, int64_t cols, const std::vector<int32_t>& rowptr,
                           const std::vector<int32_t>& col, const std::vector<float>& val) {
  CSR_Matrix m;
  m.num_rows_ = rows;
  m.num_cols_ = cols;
  m.num_nonzeros_ = (int64_t)col.size();
  m.row_offsets_ = host_vector(rowptr, kInt32);
  m.column_indices_ = host_vector(col, kInt32);
  m.values_ = host_vector(val, kFloat);
  return m;
}

std::vector<int> row_lengths(const int32_t* rowptr, int64_t rows) {
  std::vector<int> len((size_t)rows);
  for (int64_t i = 0; i < rows; ++i) len[i] = rowptr[i + 1] - rowptr[i];
  return len;
}

void require_host(const Matrix& m, const char* what) {
  if (!m.device().is_cpu()) throw Error(std::string(what) + ": expected a host matrix");
}

}  // namespace

double spmm_gflops(int64_t nnz, int64_t k, double ms) {
  return ms > 0 ? 2.0 * (double)nnz * (double)k / ms / 1e6 : 0.0;
}

void write_info_to_file(const std::string& filename, ResInfo& info) {
  std::cout << "writing info to : " << filename << std::endl;
  auto tp = [&](float ms) { return (float)spmm_gflops(info.num_nnz_, info.dense_dim_, ms); };
  info.spmm_cs_csralg2_throughput_ = tp(info.spmm_cs_csralg2_time_);
  info.spmm_cs_csralg3_throughput_ = tp(info.spmm_cs_csralg3_time_);
  info.spmm_cs_csrdef_throughput_ = tp(info.spmm_cs_csrdef_time_);
  info.spmm_cs_coo_throughput_ = tp(info.spmm_cs_coo_time_);
  info.spmm_ge_throughput_ = tp(info.spmm_ge_time_);
  info.spmm_hp_throughput_ = tp(info.spmm_hp_time_);
  std::ofstream out(filename, std::ios::app);
  if (!out) throw Error("cannot append to " + filename);
  // column order and labels of the reference's result files (spmm_common.cpp:34-41),
  // so existing post-processing keeps working
  out << info.filename_ << "," << info.num_rows_ << "," << info.num_cols_ << "," << info.num_nnz_ << ","
      << info.dense_dim_ << "," << info.stdv;
  const struct {
    const char* label;
    float ms, gflops;
  } cols[] = {
      {"cuSPARSE(CSR, ALG2): ", info.spmm_cs_csralg2_time_, info.spmm_cs_csralg2_throughput_},
      {"cuSPARSE(CSR, ALG3): ", info.spmm_cs_csralg3_time_, info.spmm_cs_csralg3_throughput_},
      {"cuSPARSE(CSR, Default): ", info.spmm_cs_csrdef_time_, info.spmm_cs_csrdef_throughput_},
      {"cuSPARSE(COO): ", info.spmm_cs_coo_time_, info.spmm_cs_coo_throughput_},
      {"GE-SpMM: ", info.spmm_ge_time_, info.spmm_ge_throughput_},
      {"HP-SpMM ", info.spmm_hp_time_, info.spmm_hp_throughput_},
  };
  for (const auto& c : cols) out << "," << c.label << "," << c.ms << "," << c.gflops;
  out << std::endl;
}

CSR_Matrix get_csr_mat_from_smtx(const std::string& filename, int64_t& num, int64_t& dim,
                                 int64_t& real_nonzero_num) {
  std::cout << "loading csr mat from smtx file... " << filename << std::endl;
  const SmtxFile f = read_smtx(filename, true);
  num = f.rows;
  dim = f.cols;
  real_nonzero_num = f.nnz;
  return csr_from_arrays(f.rows, f.cols, f.rowptr, f.col, std::vector<float>((size_t)f.nnz, 1.0f));
}

int64_t roundUpToNextMultiple(int64_t num, int64_t multiple) {
  if (multiple <= 0) return num;
  const int64_t rem = num % multiple;
  return rem == 0 ? num : num + multiple - rem;
}

COO_Matrix csr_to_coo(const CSR_Matrix& a, int padding) {
  std::vector<int32_t> order((size_t)a.num_rows_);
  std::iota(order.begin(), order.end(), 0);
  COO_Matrix m = csr_to_coo_reorder(a, order, padding);
  // the plain loader reports the padded count, the reorder loader the true one
  // (spmm_common.cpp:233 vs :294)
  m.num_nonzeros_ = m.values_.size();
  return m;
}

COO_Matrix csr_to_coo_reorder(const CSR_Matrix& a, const std::vector<int32_t>& row_order, int padding) {
  require_host(a.row_offsets_, "csr_to_coo");
  const int32_t* rp = a.row_offsets_.data<int32_t>();
  const int32_t* ci = a.column_indices_.data<int32_t>();
  const float* va = a.values_.data<float>();
  const int64_t nnz = a.values_.size();
  if ((int64_t)row_order.size() != a.num_rows_) throw Error("reorder: need one entry per row");
  std::vector<char> seen((size_t)a.num_rows_, 0);
  for (int32_t r : row_order) {
    if (r < 0 || r >= a.num_rows_ || seen[r]) throw Error("reorder: not a permutation of the rows");
    seen[r] = 1;
  }
  const int64_t padded = roundUpToNextMultiple(nnz, padding);
  COO_Matrix m;
  m.num_rows_ = a.num_rows_;
  m.num_cols_ = a.num_cols_;
  m.num_nonzeros_ = nnz;
  m.row_indices_ = starml::full({padded}, Device(kCPU), kInt32, 0);
  m.column_indices_ = starml::full({padded}, Device(kCPU), kInt32, 0);
  m.values_ = starml::full({padded}, Device(kCPU), kFloat, 0.0);
  int32_t* orow = m.row_indices_.mutable_data<int32_t>();
  int32_t* ocol = m.column_indices_.mutable_data<int32_t>();
  float* oval = m.values_.mutable_data<float>();
  int64_t w = 0;
  for (int32_t r : row_order) {
    for (int32_t j = rp[r]; j < rp[r + 1]; ++j, ++w) {
      orow[w] = r;
      ocol[w] = ci[j];
      oval[w] = va[j];
    }
  }
  return m;
}

COO_Matrix get_coo_mat_from_smtx(const std::string& filename, int64_t& num, int64_t& dim,
                                 int64_t& real_nonzero_num, int padding) {
  std::cout << "loading coo mat from smtx file... " << filename << std::endl;
  const SmtxFile f = read_smtx(filename, true);
  num = f.rows;
  dim = f.cols;
  real_nonzero_num = f.nnz;
  return csr_to_coo(csr_from_arrays(f.rows, f.cols, f.rowptr, f.col, std::vector<float>((size_t)f.nnz, 1.0f)),
                    padding);
}

COO_Matrix get_coo_mat_from_smtx_reorder(const std::string& filename, const std::string& reorder_filename,
                                         int64_t& num, int64_t& dim, int64_t& real_nonzero_num, int padding) {
  std::cout << "loading coo reorderd mat from smtx file... " << filename << std::endl;
  const SmtxFile f = read_smtx(filename, true);
  num = f.rows;
  dim = f.cols;
  real_nonzero_num = f.nnz;
  const std::string buf = slurp(reorder_filename);
  std::vector<int32_t> order;
  order.reserve((size_t)f.rows);
  parse_int_line(buf.data(), buf.data() + buf.size(), order, reorder_filename);
  return csr_to_coo_reorder(
      csr_from_arrays(f.rows, f.cols, f.rowptr, f.col, std::vector<float>((size_t)f.nnz, 1.0f)), order, padding);
}

void write_smtx(const std::string& filename, const CSR_Matrix& a) {
  require_host(a.row_offsets_, "write_smtx");
  std::FILE* fp = std::fopen(filename.c_str(), "w");
  if (!fp) throw Error("cannot write " + filename);
  std::fprintf(fp, "%lld, %lld, %lld\n", (long long)a.num_rows_, (long long)a.num_cols_,
               (long long)a.values_.size());
  const int32_t* rp = a.row_offsets_.data<int32_t>();
  for (int64_t i = 0; i <= a.num_rows_; ++i) std::fprintf(fp, "%d ", rp[i]);
  std::fputc('\n', fp);
  const int32_t* ci = a.column_indices_.data<int32_t>();
  for (int64_t j = 0; j < a.values_.size(); ++j) std::fprintf(fp, "%d ", ci[j]);
  std::fputc('\n', fp);
  std::fclose(fp);
}

double calVarStdev(const std::vector<int>& v) {
  if (v.empty()) return 0.0;
  const double mean = std::accumulate(v.begin(), v.end(), 0.0) / (double)v.size();
  double acc = 0.0;
  for (int x : v) acc += ((double)x - mean) * ((double)x - mean);
  return std::sqrt(acc / (double)v.size());
}

double calCV(const std::vector<int>& v) {
  if (v.empty()) return 0.0;
  const double mean = std::accumulate(v.begin(), v.end(), 0.0) / (double)v.size();
  return calVarStdev(v) / mean;
}

double get_standard_CV(const std::string& filename) {
  std::cout << "calculate std cov... " << std::endl;
  const SmtxFile f = read_smtx(filename, false);
  return calCV(row_lengths(f.rowptr.data(), f.rows));
}

double csr_row_length_cv(const CSR_Matrix& a) {
  require_host(a.row_offsets_, "csr_row_length_cv");
  return calCV(row_lengths(a.row_offsets_.data<int32_t>(), a.num_rows_));
}

CSR_Matrix csr_to_cuda(const CSR_Matrix& a) {
  CSR_Matrix d = a;
  d.values_ = a.values_.to(kHIP);
  d.row_offsets_ = a.row_offsets_.to(kHIP);
  d.column_indices_ = a.column_indices_.to(kHIP);
  return d;
}

CSR_Matrix csr_to_host(const CSR_Matrix& a) {
  CSR_Matrix h = a;
  h.values_ = a.values_.to(kCPU);
  h.row_offsets_ = a.row_offsets_.to(kCPU);
  h.column_indices_ = a.column_indices_.to(kCPU);
  return h;
}

COO_Matrix coo_to_cuda(const COO_Matrix& a) {
  COO_Matrix d = a;
  d.values_ = a.values_.to(kHIP);
  d.row_indices_ = a.row_indices_.to(kHIP);
  d.column_indices_ = a.column_indices_.to(kHIP);
  return d;
}

COO_Matrix coo_to_host(const COO_Matrix& a) {
  COO_Matrix h = a;
  h.values_ = a.values_.to(kCPU);
  h.row_indices_ = a.row_indices_.to(kCPU);
  h.column_indices_ = a.column_indices_.to(kCPU);
  return h;
}

Matrix csrtodense_cpu(const CSR_Matrix& a) {
  require_host(a.row_offsets_, "csrtodense_cpu");
  const int64_t m = a.num_rows_, n = a.num_cols_;
  Matrix dense = starml::full({m, n}, Device(kCPU), kFloat, 0.0);
  float* d = dense.mutable_data<float>();
  const int32_t* rp = a.row_offsets_.data<int32_t>();
  const int32_t* ci = a.column_indices_.data<int32_t>();
  const float* va = a.values_.data<float>();
  for (int64_t i = 0; i < m; ++i)
    for (int32_t j = rp[i]; j < rp[i + 1]; ++j) {
      if (ci[j] < 0 || ci[j] >= n) throw Error("csrtodense_cpu: column index out of range");
      d[(size_t)i * (size_t)n + (size_t)ci[j]] = va[j];
    }
  return dense;
}

CSR_Matrix make_synthetic_csr(const std::string& name, double scale) {
  hpspmm_graph* g = hpspmm_gen_named(name.c_str(), scale);
  if (!g) throw Error(std::string("graph generator: ") + hpspmm_gen_last_error());
  const int64_t rows = hpspmm_graph_rows(g), nnz = hpspmm_graph_nnz(g);
  CSR_Matrix m = csr_from_arrays(
      rows, hpspmm_graph_cols(g), std::vector<int32_t>(hpspmm_graph_rowptr(g), hpspmm_graph_rowptr(g) + rows + 1),
      std::vector<int32_t>(hpspmm_graph_col(g), hpspmm_graph_col(g) + nnz),
      std::vector<float>(hpspmm_graph_val(g), hpspmm_graph_val(g) + nnz));
  hpspmm_graph_free(g);
  return m;
}
