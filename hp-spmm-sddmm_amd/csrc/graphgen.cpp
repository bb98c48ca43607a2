// Seeded synthetic sparse-graph and dense-matrix generators (host, OpenMP).
//
// The reference ships no datasets (dataset/download.sh fetches them) and fills
// its dense operand from an unseeded generator
// (spmm/starml/operators/cpu/factories_kernel.cpp:14-28), so every benchmark
// input is produced here instead.  All randomness comes from a counter-based
// hash (seed, stream, index) -> 64 bits, so an output never depends on the
// number of threads or on scheduling, and any element can be regenerated in
// isolation.
//
// Every graph is returned as CSR with int32 zero-based indices, columns
// strictly increasing inside each row (duplicates merged), matching the CSR
// container of the reference (include/spmm/mm/spmm_common.h:58-82).
#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <new>
#include <string>
#include <vector>

#ifdef _OPENMP
#include <omp.h>
#endif

namespace {

thread_local std::string g_err;

inline uint64_t mix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

// One 64-bit draw for (seed, stream, index).
inline uint64_t draw(uint64_t seed, uint64_t stream, uint64_t idx) {
  return mix64(mix64(seed * 0xD1342543DE82EF95ull + stream) ^ (idx * 0x9E3779B97F4A7C15ull));
}

inline double u01(uint64_t x) { return (double)(x >> 11) * (1.0 / 9007199254740992.0); }          // [0,1)
inline double u01_open0(uint64_t x) { return (double)((x >> 11) + 1) * (1.0 / 9007199254740992.0); }  // (0,1]

enum ValueMode { kValSymUniformPM1 = 0, kValSymUniform01 = 1, kValRowNormalised = 2, kValOnes = 3,
                 kValUniformPM1 = 4 };

struct Graph {
  int64_t rows = 0, cols = 0, nnz = 0;
  std::vector<int32_t> rowptr, col;
  std::vector<float> val;
};

// Walker alias table: O(1) sampling of an index with probability w[i] / sum(w).
struct Alias {
  std::vector<double> prob;
  std::vector<int32_t> alias;
  void build(const std::vector<double>& w) {
    const int64_t n = (int64_t)w.size();
    prob.assign(n, 0.0);
    alias.assign(n, 0);
    double sum = 0;
    for (double x : w) sum += x;
    std::vector<int32_t> small, large;
    small.reserve(n);
    large.reserve(n);
    std::vector<double> p(n);
    for (int64_t i = 0; i < n; ++i) {
      p[i] = w[i] * (double)n / sum;
      (p[i] < 1.0 ? small : large).push_back((int32_t)i);
    }
    while (!small.empty() && !large.empty()) {
      const int32_t s = small.back(); small.pop_back();
      const int32_t l = large.back(); large.pop_back();
      prob[s] = p[s];
      alias[s] = l;
      p[l] = (p[l] + p[s]) - 1.0;
      (p[l] < 1.0 ? small : large).push_back(l);
    }
    for (int32_t i : large) { prob[i] = 1.0; alias[i] = i; }
    for (int32_t i : small) { prob[i] = 1.0; alias[i] = i; }
  }
  inline int32_t sample(uint64_t r) const {
    const uint64_t n = prob.size();
    // high 32 bits pick the slot, low 32 bits decide slot vs alias
    const uint64_t slot = ((r >> 32) * n) >> 32;
    const double u = (double)(r & 0xFFFFFFFFull) * (1.0 / 4294967296.0);
    return u < prob[slot] ? (int32_t)slot : alias[slot];
  }
};

inline float edge_value(int mode, uint64_t seed, int64_t i, int64_t j, int64_t ncols) {
  switch (mode) {
    case kValSymUniformPM1: {
      const int64_t a = std::min(i, j), b = std::max(i, j);
      return (float)(2.0 * u01(draw(seed, 101, (uint64_t)(a * ncols + b))) - 1.0);
    }
    case kValSymUniform01: {
      const int64_t a = std::min(i, j), b = std::max(i, j);
      return (float)u01(draw(seed, 101, (uint64_t)(a * ncols + b)));
    }
    case kValUniformPM1:
      return (float)(2.0 * u01(draw(seed, 101, (uint64_t)(i * ncols + j))) - 1.0);
    default:
      return 1.0f;
  }
}

// Build a symmetric CSR from E sampled undirected edges (u, v) = sampler(e):
// both (u,v) and (v,u) are stored, duplicates merged, optional self-loops on
// every vertex.  The sampler is called twice per edge (count pass, scatter
// pass) and must be a pure function of e.
template <class Sampler>
Graph* build_symmetric(int64_t N, int64_t E, const Sampler& sampler, bool self_loops, int value_mode,
                       uint64_t seed) {
  std::vector<int64_t> off(N + 1, 0);
  {
    std::vector<std::atomic<int32_t>> cnt(N);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < N; ++i) cnt[i].store(self_loops ? 1 : 0, std::memory_order_relaxed);
#pragma omp parallel for schedule(static)
    for (int64_t e = 0; e < E; ++e) {
      int32_t u, v;
      sampler(e, u, v);
      if (u == v) {
        if (!self_loops) cnt[u].fetch_add(1, std::memory_order_relaxed);
      } else {
        cnt[u].fetch_add(1, std::memory_order_relaxed);
        cnt[v].fetch_add(1, std::memory_order_relaxed);
      }
    }
    for (int64_t i = 0; i < N; ++i) off[i + 1] = off[i] + cnt[i].load(std::memory_order_relaxed);
  }
  const int64_t raw = off[N];
  std::vector<int32_t> raw_col((size_t)raw);
  {
    std::vector<std::atomic<int64_t>> cur(N);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < N; ++i) {
      int64_t c = off[i];
      if (self_loops) raw_col[c++] = (int32_t)i;
      cur[i].store(c, std::memory_order_relaxed);
    }
#pragma omp parallel for schedule(static)
    for (int64_t e = 0; e < E; ++e) {
      int32_t u, v;
      sampler(e, u, v);
      if (u == v) {
        if (!self_loops) raw_col[cur[u].fetch_add(1, std::memory_order_relaxed)] = v;
      } else {
        raw_col[cur[u].fetch_add(1, std::memory_order_relaxed)] = v;
        raw_col[cur[v].fetch_add(1, std::memory_order_relaxed)] = u;
      }
    }
  }
  // sort + unique inside each row (this also erases the scatter order)
  std::vector<int64_t> newoff(N + 1, 0);
#pragma omp parallel for schedule(dynamic, 256)
  for (int64_t i = 0; i < N; ++i) {
    int32_t* b = raw_col.data() + off[i];
    int32_t* e = raw_col.data() + off[i + 1];
    std::sort(b, e);
    newoff[i + 1] = std::unique(b, e) - b;
  }
  for (int64_t i = 0; i < N; ++i) newoff[i + 1] += newoff[i];
  const int64_t nnz = newoff[N];
  if (nnz > 0x7FFFFFFFll) {
    g_err = "generated graph has more than 2^31-1 nonzeros";
    return nullptr;
  }
  Graph* g = new Graph;
  g->rows = g->cols = N;
  g->nnz = nnz;
  g->rowptr.resize(N + 1);
  g->col.resize((size_t)nnz);
  g->val.resize((size_t)nnz);
#pragma omp parallel for schedule(dynamic, 256)
  for (int64_t i = 0; i < N; ++i) {
    g->rowptr[i] = (int32_t)newoff[i];
    const int64_t len = newoff[i + 1] - newoff[i];
    const int32_t* src = raw_col.data() + off[i];
    int32_t* dc = g->col.data() + newoff[i];
    float* dv = g->val.data() + newoff[i];
    for (int64_t j = 0; j < len; ++j) {
      dc[j] = src[j];
      dv[j] = (value_mode == kValRowNormalised) ? 1.0f / (float)len
                                                 : edge_value(value_mode, seed, i, src[j], N);
    }
  }
  g->rowptr[N] = (int32_t)nnz;
  return g;
}

// Chung-Lu: both endpoints drawn independently with probability ~ weight.
struct ChungLuSampler {
  const Alias* table;
  uint64_t seed;
  inline void operator()(int64_t e, int32_t& u, int32_t& v) const {
    u = table->sample(draw(seed, 11, (uint64_t)e));
    v = table->sample(draw(seed, 12, (uint64_t)e));
  }
};

// Chung-Lu with planted communities: the second endpoint stays inside the first
// endpoint's community with probability p_intra (weights still apply inside).
struct CommunitySampler {
  const Alias* table;
  const int32_t* label;       // vertex -> community
  const int64_t* cstart;      // community -> start in members[]
  const int32_t* members;     // vertices grouped by community
  const double* mcum;         // inclusive prefix sums of weights in members[] order
  double p_intra;
  uint64_t seed;
  inline void operator()(int64_t e, int32_t& u, int32_t& v) const {
    u = table->sample(draw(seed, 11, (uint64_t)e));
    const uint64_t r = draw(seed, 13, (uint64_t)e);
    if (u01(r) < p_intra) {
      const int32_t c = label[u];
      const int64_t lo = cstart[c], hi = cstart[c + 1];
      const double base = lo ? mcum[lo - 1] : 0.0;
      const double x = base + u01(draw(seed, 14, (uint64_t)e)) * (mcum[hi - 1] - base);
      const double* p = std::upper_bound(mcum + lo, mcum + hi, x);
      int64_t k = p - mcum;
      if (k >= hi) k = hi - 1;
      v = members[k];
    } else {
      v = table->sample(draw(seed, 12, (uint64_t)e));
    }
  }
};

// R-MAT: recursive quadrant choice with probabilities (a, b, c, 1-a-b-c).
struct RmatSampler {
  int scale;
  uint32_t ta, tab, tabc;  // cumulative thresholds on a 32-bit uniform
  uint64_t seed;
  inline void operator()(int64_t e, int32_t& u, int32_t& v) const {
    uint32_t r = 0, c = 0;
    uint64_t bits = 0;
    for (int level = 0; level < scale; ++level) {
      if ((level & 1) == 0) bits = draw(seed, 21 + (uint64_t)(level >> 1), (uint64_t)e);
      const uint32_t x = (uint32_t)(bits & 0xFFFFFFFFull);
      bits >>= 32;
      const uint32_t rb = x >= tab ? 1u : 0u;                       // lower half: c or d
      const uint32_t cb = (x >= ta && x < tab) || x >= tabc ? 1u : 0u;  // right half: b or d
      r = (r << 1) | rb;
      c = (c << 1) | cb;
    }
    u = (int32_t)r;
    v = (int32_t)c;
  }
};

// Edges kept in arrays (a generator that builds its edge list one edge after the other).
struct ListSampler {
  const int32_t* us;
  const int32_t* vs;
  inline void operator()(int64_t e, int32_t& u, int32_t& v) const {
    u = us[e];
    v = vs[e];
  }
};

// side x side grid, vertex = y * side + x: edges to the right, lower, lower-right and lower-left
// neighbours (with their mirror images: the 8 neighbours of a 9-point stencil) and `noise` edges per
// vertex to uniformly random vertices.  Edge e belongs to vertex e / (4 + noise).
struct GridSampler {
  int64_t side;
  int noise;
  uint64_t seed;
  inline void operator()(int64_t e, int32_t& u, int32_t& v) const {
    const int64_t per = 4 + noise, vert = e / per, which = e - vert * per;
    const int64_t x = vert % side, y = vert / side;
    u = (int32_t)vert;
    int64_t nx = x, ny = y;
    if (which == 0) nx = x + 1;
    else if (which == 1) ny = y + 1;
    else if (which == 2) { nx = x + 1; ny = y + 1; }
    else if (which == 3) { nx = x - 1; ny = y + 1; }
    else {
      v = (int32_t)(((unsigned __int128)draw(seed, 51, (uint64_t)e) * (uint64_t)(side * side)) >> 64);
      return;
    }
    v = (nx < 0 || nx >= side || ny >= side) ? u : (int32_t)(ny * side + nx);  // off the grid: a self-loop
  }
};

// Communities of mixed sizes as consecutive vertex ranges: the second endpoint is uniform inside the
// first one's community with probability p_intra, else uniform over all vertices.
struct BlockSampler {
  const int64_t* bstart;  // community -> first vertex; [n_blocks] = n
  const int32_t* block;   // vertex -> community
  int64_t n;
  double p_intra;
  uint64_t seed;
  inline void operator()(int64_t e, int32_t& u, int32_t& v) const {
    u = (int32_t)(((unsigned __int128)draw(seed, 61, (uint64_t)e) * (uint64_t)n) >> 64);
    const uint64_t r = draw(seed, 62, (uint64_t)e);
    if (u01(draw(seed, 63, (uint64_t)e)) < p_intra) {
      const int64_t lo = bstart[block[u]], hi = bstart[block[u] + 1];
      v = (int32_t)(lo + (int64_t)(((unsigned __int128)r * (uint64_t)(hi - lo)) >> 64));
    } else {
      v = (int32_t)(((unsigned __int128)r * (uint64_t)n) >> 64);
    }
  }
};

}  // namespace

extern "C" {

typedef struct hpspmm_graph hpspmm_graph;

const char* hpspmm_gen_last_error(void) { return g_err.c_str(); }

int64_t hpspmm_graph_rows(const hpspmm_graph* g) { return ((const Graph*)g)->rows; }
int64_t hpspmm_graph_cols(const hpspmm_graph* g) { return ((const Graph*)g)->cols; }
int64_t hpspmm_graph_nnz(const hpspmm_graph* g) { return ((const Graph*)g)->nnz; }
const int32_t* hpspmm_graph_rowptr(const hpspmm_graph* g) { return ((const Graph*)g)->rowptr.data(); }
const int32_t* hpspmm_graph_col(const hpspmm_graph* g) { return ((const Graph*)g)->col.data(); }
const float* hpspmm_graph_val(const hpspmm_graph* g) { return ((const Graph*)g)->val.data(); }
void hpspmm_graph_free(hpspmm_graph* g) { delete (Graph*)g; }

// rows x cols, exactly nnz_per_row distinct uniformly placed columns per row,
// values U(-1,1).
hpspmm_graph* hpspmm_gen_uniform_rows(int64_t rows, int64_t cols, int64_t nnz_per_row, uint64_t seed) {
  if (rows < 0 || cols <= 0 || nnz_per_row < 0 || nnz_per_row > cols ||
      rows * nnz_per_row > 0x7FFFFFFFll) {
    g_err = "gen_uniform_rows: bad arguments";
    return nullptr;
  }
  Graph* g = new Graph;
  g->rows = rows;
  g->cols = cols;
  g->nnz = rows * nnz_per_row;
  g->rowptr.resize(rows + 1);
  g->col.resize((size_t)g->nnz);
  g->val.resize((size_t)g->nnz);
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < rows; ++i) {
    g->rowptr[i] = (int32_t)(i * nnz_per_row);
    int32_t* c = g->col.data() + i * nnz_per_row;
    // Floyd's sampling without replacement: for t = cols-k .. cols-1 pick
    // j in [0, t]; take j unless already taken, else take t.
    int64_t got = 0;
    for (int64_t t = cols - nnz_per_row; t < cols; ++t) {
      const uint64_t r = draw(seed, 31, (uint64_t)(i * nnz_per_row + got));
      int32_t j = (int32_t)(((unsigned __int128)r * (uint64_t)(t + 1)) >> 64);
      bool dup = false;
      for (int64_t q = 0; q < got; ++q) dup |= (c[q] == j);
      c[got++] = dup ? (int32_t)t : j;
    }
    std::sort(c, c + nnz_per_row);
    float* v = g->val.data() + i * nnz_per_row;
    for (int64_t q = 0; q < nnz_per_row; ++q) v[q] = edge_value(kValUniformPM1, seed, i, c[q], cols);
  }
  g->rowptr[rows] = (int32_t)g->nnz;
  return (hpspmm_graph*)g;
}

// Citation-style graph: vertex weights from a Zipf(alpha) law on {1..wmax},
// n_edges Chung-Lu edges, symmetrised, self-loop on every vertex, values
// 1/deg(row).
hpspmm_graph* hpspmm_gen_citation(int64_t n, double alpha, int64_t wmax, int64_t n_edges, uint64_t seed) {
  if (n <= 0 || wmax <= 0 || n_edges < 0 || alpha <= 1.0) {
    g_err = "gen_citation: bad arguments";
    return nullptr;
  }
  std::vector<double> zcum((size_t)wmax);
  double s = 0;
  for (int64_t k = 1; k <= wmax; ++k) { s += std::pow((double)k, -alpha); zcum[k - 1] = s; }
  std::vector<double> w((size_t)n);
  for (int64_t i = 0; i < n; ++i) {
    const double x = u01(draw(seed, 1, (uint64_t)i)) * s;
    w[i] = (double)((std::upper_bound(zcum.begin(), zcum.end(), x) - zcum.begin()) + 1);
    if (w[i] > (double)wmax) w[i] = (double)wmax;
  }
  Alias table;
  table.build(w);
  ChungLuSampler smp{&table, seed};
  return (hpspmm_graph*)build_symmetric(n, n_edges, smp, true, kValRowNormalised, seed);
}

// Social-style graph: Chung-Lu on power-law weights w_i = (i + i0)^(-1/(gamma-1)),
// randomly relabelled, n_edges undirected samples, values U(0,1).
hpspmm_graph* hpspmm_gen_powerlaw(int64_t n, double gamma, double i0, int64_t n_edges, int value_mode,
                                  uint64_t seed) {
  if (n <= 0 || gamma <= 1.0 || i0 <= 0 || n_edges < 0) {
    g_err = "gen_powerlaw: bad arguments";
    return nullptr;
  }
  // random relabelling so that hubs are spread over the index range
  std::vector<std::pair<uint64_t, int32_t>> key((size_t)n);
  for (int64_t i = 0; i < n; ++i) key[i] = {draw(seed, 2, (uint64_t)i), (int32_t)i};
  std::sort(key.begin(), key.end());
  std::vector<double> w((size_t)n);
  const double beta = 1.0 / (gamma - 1.0);
  for (int64_t r = 0; r < n; ++r) w[key[r].second] = std::pow((double)r + i0, -beta);
  Alias table;
  table.build(w);
  ChungLuSampler smp{&table, seed};
  return (hpspmm_graph*)build_symmetric(n, n_edges, smp, false, value_mode, seed);
}

// Co-purchase-style graph: lognormal(mu, sigma) weights, n_comm random
// community labels, a fraction p_intra of sampled edges stays inside the first
// endpoint's community; values U(0,1).
hpspmm_graph* hpspmm_gen_community(int64_t n, double mu, double sigma, int64_t n_comm, double p_intra,
                                   int64_t n_edges, uint64_t seed) {
  if (n <= 0 || n_comm <= 0 || n_edges < 0 || p_intra < 0 || p_intra > 1) {
    g_err = "gen_community: bad arguments";
    return nullptr;
  }
  std::vector<double> w((size_t)n);
  std::vector<int32_t> label((size_t)n);
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    const double u1 = u01_open0(draw(seed, 3, (uint64_t)i));
    const double u2 = u01(draw(seed, 4, (uint64_t)i));
    const double z = std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586 * u2);
    w[i] = std::exp(mu + sigma * z);
    label[i] = (int32_t)(((unsigned __int128)draw(seed, 5, (uint64_t)i) * (uint64_t)n_comm) >> 64);
  }
  std::vector<int64_t> cstart((size_t)n_comm + 1, 0);
  for (int64_t i = 0; i < n; ++i) cstart[label[i] + 1]++;
  for (int64_t c = 0; c < n_comm; ++c) cstart[c + 1] += cstart[c];
  std::vector<int32_t> members((size_t)n);
  {
    std::vector<int64_t> cur(cstart.begin(), cstart.end() - 1);
    for (int64_t i = 0; i < n; ++i) members[cur[label[i]]++] = (int32_t)i;
  }
  std::vector<double> mcum((size_t)n);
  double s = 0;
  for (int64_t k = 0; k < n; ++k) { s += w[members[k]]; mcum[k] = s; }
  Alias table;
  table.build(w);
  CommunitySampler smp{&table, label.data(), cstart.data(), members.data(), mcum.data(), p_intra, seed};
  return (hpspmm_graph*)build_symmetric(n, n_edges, smp, false, kValSymUniform01, seed);
}

// R-MAT graph on 2^scale vertices with n_edges samples, duplicates merged,
// symmetrised, vertex ids left as generated (hubs at low ids, many empty
// rows); values U(-1,1).
hpspmm_graph* hpspmm_gen_rmat(int scale, int64_t n_edges, double a, double b, double c, uint64_t seed) {
  if (scale <= 0 || scale > 30 || n_edges < 0 || a <= 0 || b < 0 || c < 0 || a + b + c >= 1.0) {
    g_err = "gen_rmat: bad arguments";
    return nullptr;
  }
  RmatSampler smp;
  smp.scale = scale;
  smp.ta = (uint32_t)(a * 4294967296.0);
  smp.tab = (uint32_t)((a + b) * 4294967296.0);
  smp.tabc = (uint32_t)((a + b + c) * 4294967296.0);
  smp.seed = seed;
  return (hpspmm_graph*)build_symmetric((int64_t)1 << scale, n_edges, smp, false, kValSymUniformPM1, seed);
}

// ---------------------------------------------------------------------------------------------
// Families that none of the library's thresholds was chosen on: they exist to check that the plan's
// choice of strategy holds up on matrices unlike the benchmark's four.
// ---------------------------------------------------------------------------------------------

// Preferential attachment (Barabasi-Albert): vertex t brings m edges whose other ends are drawn in
// proportion to the degrees so far (an endpoint of a uniformly chosen earlier edge, or the vertex
// before when there is none yet); vertices relabelled at random; values U(0,1).
hpspmm_graph* hpspmm_gen_pref_attach(int64_t n, int64_t m, uint64_t seed) {
  if (n < 2 || m < 1 || n * m > 0x3FFFFFFFll) {
    g_err = "gen_pref_attach: bad arguments";
    return nullptr;
  }
  const int64_t E = (n - 1) * m;
  std::vector<int32_t> us((size_t)E), vs((size_t)E);
  std::vector<int32_t> label((size_t)n);
  {
    std::vector<std::pair<uint64_t, int32_t>> key((size_t)n);
    for (int64_t i = 0; i < n; ++i) key[i] = {draw(seed, 71, (uint64_t)i), (int32_t)i};
    std::sort(key.begin(), key.end());
    for (int64_t i = 0; i < n; ++i) label[key[i].second] = (int32_t)i;
  }
  // (sequential by nature: every draw looks at the edges before it; unlabelled vertices here)
  for (int64_t e = 0; e < E; ++e) {
    const int64_t t = 1 + e / m;
    int32_t other = (int32_t)(t - 1);
    if (e >= m) {  // an endpoint of one of the edges brought by earlier vertices
      const int64_t before = (t - 1) * m;
      const uint64_t r = draw(seed, 72, (uint64_t)e);
      const int64_t pick = (int64_t)(((unsigned __int128)r * (uint64_t)(2 * before)) >> 64);
      other = (pick & 1) ? vs[pick >> 1] : us[pick >> 1];
    }
    us[e] = (int32_t)t;
    vs[e] = other;
  }
#pragma omp parallel for schedule(static)
  for (int64_t e = 0; e < E; ++e) {
    us[e] = label[us[e]];
    vs[e] = label[vs[e]];
  }
  ListSampler smp{us.data(), vs.data()};
  return (hpspmm_graph*)build_symmetric(n, E, smp, false, kValSymUniform01, seed);
}

// 9-point stencil on a side x side grid plus `noise` random long-range edges per vertex, symmetric,
// a self-loop on every vertex; values 1 / (row length): an averaging operator.
hpspmm_graph* hpspmm_gen_grid(int64_t side, int noise, uint64_t seed) {
  if (side < 2 || noise < 0 || side * side * (4 + noise) > 0x3FFFFFFFll) {
    g_err = "gen_grid: bad arguments";
    return nullptr;
  }
  GridSampler smp{side, noise, seed};
  return (hpspmm_graph*)build_symmetric(side * side, side * side * (4 + noise), smp, true, kValRowNormalised, seed);
}

// Rectangular users x items: every user (row) draws a lognormal(mu, sigma) number of items (columns)
// from a Zipf(alpha)-weighted popularity, duplicates merged; values U(-1,1).  Not symmetric, not square.
hpspmm_graph* hpspmm_gen_bipartite(int64_t users, int64_t items, double mu, double sigma, double alpha,
                                   uint64_t seed) {
  if (users < 1 || items < 1 || alpha <= 0) {
    g_err = "gen_bipartite: bad arguments";
    return nullptr;
  }
  std::vector<double> w((size_t)items);
  {
    // popularity rank -> item id shuffled, so that popular items are spread over the columns
    std::vector<std::pair<uint64_t, int32_t>> key((size_t)items);
    for (int64_t i = 0; i < items; ++i) key[i] = {draw(seed, 81, (uint64_t)i), (int32_t)i};
    std::sort(key.begin(), key.end());
    for (int64_t r = 0; r < items; ++r) w[key[r].second] = std::pow((double)r + 10.0, -alpha);
  }
  Alias table;
  table.build(w);
  std::vector<int64_t> off((size_t)users + 1, 0);
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < users; ++i) {
    const double u1 = u01_open0(draw(seed, 82, (uint64_t)i));
    const double u2 = u01(draw(seed, 83, (uint64_t)i));
    const double z = std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586 * u2);
    off[i + 1] = std::min<int64_t>(items, std::max<int64_t>(1, (int64_t)std::llround(std::exp(mu + sigma * z))));
  }
  for (int64_t i = 0; i < users; ++i) off[i + 1] += off[i];
  if (off[users] > 0x7FFFFFFFll) {
    g_err = "gen_bipartite: too many nonzeros";
    return nullptr;
  }
  std::vector<int32_t> raw((size_t)off[users]);
  std::vector<int64_t> newoff((size_t)users + 1, 0);
#pragma omp parallel for schedule(dynamic, 256)
  for (int64_t i = 0; i < users; ++i) {
    int32_t* b = raw.data() + off[i];
    const int64_t d = off[i + 1] - off[i];
    for (int64_t j = 0; j < d; ++j) b[j] = table.sample(draw(seed, 84, (uint64_t)(off[i] + j)));
    std::sort(b, b + d);
    newoff[i + 1] = std::unique(b, b + d) - b;
  }
  for (int64_t i = 0; i < users; ++i) newoff[i + 1] += newoff[i];
  Graph* g = new Graph;
  g->rows = users;
  g->cols = items;
  g->nnz = newoff[users];
  g->rowptr.resize((size_t)users + 1);
  g->col.resize((size_t)g->nnz);
  g->val.resize((size_t)g->nnz);
#pragma omp parallel for schedule(dynamic, 256)
  for (int64_t i = 0; i < users; ++i) {
    g->rowptr[i] = (int32_t)newoff[i];
    const int64_t len = newoff[i + 1] - newoff[i];
    for (int64_t j = 0; j < len; ++j) {
      const int32_t c = raw[off[i] + j];
      g->col[newoff[i] + j] = c;
      g->val[newoff[i] + j] = edge_value(kValUniformPM1, seed, i, c, items);
    }
  }
  g->rowptr[users] = (int32_t)g->nnz;
  return (hpspmm_graph*)g;
}

// Communities of mixed sizes (power law between min_size and max_size, exponent 2) as consecutive
// vertex ranges; n_edges undirected samples of which p_intra stay inside a community; values U(0,1).
hpspmm_graph* hpspmm_gen_blocks(int64_t n, int64_t min_size, int64_t max_size, double p_intra, int64_t n_edges,
                                uint64_t seed) {
  if (n < 1 || min_size < 1 || max_size < min_size || n_edges < 0 || p_intra < 0 || p_intra > 1) {
    g_err = "gen_blocks: bad arguments";
    return nullptr;
  }
  std::vector<int64_t> bstart{0};
  while (bstart.back() < n) {
    // inverse-CDF draw of a size with density ~ s^-2 on [min_size, max_size]
    const double u = u01(draw(seed, 91, (uint64_t)bstart.size()));
    const double a = 1.0 / (double)min_size, b = 1.0 / (double)max_size;
    const int64_t size = std::max<int64_t>(min_size, (int64_t)(1.0 / (a - u * (a - b))));
    bstart.push_back(std::min(n, bstart.back() + size));
  }
  const int64_t n_blocks = (int64_t)bstart.size() - 1;
  std::vector<int32_t> block((size_t)n);
#pragma omp parallel for schedule(dynamic, 64)
  for (int64_t c = 0; c < n_blocks; ++c)
    for (int64_t v = bstart[c]; v < bstart[c + 1]; ++v) block[v] = (int32_t)c;
  BlockSampler smp{bstart.data(), block.data(), n, p_intra, seed};
  return (hpspmm_graph*)build_symmetric(n, n_edges, smp, false, kValSymUniform01, seed);
}

// ---------------------------------------------------------------------------------------------
// Cache model (CPU side, for traffic estimates): misses of a fully associative LRU cache of
// `capacity` entries over a stream of n ids in [0, id_range).  Negative ids are skipped.
// ---------------------------------------------------------------------------------------------
int64_t hpspmm_model_lru_misses(const int32_t* ids, int64_t n, int64_t id_range, int64_t capacity) {
  if (!ids || n < 0 || id_range <= 0 || capacity <= 0) return -1;
  // doubly linked list over the ids, most recent at the head
  std::vector<int32_t> prev((size_t)id_range, -1), next((size_t)id_range, -1);
  std::vector<uint8_t> in((size_t)id_range, 0);
  int32_t head = -1, tail = -1;
  int64_t held = 0, misses = 0;
  for (int64_t i = 0; i < n; ++i) {
    const int32_t c = ids[i];
    if (c < 0 || c >= id_range) continue;
    if (in[c]) {
      if (head == c) continue;
      // unlink
      const int32_t p = prev[c], q = next[c];
      next[p] = q;
      if (q >= 0) prev[q] = p; else tail = p;
    } else {
      ++misses;
      in[c] = 1;
      if (held == capacity) {  // evict the least recent
        const int32_t t = tail;
        tail = prev[t];
        if (tail >= 0) next[tail] = -1; else head = -1;
        in[t] = 0;
      } else {
        ++held;
      }
    }
    prev[c] = -1;
    next[c] = head;
    if (head >= 0) prev[head] = c;
    head = c;
    if (tail < 0) tail = c;
  }
  return misses;
}

// The benchmark configurations by name.  scale < 1 shrinks vertex and edge
// counts together (tests); scale = 1 is the benchmark size.  Parameters were
// calibrated so that the full-size graphs land on the configured statistics:
//   c1_citation   20,000 vertices, mean degree ~5, max ~170-190
//   c2_social     232,965 vertices, ~114.6 M nonzeros, max degree ~21,000
//   c3_copurchase 2,449,029 vertices, ~123.7 M nonzeros (80 % of the edge
//                 samples are intra-community; communities of ~37 vertices
//                 saturate, so more samples than stored edges are drawn)
//   c4_rmat       R-MAT scale 22, edge factor 16
hpspmm_graph* hpspmm_gen_named(const char* name, double scale) {
  const std::string n = name ? name : "";
  if (!(scale > 0)) {
    g_err = "gen_named: scale must be positive";
    return nullptr;
  }
  auto scaled = [&](double full, int64_t floor_) {
    return std::max<int64_t>(floor_, (int64_t)std::llround(full * scale));
  };
  if (n == "c0_uniform") {
    const int64_t v = scaled(4096, 16);
    return hpspmm_gen_uniform_rows(v, v, 16, 0);
  }
  if (n == "c1_citation") {
    const int64_t v = scaled(20000, 64);
    return hpspmm_gen_citation(v, 2.5, 70, (int64_t)std::llround(2.05 * (double)v), 1);
  }
  if (n == "c2_social")
    return hpspmm_gen_powerlaw(scaled(232965, 64), 2.1, std::max(4.0, 520.0 * scale),
                               (int64_t)std::llround(60.45e6 * scale), kValSymUniform01, 2);
  if (n == "c3_copurchase")
    return hpspmm_gen_community(scaled(2449029, 64), 3.5, 1.0, scaled(65536, 1), 0.8,
                                (int64_t)std::llround(165.4e6 * scale), 3);
  if (n == "c4_rmat") {
    const int sc = scale >= 1 ? 22 : std::max(6, 22 + (int)std::floor(std::log2(scale)));
    return hpspmm_gen_rmat(sc, (int64_t)16 << sc, 0.57, 0.19, 0.19, 4);
  }
  // Held-out families (scale 1 = about 10^8 nonzeros):
  //   h1_prefattach  preferential attachment, 24 edges per new vertex
  //   h2_rmat        R-MAT with a flatter quadrant law (0.45, 0.22, 0.22, 0.11), edge factor 24
  //   h3_grid        9-point stencil + 2 random edges per vertex, about 13 nonzeros per row
  //   h4_bipartite   users x items (8 : 1), lognormal basket sizes (mean ~60), Zipf(0.9) popularity
  //   h5_blocks      communities of 8 to 4096 vertices, 90 % of the edges inside, mean degree ~40
  //   h6_uniform100  100 uniformly placed nonzeros in every row
  //   h7_groups      users x items (1 : 2) with communities: the first half of the rows of a community graph
  //                  (lognormal(3.2, 0.8) weights, communities of ~48, 70 % of the edges inside)
  if (n == "h1_prefattach") return hpspmm_gen_pref_attach(scaled(2.1e6, 64), 24, 11);
  if (n == "h2_rmat") {
    const int sc = std::max(6, 21 + (int)std::lround(std::log2(scale)));
    return hpspmm_gen_rmat(sc, (int64_t)24 << sc, 0.45, 0.22, 0.22, 12);
  }
  if (n == "h3_grid") return hpspmm_gen_grid(std::max<int64_t>(8, (int64_t)std::llround(2800.0 * std::sqrt(scale))), 2, 13);
  if (n == "h4_bipartite") return hpspmm_gen_bipartite(scaled(1.7e6, 64), scaled(2.1e5, 64), 3.8, 0.8, 0.9, 14);
  if (n == "h5_blocks") {
    const int64_t v = scaled(2.5e6, 64);
    return hpspmm_gen_blocks(v, 8, 4096, 0.9, (int64_t)std::llround(21.0 * (double)v), 15);
  }
  if (n == "h6_uniform100") {
    const int64_t v = scaled(1.0e6, 128);
    return hpspmm_gen_uniform_rows(v, v, 100, 16);
  }
  if (n == "h7_groups") {
    const int64_t v = scaled(3.2e6, 128);
    hpspmm_graph* whole = hpspmm_gen_community(v, 3.2, 0.8, std::max<int64_t>(1, v / 48), 0.7,
                                               (int64_t)std::llround(61.5 * (double)v), 17);
    if (!whole) return nullptr;
    Graph* g = (Graph*)whole;  // keep rows [0, v / 2): every community has members on both sides
    g->rows = v / 2;
    g->rowptr.resize((size_t)g->rows + 1);
    g->nnz = g->rowptr[(size_t)g->rows];
    g->col.resize((size_t)g->nnz);
    g->val.resize((size_t)g->nnz);
    return whole;
  }
  g_err = "gen_named: unknown configuration '" + n + "'";
  return nullptr;
}

// out[i] ~ N(0,1), Box-Muller on pairs (2p, 2p+1).
void hpspmm_gen_dense_normal(uint64_t seed, int64_t count, float* out) {
  const int64_t pairs = (count + 1) / 2;
#pragma omp parallel for schedule(static)
  for (int64_t p = 0; p < pairs; ++p) {
    const double u1 = u01_open0(draw(seed, 41, (uint64_t)p));
    const double u2 = u01(draw(seed, 42, (uint64_t)p));
    const double r = std::sqrt(-2.0 * std::log(u1));
    const double t = 6.283185307179586 * u2;
    out[2 * p] = (float)(r * std::cos(t));
    if (2 * p + 1 < count) out[2 * p + 1] = (float)(r * std::sin(t));
  }
}

// out[i] ~ U(lo, hi): the distribution the reference's rand() draws its dense
// operand from (test/test_all.cpp:53), here with a seed.
void hpspmm_gen_dense_uniform(uint64_t seed, int64_t count, float lo, float hi, float* out) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < count; ++i)
    out[i] = (float)((double)lo + ((double)hi - (double)lo) * u01(draw(seed, 43, (uint64_t)i)));
}

}  // extern "C"
