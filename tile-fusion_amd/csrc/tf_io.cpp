// Readers for the on-disk inputs the reference's drivers take: MatrixMarket ".mtx"
// (coordinate or array; symmetric files expanded to the full matrix, as the drivers do with
// make_full before anything else, fusion/example/SpMM_SpMM_SP_Demo.cpp:24-32) and the DLMC
// ".smtx" pattern format (fusion/src/Fusion_Utils.cpp:205-250: "rows, cols, nnz", the row
// pointers, the column indices; every value is 1).  Host-only code, no GPU involved.
#include <algorithm>
#include <cctype>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <numeric>
#include <sstream>
#include <string>
#include <vector>

#include "tf_internal.h"

namespace {

std::string lower(std::string s) {
  for (auto &c : s) c = (char)std::tolower((unsigned char)c);
  return s;
}

struct Triplet {
  int r, c;
  double v;
};

// Sorted CSR with duplicates summed, handed to the caller in malloc'ed arrays.
tf_status to_csr(int M, int N, std::vector<Triplet> &t, int *outM, int *outN, int *out_nnz, int **Ap, int **Ai,
                 float **Ax) {
  std::sort(t.begin(), t.end(), [](const Triplet &a, const Triplet &b) { return a.r != b.r ? a.r < b.r : a.c < b.c; });
  size_t w = 0;
  for (size_t i = 0; i < t.size(); ++i) {
    if (w > 0 && t[w - 1].r == t[i].r && t[w - 1].c == t[i].c) t[w - 1].v += t[i].v;
    else t[w++] = t[i];
  }
  t.resize(w);
  if (w > (size_t)INT32_MAX) return tf::fail(TF_EUNSUPPORTED, "matrix has more than 2^31-1 entries");
  int *p = (int *)std::malloc(sizeof(int) * ((size_t)M + 1));
  int *ci = (int *)std::malloc(sizeof(int) * std::max<size_t>(w, 1));
  float *x = (float *)std::malloc(sizeof(float) * std::max<size_t>(w, 1));
  if (!p || !ci || !x) {
    std::free(p); std::free(ci); std::free(x);
    return tf::fail(TF_ENOMEM, "out of host memory reading a matrix");
  }
  std::fill(p, p + M + 1, 0);
  for (const auto &e : t) ++p[e.r + 1];
  for (int i = 0; i < M; ++i) p[i + 1] += p[i];
  for (size_t k = 0; k < w; ++k) { ci[k] = t[k].c; x[k] = (float)t[k].v; }
  *outM = M; *outN = N; *out_nnz = (int)w; *Ap = p; *Ai = ci; *Ax = x;
  return TF_OK;
}

bool has_suffix(const std::string &s, const char *suf) {
  const size_t n = std::strlen(suf);
  return s.size() >= n && lower(s.substr(s.size() - n)) == suf;
}

// MatrixMarket banner: %%MatrixMarket matrix <coordinate|array> <real|integer|pattern|complex> <general|symmetric|skew-symmetric|hermitian>
struct Banner {
  bool coordinate = true, pattern = false;
  int sym = 0;  // 0 general, 1 symmetric, -1 skew-symmetric
};

tf_status read_banner(std::ifstream &f, const char *path, Banner *b, std::string *size_line) {
  std::string line;
  if (!std::getline(f, line)) return tf::fail(TF_EINVAL, "%s: empty file", path);
  std::istringstream ss(line);
  std::string mm, obj, fmt, field, symm;
  ss >> mm >> obj >> fmt >> field >> symm;
  if (lower(mm) != "%%matrixmarket" || lower(obj) != "matrix")
    return tf::fail(TF_EINVAL, "%s: not a MatrixMarket matrix file", path);
  fmt = lower(fmt); field = lower(field); symm = lower(symm);
  if (fmt != "coordinate" && fmt != "array") return tf::fail(TF_EUNSUPPORTED, "%s: format '%s'", path, fmt.c_str());
  b->coordinate = fmt == "coordinate";
  if (field == "complex") return tf::fail(TF_EUNSUPPORTED, "%s: complex matrices are not supported", path);
  if (field != "real" && field != "integer" && field != "pattern" && field != "double")
    return tf::fail(TF_EUNSUPPORTED, "%s: field '%s'", path, field.c_str());
  b->pattern = field == "pattern";
  if (symm == "general") b->sym = 0;
  else if (symm == "symmetric") b->sym = 1;
  else if (symm == "skew-symmetric") b->sym = -1;
  else return tf::fail(TF_EUNSUPPORTED, "%s: symmetry '%s'", path, symm.c_str());
  while (std::getline(f, line)) {
    size_t i = 0;
    while (i < line.size() && std::isspace((unsigned char)line[i])) ++i;
    if (i == line.size() || line[i] == '%') continue;
    *size_line = line;
    return TF_OK;
  }
  return tf::fail(TF_EINVAL, "%s: no size line", path);
}

}  // namespace

static tf_status read_matrix_impl(const char *path, int *M, int *N, int *nnz, int **Ap, int **Ai, float **Ax);

// No C++ exception leaves the C ABI: a malformed size line must not end the process.
extern "C" tf_status tf_read_matrix(const char *path, int *M, int *N, int *nnz, int **Ap, int **Ai, float **Ax) {
  if (!path || !M || !N || !nnz || !Ap || !Ai || !Ax) return tf::fail(TF_EINVAL, "tf_read_matrix: null argument");
  *Ap = nullptr; *Ai = nullptr; *Ax = nullptr;
  try {
    return read_matrix_impl(path, M, N, nnz, Ap, Ai, Ax);
  } catch (const std::bad_alloc &) {
    return tf::fail(TF_ENOMEM, "%s: out of host memory", path);
  } catch (const std::exception &e) {
    return tf::fail(TF_EINVAL, "%s: %s", path, e.what());
  }
}

static tf_status read_matrix_impl(const char *path, int *M, int *N, int *nnz, int **Ap, int **Ai, float **Ax) {
  const std::string p(path);
  std::ifstream f(path);
  if (!f.is_open()) return tf::fail(TF_EINVAL, "%s: cannot open", path);
  std::vector<Triplet> t;
  if (has_suffix(p, ".smtx")) {
    std::string line;
    if (!std::getline(f, line)) return tf::fail(TF_EINVAL, "%s: empty file", path);
    std::replace(line.begin(), line.end(), ',', ' ');
    std::istringstream first(line);
    long long rows = -1, cols = -1, n = -1;
    first >> rows >> cols >> n;
    if (rows < 0 || cols < 0 || n < 0 || rows > INT32_MAX || cols > INT32_MAX || n > INT32_MAX)
      return tf::fail(TF_EINVAL, "%s: bad size line", path);
    std::vector<long long> ptr((size_t)rows + 1);
    for (auto &v : ptr)
      if (!(f >> v)) return tf::fail(TF_EINVAL, "%s: row pointers end early", path);
    if (ptr[0] != 0 || ptr[(size_t)rows] != n) return tf::fail(TF_EINVAL, "%s: row pointers do not span the entries", path);
    for (long long i = 0; i < rows; ++i) {
      if (ptr[i + 1] < ptr[i]) return tf::fail(TF_EINVAL, "%s: row pointers decrease at row %lld", path, i);
      for (long long k = ptr[i]; k < ptr[i + 1]; ++k) {
        long long c;
        if (!(f >> c)) return tf::fail(TF_EINVAL, "%s: column indices end early", path);
        if (c < 0 || c >= cols) return tf::fail(TF_EINVAL, "%s: column %lld out of range in row %lld", path, c, i);
        t.push_back({(int)i, (int)c, 1.0});
      }
    }
    return to_csr((int)rows, (int)cols, t, M, N, nnz, Ap, Ai, Ax);
  }
  if (!has_suffix(p, ".mtx")) return tf::fail(TF_EUNSUPPORTED, "%s: file extension is not supported (.mtx, .smtx)", path);
  Banner b;
  std::string size_line;
  if (tf_status rc = read_banner(f, path, &b, &size_line)) return rc;
  std::istringstream ss(size_line);
  long long rows = -1, cols = -1, n = -1;
  if (b.coordinate) ss >> rows >> cols >> n;
  else { ss >> rows >> cols; n = rows * cols; }
  if (rows < 0 || cols < 0 || n < 0 || rows > INT32_MAX || cols > INT32_MAX)
    return tf::fail(TF_EINVAL, "%s: bad size line", path);
  // int32 indexing: a symmetric file may double its entries on expansion
  if (b.coordinate && n > (b.sym ? INT32_MAX / 2 : INT32_MAX))
    return tf::fail(TF_EUNSUPPORTED, "%s: %lld entries exceed int32 indexing", path, n);
  if (b.sym != 0 && rows != cols) return tf::fail(TF_EINVAL, "%s: a symmetric matrix must be square", path);
  {  // an entry takes at least two bytes of the file, whatever the size line claims
    const std::streampos here = f.tellg();
    f.seekg(0, std::ios::end);
    const long long left = (long long)(f.tellg() - here);
    f.seekg(here);
    const long long cap = std::max<long long>(left / 2 + 1, 0);
    t.reserve((size_t)std::min<long long>(b.sym ? 2 * std::min(n, cap) : std::min(n, cap), (long long)INT32_MAX));
  }
  if (b.coordinate) {
    for (long long k = 0; k < n; ++k) {
      long long r, c;
      double v = 1.0;
      if (!(f >> r >> c)) return tf::fail(TF_EINVAL, "%s: entries end early (%lld of %lld)", path, k, n);
      if (!b.pattern && !(f >> v)) return tf::fail(TF_EINVAL, "%s: entry %lld has no value", path, k);
      if (r < 1 || r > rows || c < 1 || c > cols) return tf::fail(TF_EINVAL, "%s: entry %lld (%lld, %lld) out of range", path, k, r, c);
      t.push_back({(int)(r - 1), (int)(c - 1), v});
      if (b.sym != 0 && r != c) t.push_back({(int)(c - 1), (int)(r - 1), b.sym > 0 ? v : -v});
    }
  } else {  // dense array, column by column; symmetric files hold the lower triangle only
    for (long long c = 0; c < cols; ++c)
      for (long long r = (b.sym != 0 ? c + (b.sym < 0 ? 1 : 0) : 0); r < rows; ++r) {
        double v;
        if (!(f >> v)) return tf::fail(TF_EINVAL, "%s: values end early", path);
        if (v != 0.0) {
          t.push_back({(int)r, (int)c, v});
          if (b.sym != 0 && r != c) t.push_back({(int)c, (int)r, b.sym > 0 ? v : -v});
        }
      }
  }
  return to_csr((int)rows, (int)cols, t, M, N, nnz, Ap, Ai, Ax);
}

extern "C" tf_status tf_read_dense(const char *path, int *M, int *N, float **data) {
  if (!path || !M || !N || !data) return tf::fail(TF_EINVAL, "tf_read_dense: null argument");
  *data = nullptr;
  int nnz = 0, *Ap = nullptr, *Ai = nullptr;
  float *Ax = nullptr;
  if (tf_status rc = tf_read_matrix(path, M, N, &nnz, &Ap, &Ai, &Ax)) return rc;
  float *d = (float *)std::calloc(std::max<size_t>((size_t)*M * (size_t)*N, 1), sizeof(float));
  if (!d) {
    std::free(Ap); std::free(Ai); std::free(Ax);
    return tf::fail(TF_ENOMEM, "out of host memory reading a dense matrix");
  }
  for (int i = 0; i < *M; ++i)
    for (int k = Ap[i]; k < Ap[i + 1]; ++k) d[(size_t)i * *N + Ai[k]] = Ax[k];
  std::free(Ap); std::free(Ai); std::free(Ax);
  *data = d;
  return TF_OK;
}

extern "C" void tf_host_free(void *p) { std::free(p); }
