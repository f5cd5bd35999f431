// Reordering for locality: reverse Cuthill-McKee and a partition-based ordering on the symmetrised
// pattern, and the symmetric permutation of a CSR matrix.  The reference reorders its inputs offline with
// scipy.sparse.csgraph.reverse_cuthill_mckee and A[perm,:][:,perm]
// (fusion/scripts/reorder_graphs.py:3,21-22) so that rows that depend on each other sit close
// together and tiles fuse; this is the same step as a library call.  Host-only code.
#include <algorithm>
#include <climits>
#include <cstdlib>
#include <stdexcept>
#include <numeric>
#include <vector>

#include "tf_internal.h"

namespace {

// Adjacency of A + A^T without the diagonal, as CSR (neighbours sorted by index).
void symmetrise(int M, const int *Ap, const int *Ai, std::vector<int> *ptr, std::vector<int> *adj) {
  std::vector<int> cnt(M + 1, 0);
  long long total = 0;
  for (int i = 0; i < M; ++i)
    for (int k = Ap[i]; k < Ap[i + 1]; ++k)
      if (Ai[k] != i) { ++cnt[i + 1]; ++cnt[Ai[k] + 1]; total += 2; }
  if (total > INT_MAX) throw std::length_error("the symmetrised pattern exceeds int32 indexing");
  for (int i = 0; i < M; ++i) cnt[i + 1] += cnt[i];
  std::vector<int> raw(cnt[M]), pos(cnt.begin(), cnt.end() - 1);
  for (int i = 0; i < M; ++i)
    for (int k = Ap[i]; k < Ap[i + 1]; ++k)
      if (Ai[k] != i) { raw[pos[i]++] = Ai[k]; raw[pos[Ai[k]]++] = i; }
  ptr->assign(M + 1, 0);
  adj->clear();
  adj->reserve(raw.size());
  for (int i = 0; i < M; ++i) {
    std::sort(raw.begin() + cnt[i], raw.begin() + cnt[i + 1]);
    const auto e = std::unique(raw.begin() + cnt[i], raw.begin() + cnt[i + 1]);
    adj->insert(adj->end(), raw.begin() + cnt[i], e);
    (*ptr)[i + 1] = (int)adj->size();
  }
}

// Breadth-first levels from `root` inside its component; returns the last level's nodes and the depth.
int bfs_levels(int root, const std::vector<int> &ptr, const std::vector<int> &adj, std::vector<int> &mark, int stamp,
               std::vector<int> &queue, std::vector<int> *last_level) {
  queue.clear();
  queue.push_back(root);
  mark[root] = stamp;
  size_t level_begin = 0;
  int depth = 0;
  for (;;) {
    const size_t level_end = queue.size();
    for (size_t q = level_begin; q < level_end; ++q)
      for (int k = ptr[queue[q]]; k < ptr[queue[q] + 1]; ++k)
        if (mark[adj[k]] != stamp) { mark[adj[k]] = stamp; queue.push_back(adj[k]); }
    if (queue.size() == level_end) {
      last_level->assign(queue.begin() + level_begin, queue.begin() + level_end);
      return depth;
    }
    level_begin = level_end;
    ++depth;
  }
}

}  // namespace

extern "C" tf_status tf_reorder_rcm(int M, const int *Ap, const int *Ai, int *perm) {
  if (M < 0 || !Ap || !perm || (M > 0 && Ap[M] > 0 && !Ai)) return tf::fail(TF_EINVAL, "tf_reorder_rcm: null argument");
  if (M == 0) return TF_OK;
  if (Ap[0] != 0) return tf::fail(TF_EINVAL, "tf_reorder_rcm: Ap[0] must be 0");
  for (int i = 0; i < M; ++i) {
    if (Ap[i + 1] < Ap[i]) return tf::fail(TF_EINVAL, "tf_reorder_rcm: row pointers decrease at row %d", i);
    for (int k = Ap[i]; k < Ap[i + 1]; ++k)
      if (Ai[k] < 0 || Ai[k] >= M) return tf::fail(TF_EINVAL, "tf_reorder_rcm: column %d out of range in row %d (the matrix must be square)", Ai[k], i);
  }
  try {
    std::vector<int> ptr, adj;
    symmetrise(M, Ap, Ai, &ptr, &adj);
    auto degree = [&](int v) { return ptr[v + 1] - ptr[v]; };
    std::vector<int> by_degree(M);
    std::iota(by_degree.begin(), by_degree.end(), 0);
    std::stable_sort(by_degree.begin(), by_degree.end(), [&](int a, int b) { return degree(a) < degree(b); });
    std::vector<int> mark(M, 0), queue, last, order;
    std::vector<char> placed(M, 0);
    order.reserve(M);
    queue.reserve(M);
    int stamp = 0;
    std::vector<int> nb;
    for (int s : by_degree) {
      if (placed[s]) continue;
      // pseudo-peripheral start (George & Liu): walk to a minimum-degree node of the last
      // level while the level structure keeps getting deeper
      int root = s;
      int depth = bfs_levels(root, ptr, adj, mark, ++stamp, queue, &last);
      for (int it = 0; it < 8; ++it) {
        int cand = last[0];
        for (int v : last)
          if (degree(v) < degree(cand)) cand = v;
        std::vector<int> last2;
        const int d2 = bfs_levels(cand, ptr, adj, mark, ++stamp, queue, &last2);
        if (d2 <= depth) break;
        root = cand; depth = d2; last.swap(last2);
      }
      // Cuthill-McKee: breadth first, the new neighbours of a node in order of degree
      size_t head = order.size();
      order.push_back(root);
      placed[root] = 1;
      while (head < order.size()) {
        const int v = order[head++];
        nb.clear();
        for (int k = ptr[v]; k < ptr[v + 1]; ++k)
          if (!placed[adj[k]]) { placed[adj[k]] = 1; nb.push_back(adj[k]); }
        std::stable_sort(nb.begin(), nb.end(), [&](int a, int b) { return degree(a) < degree(b); });
        order.insert(order.end(), nb.begin(), nb.end());
      }
    }
    for (int i = 0; i < M; ++i) perm[i] = order[M - 1 - i];  // reversed
  } catch (const std::bad_alloc &) {
    return tf::fail(TF_ENOMEM, "tf_reorder_rcm: out of host memory");
  } catch (const std::exception &e) {
    return tf::fail(TF_EUNSUPPORTED, "tf_reorder_rcm: %s", e.what());
  }
  return TF_OK;
}

// Partition-based ordering: the vertices in `n_parts` parts of (almost) equal size, each grown breadth-first
// from a seed so that most edges stay inside a part, the parts one after the other; vertices of very high
// degree ("hubs": more than hub_degree neighbours) are taken out first and placed in front, by falling degree.
// The reference reorders with a graph partitioner for the same purpose (METIS, metis_perm_general at
// fusion/src/Fusion_Utils.cpp:181-203; not shipped with it): rows that depend on each other end up in one
// stretch of the matrix, so that tiles of consecutive rows hold their dependences.  Greedy graph growing is
// the classical initial partitioner of such packages; it needs no refinement to cut a mesh into compact
// pieces.  On a power-law graph the hubs would pull every part into one blob within two BFS levels, which
// is why they are set aside: in front, they also make the most-read intermediate rows one contiguous
// stretch of memory.
extern "C" tf_status tf_reorder_partition(int M, const int *Ap, const int *Ai, int n_parts, int hub_degree, int *perm,
                                          int *part_ptr) {
  if (M < 0 || !Ap || !perm || (M > 0 && Ap[M] > 0 && !Ai)) return tf::fail(TF_EINVAL, "tf_reorder_partition: null argument");
  if (n_parts <= 0) return tf::fail(TF_EINVAL, "tf_reorder_partition: n_parts must be positive");
  if (M == 0) {
    if (part_ptr) for (int p = 0; p <= n_parts + 1; ++p) part_ptr[p] = 0;
    return TF_OK;
  }
  if (Ap[0] != 0) return tf::fail(TF_EINVAL, "tf_reorder_partition: Ap[0] must be 0");
  for (int i = 0; i < M; ++i) {
    if (Ap[i + 1] < Ap[i]) return tf::fail(TF_EINVAL, "tf_reorder_partition: row pointers decrease at row %d", i);
    for (int k = Ap[i]; k < Ap[i + 1]; ++k)
      if (Ai[k] < 0 || Ai[k] >= M) return tf::fail(TF_EINVAL, "tf_reorder_partition: column %d out of range in row %d (the matrix must be square)", Ai[k], i);
  }
  try {
    std::vector<int> ptr, adj;
    symmetrise(M, Ap, Ai, &ptr, &adj);
    auto degree = [&](int v) { return ptr[v + 1] - ptr[v]; };
    if (hub_degree <= 0) {  // default: 16 times the mean degree, at least 64
      const long long mean = ptr[M] / std::max(M, 1);
      hub_degree = (int)std::min<long long>(INT_MAX, std::max<long long>(64, 16 * mean));
    }
    std::vector<char> placed(M, 0);
    std::vector<int> order;
    order.reserve(M);
    for (int v = 0; v < M; ++v)
      if (degree(v) > hub_degree) { order.push_back(v); placed[v] = 1; }
    std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return degree(a) > degree(b); });
    const int n_hubs = (int)order.size();
    if (part_ptr) { part_ptr[0] = 0; part_ptr[1] = n_hubs; }
    // seeds in order of rising degree: a part starts at the rim of what is left, not in its middle
    std::vector<int> by_degree;
    by_degree.reserve(M - n_hubs);
    for (int v = 0; v < M; ++v)
      if (!placed[v]) by_degree.push_back(v);
    std::stable_sort(by_degree.begin(), by_degree.end(), [&](int a, int b) { return degree(a) < degree(b); });
    size_t next_seed = 0;
    const int rest = M - n_hubs;
    for (int p = 0; p < n_parts; ++p) {
      const int target = n_hubs + (int)((long long)rest * (p + 1) / n_parts);  // where this part ends
      size_t head = order.size();
      while ((int)order.size() < target) {
        if (head == order.size()) {  // frontier empty: the next seed continues the part
          while (next_seed < by_degree.size() && placed[by_degree[next_seed]]) ++next_seed;
          if (next_seed == by_degree.size()) break;
          const int s = by_degree[next_seed];
          placed[s] = 1;
          order.push_back(s);
        }
        const int v = order[head++];
        for (int k = ptr[v]; k < ptr[v + 1] && (int)order.size() < target; ++k)
          if (!placed[adj[k]]) { placed[adj[k]] = 1; order.push_back(adj[k]); }
      }
      if (part_ptr) part_ptr[p + 2] = (int)order.size();
    }
    if ((int)order.size() != M) return tf::fail(TF_EINVAL, "tf_reorder_partition: internal error, %zu of %d vertices placed", order.size(), M);
    for (int i = 0; i < M; ++i) perm[i] = order[i];
  } catch (const std::bad_alloc &) {
    return tf::fail(TF_ENOMEM, "tf_reorder_partition: out of host memory");
  } catch (const std::exception &e) {
    return tf::fail(TF_EUNSUPPORTED, "tf_reorder_partition: %s", e.what());
  }
  return TF_OK;
}

extern "C" tf_status tf_permute_csr(int M, const int *Ap, const int *Ai, const float *Ax, const int *perm, int **Bp,
                                    int **Bi, float **Bx) {
  if (M < 0 || !Ap || !perm || !Bp || !Bi || !Bx) return tf::fail(TF_EINVAL, "tf_permute_csr: null argument");
  *Bp = nullptr; *Bi = nullptr; *Bx = nullptr;
  const long long nnz = M > 0 ? Ap[M] : 0;
  if (nnz > 0 && (!Ai || !Ax)) return tf::fail(TF_EINVAL, "tf_permute_csr: null argument");
  std::vector<int> inv;
  try {
    inv.assign(M, -1);
  } catch (const std::bad_alloc &) {
    return tf::fail(TF_ENOMEM, "tf_permute_csr: out of host memory");
  }
  std::vector<std::pair<int, float>> row;
  try {  // room for the longest row now, so that nothing below allocates
    int longest = 0;
    for (int i = 0; i < M; ++i) longest = std::max(longest, Ap[i + 1] - Ap[i]);
    row.reserve((size_t)std::max(longest, 0));
  } catch (const std::exception &) {
    return tf::fail(TF_ENOMEM, "tf_permute_csr: out of host memory");
  }
  for (int i = 0; i < M; ++i) {
    if (perm[i] < 0 || perm[i] >= M || inv[perm[i]] >= 0) return tf::fail(TF_EINVAL, "tf_permute_csr: perm is not a permutation of 0..%d", M - 1);
    inv[perm[i]] = i;
  }
  int *p = (int *)std::malloc(sizeof(int) * ((size_t)M + 1));
  int *ci = (int *)std::malloc(sizeof(int) * (size_t)std::max<long long>(nnz, 1));
  float *x = (float *)std::malloc(sizeof(float) * (size_t)std::max<long long>(nnz, 1));
  if (!p || !ci || !x) {
    std::free(p); std::free(ci); std::free(x);
    return tf::fail(TF_ENOMEM, "tf_permute_csr: out of host memory");
  }
  p[0] = 0;
  for (int i = 0; i < M; ++i) {  // new row i is old row perm[i], old column c becomes inv[c]
    const int o = perm[i];
    row.clear();
    for (int k = Ap[o]; k < Ap[o + 1]; ++k) {
      if (Ai[k] < 0 || Ai[k] >= M) {
        std::free(p); std::free(ci); std::free(x);
        return tf::fail(TF_EINVAL, "tf_permute_csr: column %d out of range in row %d (the matrix must be square)", Ai[k], o);
      }
      row.emplace_back(inv[Ai[k]], Ax[k]);
    }
    std::stable_sort(row.begin(), row.end(), [](const std::pair<int, float> &a, const std::pair<int, float> &b) { return a.first < b.first; });
    int w = p[i];
    for (const auto &e : row) { ci[w] = e.first; x[w] = e.second; ++w; }
    p[i + 1] = w;
  }
  *Bp = p; *Bi = ci; *Bx = x;
  return TF_OK;
}
