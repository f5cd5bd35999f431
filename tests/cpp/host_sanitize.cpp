// Host-only sanitizer harness: the inspector (every kind of schedule), its validator, the file
// readers and the reordering, compiled with -fsanitize=address,undefined together with
// csrc/tf_inspector.cpp, tf_march.cpp, tf_io.cpp and tf_reorder.cpp (no GPU code: the three functions those
// files take from the HIP side are stubbed here).  Exits 0 when every schedule validates.
#include <algorithm>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>
#include "tf_internal.h"
namespace tf {
static char g_err[512];
tf_status fail(tf_status code, const char *fmt, ...) { va_list ap; va_start(ap, fmt); vsnprintf(g_err, sizeof g_err, fmt, ap); va_end(ap); return code; }
int default_compute_units() { return 256; }
void release_device_schedule(DeviceSchedule *) {}
}
static void band(int M, int bw, int per, unsigned seed, std::vector<int> &p, std::vector<int> &i) {
  std::mt19937 g(seed); p.assign(1, 0); i.clear();
  for (int r = 0; r < M; ++r) { std::vector<int> c; for (int k = 0; k < per; ++k) { int x = r - bw / 2 + (int)(g() % bw); if (x >= 0 && x < M) c.push_back(x); }
    std::sort(c.begin(), c.end()); c.erase(std::unique(c.begin(), c.end()), c.end()); i.insert(i.end(), c.begin(), c.end()); p.push_back((int)i.size()); }
}
static void powerlaw(int M, int nnz, unsigned seed, std::vector<int> &p, std::vector<int> &i) {
  std::mt19937 g(seed); std::vector<std::vector<int>> rows(M);
  auto pick = [&]() { double u = (g() % 1000000 + 1) / 1000001.0; return (int)((M - 1) * u * u * u * u); };
  for (int k = 0; k < nnz; ++k) rows[pick()].push_back(pick());
  p.assign(1, 0); i.clear();
  for (auto &c : rows) { std::sort(c.begin(), c.end()); c.erase(std::unique(c.begin(), c.end()), c.end()); i.insert(i.end(), c.begin(), c.end()); p.push_back((int)i.size()); }
}
static int run(const char *name, int M, const std::vector<int> &p, const std::vector<int> &i, tf_inspect_opts o) {
  tf_schedule *s = nullptr;
  tf_status rc = tf_inspect(M, M, p.data(), i.data(), &o, &s);
  if (rc) { printf("%s: inspect %d %s\n", name, rc, tf::g_err); return o.op < 0 ? 0 : 1; }
  rc = tf_schedule_validate_inner(s, M, M, p.data(), i.data(), o.inner_Ap, o.inner_Ai, o.inner_cols);
  tf_schedule_info info; info.struct_size = sizeof(info); tf_schedule_get_info(s, &info);
  tf_schedule_view v; v.struct_size = sizeof(v); tf_schedule_get_view(s, &v);
  printf("%s: validate %d tiles %d fused %d long %d hot %d wide %d streamed %d ws %lld %s\n", name, rc, info.n_tiles, info.n_fused_rows, info.n_long_rows, info.long_row_hot_cols, info.wide_strips, info.streamed, info.workspace_bytes, rc ? tf::g_err : "");
  tf_schedule_free(s);
  return rc != 0;
}
int main() {
  int bad = 0;
  std::vector<int> p, i;
  band(40000, 32, 16, 1, p, i);
  { tf_inspect_opts o{}; o.struct_size = sizeof(o); o.op = TF_OP_SPMM_SPMM; o.N = 128; o.inner_Ap = p.data(); o.inner_Ai = i.data(); o.inner_cols = 40000; bad += run("band wide", 40000, p, i, o);
    o.wide_strips = -1; bad += run("band narrow", 40000, p, i, o); o.inner_Ap = nullptr; o.inner_Ai = nullptr; o.wide_strips = 0; bad += run("band general", 40000, p, i, o);
    tf_inspect_opts g{}; g.struct_size = sizeof(g); g.op = TF_OP_GEMM_SPMM; g.N = 128; g.K = 100; bad += run("band gemm stream", 40000, p, i, g); g.N = 64; g.K = 20; g.compute_units = 1024; bad += run("band gemm tiles", 40000, p, i, g); }
  {  // 7-point stencil on a 21 x 17 x 26 grid: marching runs, found from the pattern and with tiles given
    const int nx = 21, ny = 17, nz = 26, M = nx * ny * nz;
    p.assign(1, 0); i.clear();
    for (int z = 0; z < nz; ++z) for (int y = 0; y < ny; ++y) for (int x = 0; x < nx; ++x) {
      const int r = (z * ny + y) * nx + x;
      if (z > 0) i.push_back(r - nx * ny);
      if (y > 0) i.push_back(r - nx);
      if (x > 0) i.push_back(r - 1);
      i.push_back(r);
      if (x < nx - 1) i.push_back(r + 1);
      if (y < ny - 1) i.push_back(r + nx);
      if (z < nz - 1) i.push_back(r + nx * ny);
      p.push_back((int)i.size());
    }
    tf_inspect_opts o{}; o.struct_size = sizeof(o); o.op = TF_OP_SPMM_SPMM; o.N = 64; o.inner_Ap = p.data(); o.inner_Ai = i.data(); o.inner_cols = M; o.march = 1;
    bad += run("stencil march", M, p, i, o);
    o.march_tile_x = 5; o.march_tile_y = 3; o.compute_units = 7; bad += run("stencil march 5x3", M, p, i, o);
    o.march_tile_x = o.march_tile_y = 0; o.grid_nx = ny; o.grid_ny = nx; o.grid_nz = nz; bad += run("stencil march, wrong grid", M, p, i, o); }
  {  // 27-point stencil on a 13 x 11 x 9 grid: marching runs with ELL rows of 32 pairs, the grid found from thirteen distances
    const int nx = 13, ny = 11, nz = 9, M = nx * ny * nz;
    p.assign(1, 0); i.clear();
    for (int z = 0; z < nz; ++z) for (int y = 0; y < ny; ++y) for (int x = 0; x < nx; ++x) {
      for (int dz = -1; dz <= 1; ++dz) for (int dy = -1; dy <= 1; ++dy) for (int dx = -1; dx <= 1; ++dx) {
        const int X = x + dx, Y = y + dy, Z = z + dz;
        if (X >= 0 && X < nx && Y >= 0 && Y < ny && Z >= 0 && Z < nz) i.push_back((Z * ny + Y) * nx + X);
      }
      p.push_back((int)i.size());
    }
    tf_inspect_opts o{}; o.struct_size = sizeof(o); o.op = TF_OP_SPMM_SPMM; o.N = 128; o.inner_Ap = p.data(); o.inner_Ai = i.data(); o.inner_cols = M; o.march = 1;
    bad += run("27-point stencil march", M, p, i, o);
    o.compute_units = 5; bad += run("27-point stencil march, 5 units", M, p, i, o); }
  {  // 5-point stencil on a 300 x 90 grid (runs along the grid's lines) and a tall 7-point grid (more planes
     // than a run's table holds: cut into several runs along z)
    auto stencil = [&](int nx, int ny, int nz) {
      p.assign(1, 0); i.clear();
      for (int z = 0; z < nz; ++z) for (int y = 0; y < ny; ++y) for (int x = 0; x < nx; ++x) {
        const int r = (z * ny + y) * nx + x;
        if (z > 0) i.push_back(r - nx * ny);
        if (y > 0) i.push_back(r - nx);
        if (x > 0) i.push_back(r - 1);
        i.push_back(r);
        if (x < nx - 1) i.push_back(r + 1);
        if (y < ny - 1) i.push_back(r + nx);
        if (z < nz - 1) i.push_back(r + nx * ny);
        p.push_back((int)i.size());
      }
      return nx * ny * nz;
    };
    int M = stencil(300, 1, 90);
    tf_inspect_opts o{}; o.struct_size = sizeof(o); o.op = TF_OP_SPMM_SPMM; o.N = 64; o.inner_Ap = p.data(); o.inner_Ai = i.data(); o.inner_cols = M; o.march = 1;
    bad += run("flat stencil march", M, p, i, o);
    M = stencil(10, 9, 700);
    o.inner_Ap = p.data(); o.inner_Ai = i.data(); o.inner_cols = M; o.compute_units = 4;
    bad += run("tall stencil march", M, p, i, o); }
  powerlaw(60000, 1500000, 2, p, i);
  { tf_inspect_opts o{}; o.struct_size = sizeof(o); o.op = TF_OP_GEMM_SPMM; o.N = 128; o.K = 128; o.long_row_partition = 1; bad += run("powerlaw part", 60000, p, i, o);
    o.long_row_partition = -1; bad += run("powerlaw chunks", 60000, p, i, o);
    o.op = TF_OP_SPMM_SPMM; o.K = 0; o.N = 20; o.long_row_partition = 1; bad += run("powerlaw spmm part", 60000, p, i, o); }
  { std::vector<int> perm(60000); tf_status rc = tf_reorder_rcm(60000, p.data(), i.data(), perm.data()); std::vector<float> x(i.size(), 1.f); int *bp, *bi; float *bx;
    rc = rc ? rc : tf_permute_csr(60000, p.data(), i.data(), x.data(), perm.data(), &bp, &bi, &bx); printf("rcm+permute %d\n", rc); bad += rc != 0; tf_host_free(bp); tf_host_free(bi); tf_host_free(bx); }
  { std::vector<int> perm(60000), pp(18); tf_status rc = tf_reorder_partition(60000, p.data(), i.data(), 16, 0, perm.data(), pp.data());
    printf("partition ordering %d hubs %d\n", rc, pp[1]); bad += rc != 0 || pp[17] != 60000; }
  { FILE *f = fopen("host_sanitize_t.mtx", "w"); fprintf(f, "%%%%MatrixMarket matrix coordinate real symmetric\n4 4 3\n1 1 2.0\n3 1 -1\n4 4 5e-1\n"); fclose(f);
    int M, N, nnz, *ap, *ai; float *ax; tf_status rc = tf_read_matrix("host_sanitize_t.mtx", &M, &N, &nnz, &ap, &ai, &ax); printf("read %d nnz %d\n", rc, nnz); bad += rc != 0 || nnz != 4; tf_host_free(ap); tf_host_free(ai); tf_host_free(ax); }
  printf("bad %d\n", bad);
  return bad;
}
