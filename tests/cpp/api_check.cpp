// Exercises include/tile-fusion.h the way a user of the reference's README API would:
// host arrays in, inspector once, executors many times, D accumulated into.
// The operands are the reference's own SpMM-SpMM demo input (A = B = Laplacian, dense C
// all ones, fusion/example/SpMM_SpMM_Demo_Utils.h:53-59), whose result is a small integer
// per entry and is recomputed here with a grid stencil.  Prints "api_check ok" on success.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "tile-fusion.h"

using namespace swiftware;

static void stencil(int n, int N, const std::vector<float> &u, std::vector<float> &out) {
  out.assign(u.size(), 0.f);
  for (int y = 0; y < n; ++y)
    for (int x = 0; x < n; ++x)
      for (int c = 0; c < N; ++c) {
        auto at = [&](int yy, int xx) { return (yy < 0 || yy >= n || xx < 0 || xx >= n) ? 0.f : u[(size_t)(yy * n + xx) * N + c]; };
        out[(size_t)(y * n + x) * N + c] = 4.f * at(y, x) - at(y - 1, x) - at(y + 1, x) - at(y, x - 1) - at(y, x + 1);
      }
}

int main() {
  const int n = 48, M = n * n, N = 64, K = 32;
  std::vector<int> Ap(1, 0), Ai;
  std::vector<float> Ax;
  for (int y = 0; y < n; ++y)
    for (int x = 0; x < n; ++x) {
      auto put = [&](int yy, int xx, float v) { if (yy >= 0 && yy < n && xx >= 0 && xx < n) { Ai.push_back(yy * n + xx); Ax.push_back(v); } };
      put(y - 1, x, -1); put(y, x - 1, -1); put(y, x, 4); put(y, x + 1, -1); put(y + 1, x, -1);
      Ap.push_back((int)Ai.size());
    }
  def::CSRMatrix A(M, M, Ap.data(), Ai.data(), Ax.data());
  def::FusedSchedule sched = fusion::inspector(A, 8);

  // SpMM-SpMM, host operands: D must be zero on entry and is accumulated into.
  std::vector<float> ones((size_t)M * N, 1.f), D((size_t)M * N, 0.f), t, want;
  def::Matrix C(M, N, ones.data()), Dm(M, N, D.data());
  fusion::spMMSpMMExecutor(A, A, C, Dm, sched, 8);
  sched.validateAll();  // the schedule the executor just ran (built with B = A: windowed tiles)
  sched.validate(TF_OP_SPMM_SPMM, N, 0, true);
  stencil(n, N, ones, t);
  stencil(n, N, t, want);
  for (size_t i = 0; i < D.size(); ++i)
    if (D[i] != want[i]) { std::printf("spmm-spmm mismatch at %zu: %g vs %g\n", i, D[i], want[i]); return 1; }
  // A second call accumulates: D = 2 * A*(A*1).
  fusion::spMMSpMMExecutor(A, A, C, Dm, sched, 8);
  for (size_t i = 0; i < D.size(); ++i)
    if (D[i] != 2.f * want[i]) { std::printf("accumulate mismatch at %zu\n", i); return 1; }

  // GeMM-SpMM with device-resident operands: B = ones (M x K), C = ones (K x N) -> T = K everywhere.
  std::vector<float> Bh((size_t)M * K, 1.f), Wh((size_t)K * N, 1.f), D2((size_t)M * N, 0.f), kk((size_t)M * N, (float)K);
  def::Matrix B(M, K, Bh.data()), W(K, N, Wh.data()), D2m(M, N, D2.data());
  A.toDevice(); B.toDevice(); W.toDevice(); D2m.toDevice();
  fusion::geMMSpMMExecutor(A, B, W, D2m, sched, 8);
  sched.validate(TF_OP_GEMM_SPMM, N, K);
  sched.validateAll();
  D2m.toHost();
  stencil(n, N, kk, want);
  for (size_t i = 0; i < D2.size(); ++i)
    if (D2[i] != want[i]) { std::printf("gemm-spmm mismatch at %zu: %g vs %g\n", i, D2[i], want[i]); return 1; }
  if (sched.n1_ != 2 || sched.ptr1_[0] != 0 || sched.ptr2_[0] != 0) { std::printf("schedule view is off\n"); return 1; }

  // A width the MFMA kernels do not take (the reference's bCols is free): 44 columns, host operands.
  {
    const int N2 = 44;
    std::vector<float> W2h((size_t)K * N2, 1.f), D3((size_t)M * N2, 0.f), kk2((size_t)M * N2, (float)K), want2((size_t)M * N2);
    def::Matrix Bq(M, K, Bh.data()), W2(K, N2, W2h.data()), D3m(M, N2, D3.data());
    fusion::geMMSpMMExecutor(A, Bq, W2, D3m, sched, 8);
    stencil(n, N2, kk2, want2);
    for (size_t i = 0; i < D3.size(); ++i)
      if (D3[i] != want2[i]) { std::printf("gemm-spmm (44 columns) mismatch at %zu: %g vs %g\n", i, D3[i], want2[i]); return 1; }
  }

  // Errors throw instead of exiting.
  bool threw = false;
  try {
    def::Matrix bad(M, N + 4, ones.data());
    fusion::spMMSpMMExecutor(A, A, C, bad, sched, 8);
  } catch (const std::runtime_error &) { threw = true; }
  if (!threw) { std::printf("shape mismatch did not throw\n"); return 1; }
  std::printf("api_check ok\n");
  return 0;
}
