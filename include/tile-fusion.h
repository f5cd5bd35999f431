// tile-fusion.h -- the fused-operation API of tile-fusion, backed by libtilefusion_hip
// (MI355X / gfx950).
//
// The reference documents this header in its README ("Fused Operation API",
// README.md:19-38) without shipping it; the names and signatures below are the
// README's:
//
//   swiftware::def::FusedSchedule swiftware::fusion::inspector(CSRMatrix A, int NumThreads);
//   swiftware::fusion::spMMSpMMExecutor(CSRMatrix A, CSRMatrix B, Matrix C, Matrix D,
//                                       FusedSchedule schedule, int NumThreads);
//   swiftware::fusion::geMMSpMMExecutor(CSRMatrix A, Matrix B,    Matrix C, Matrix D,
//                                       FusedSchedule schedule, int NumThreads);
//   swiftware::CSRMatrix(int M, int N, int* Ap, int* Ai, float* Ax);
//   swiftware::Matrix(int M, int N, float* Data);
//
// computing D += A * (B * C) in fp32 with int32 CSR, as the executors behind it do
// (fusion/src/SpMM_SpMM_vectorized.cpp:876-989,
//  fusion/gcn/GCN_Layer_MKL_Forward_Utils.h:218-291; callers zero D first).
//
// What is new is where the data lives.  CSRMatrix and Matrix are cheap by-value handles
// over caller-owned host arrays, as in the README, and they gain a device-resident
// buffer:
//   * toDevice() uploads the host arrays once and pins them in HBM; copies of the handle
//     share the buffer.  Call it again after changing the host data.
//   * An operand that was not pinned is staged for the duration of one executor call.
//   * If D is pinned the result stays in HBM (fetch it with D.toHost()); otherwise D is
//     uploaded, accumulated into and copied back -- exactly the reference's behaviour.
// NumThreads is accepted everywhere for source compatibility and ignored: parallelism is
// the GPU's.  Errors, which the reference does not report, throw std::runtime_error.
//
// Header-only over the C ABI in tilefusion_hip.h; link with -ltilefusion_hip.
#ifndef TILE_FUSION_H
#define TILE_FUSION_H

#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <tuple>
#include <vector>

#include "tilefusion_hip.h"

namespace swiftware {

namespace detail {
inline void check(tf_status s, const char *where) {
  if (s != TF_OK)
    throw std::runtime_error(std::string(where) + ": " + tf_last_error_string() + " (status " + std::to_string(s) + ")");
}
struct CsrState {
  tf_csr *h = nullptr;
  ~CsrState() { tf_csr_free(h); }
};
struct DenseState {
  tf_dense *h = nullptr;
  ~DenseState() { tf_dense_free(h); }
};
}  // namespace detail

namespace def {

// Non-owning CSR view: int32 Ap[M+1], Ai[nnz], fp32 Ax[nnz]  (README.md:35).
struct CSRMatrix {
  int M, N;
  int *Ap, *Ai;
  float *Ax;
  CSRMatrix(int M_, int N_, int *Ap_, int *Ai_, float *Ax_)
      : M(M_), N(N_), Ap(Ap_), Ai(Ai_), Ax(Ax_), st_(std::make_shared<detail::CsrState>()) {}
  int nnz() const { return Ap[M]; }
  // Copies the matrix to HBM and keeps it there (re-uploads if called again).
  void toDevice() {
    tf_csr *h = nullptr;
    detail::check(tf_csr_upload(M, N, Ap, Ai, Ax, &h), "CSRMatrix::toDevice");
    tf_csr_free(st_->h);
    st_->h = h;
  }
  bool onDevice() const { return st_->h != nullptr; }
  void releaseDevice() { tf_csr_free(st_->h); st_->h = nullptr; }
  const tf_csr *device() const { return st_->h; }

 private:
  std::shared_ptr<detail::CsrState> st_;
};

// Non-owning dense row-major view  (README.md:36).
struct Matrix {
  int M, N;
  float *Data;
  Matrix(int M_, int N_, float *Data_) : M(M_), N(N_), Data(Data_), st_(std::make_shared<detail::DenseState>()) {}
  // Copies Data to HBM and keeps it there (re-uploads if called again).
  void toDevice() {
    tf_dense *h = nullptr;
    detail::check(tf_dense_upload(M, N, Data, &h), "Matrix::toDevice");
    tf_dense_free(st_->h);
    st_->h = h;
  }
  // Copies the device buffer back into Data.
  void toHost() {
    if (!st_->h) throw std::runtime_error("Matrix::toHost: matrix is not on the device");
    detail::check(tf_dense_download(st_->h, Data), "Matrix::toHost");
  }
  bool onDevice() const { return st_->h != nullptr; }
  void releaseDevice() { tf_dense_free(st_->h); st_->h = nullptr; }
  tf_dense *device() const { return st_->h; }

 private:
  std::shared_ptr<detail::DenseState> st_;
};

// Owns the schedule(s) built for one sparsity pattern.  The README's inspector receives
// neither the dense widths nor the operation, which the tile height depends on (the
// reference passes them to its inspector classes out of band, Fusion_Inspector.h:851), so
// the schedule for a given (operation, N, K) is built on first use and cached here.
// After a build the reference's flat arrays (MultiDimensionalSet.h:15-21) are exposed
// through n1_/ptr1_/ptr2_/ker_begin_/id_/type_.
class FusedSchedule {
 public:
  int n1_ = 0;
  const int *ptr1_ = nullptr, *ptr2_ = nullptr, *ker_begin_ = nullptr, *id_ = nullptr, *type_ = nullptr;

  FusedSchedule() = default;
  FusedSchedule(const CSRMatrix &A, const tf_inspect_opts &base) : st_(std::make_shared<State>()) {
    st_->L = A.M;
    st_->M = A.N;
    st_->Ap.assign(A.Ap, A.Ap + A.M + 1);
    st_->Ai.assign(A.Ai, A.Ai + A.Ap[A.M]);
    st_->base = base;
  }
  // The schedule for this operation and these widths (built once, then cached).
  // inner_is_outer: SpMM-SpMM whose inner matrix B is A itself (every run of the reference,
  // fusion/example/SpMM_SpMM_Demo_Utils.h:53-54); lets the inspector build windowed tiles.
  // The flat arrays above are those of the schedule an executor last used.
  tf_schedule *get(int op, int N, int K, bool inner_is_outer = false) { return lookup(op, N, K, inner_is_outer, true); }

 private:
  tf_schedule *lookup(int op, int N, int K, bool inner_is_outer, bool expose) {
    if (!st_) throw std::runtime_error("FusedSchedule: empty schedule (call inspector first)");
    auto key = std::make_tuple(op, N, inner_is_outer ? -1 : K);
    auto it = st_->built.find(key);
    if (it == st_->built.end()) {
      tf_inspect_opts o = st_->base;
      o.struct_size = sizeof(o);
      o.op = op; o.N = N; o.K = K;
      if (inner_is_outer && st_->L == st_->M) {
        o.inner_Ap = st_->Ap.data(); o.inner_Ai = st_->Ai.data(); o.inner_cols = st_->M;
      }
      tf_schedule *s = nullptr;
      detail::check(tf_inspect(st_->L, st_->M, st_->Ap.data(), st_->Ai.data(), &o, &s), "inspector");
      it = st_->built.emplace(key, std::shared_ptr<tf_schedule>(s, tf_schedule_free)).first;
    }
    if (expose) {
      st_->last_used = it->second.get();
      refresh();
    }
    return it->second.get();
  }

 public:
  // Points n1_ ... type_ at the schedule an executor last used.  The executors receive the
  // FusedSchedule by value (README.md:30-31), so the caller's own copy is brought up to date by
  // this call; validate(), validateAll() and info() make it too.
  void refresh() {
    if (!st_ || !st_->last_used) return;
    tf_schedule_view v;
    v.struct_size = sizeof(v);
    detail::check(tf_schedule_get_view(st_->last_used, &v), "FusedSchedule");
    n1_ = v.n1; ptr1_ = v.ptr1; ptr2_ = v.ptr2; ker_begin_ = v.ker_begin; id_ = v.id; type_ = v.type;
  }
  // Exact check of the schedule for (op, N, K) against the pattern it was built from.  Pass
  // inner_is_outer = true for the schedule spMMSpMMExecutor uses when B is A (windowed tiles).
  void validate(int op, int N, int K, bool inner_is_outer = false) {
    tf_schedule *s = lookup(op, N, K, inner_is_outer, false);
    const bool inner = inner_is_outer && st_->L == st_->M;
    detail::check(tf_schedule_validate_inner(s, st_->L, st_->M, st_->Ap.data(), st_->Ai.data(), inner ? st_->Ap.data() : nullptr,
                                             inner ? st_->Ai.data() : nullptr, inner ? st_->M : 0),
                  "FusedSchedule::validate");
    refresh();
  }
  // Checks every schedule built so far (the ones the executors have run).
  void validateAll() {
    for (auto &kv : st_->built) {
      const bool inner = std::get<2>(kv.first) == -1 && st_->L == st_->M;
      detail::check(tf_schedule_validate_inner(kv.second.get(), st_->L, st_->M, st_->Ap.data(), st_->Ai.data(),
                                               inner ? st_->Ap.data() : nullptr, inner ? st_->Ai.data() : nullptr, inner ? st_->M : 0),
                    "FusedSchedule::validateAll");
    }
    refresh();
  }
  tf_schedule_info info(int op, int N, int K, bool inner_is_outer = false) {
    tf_schedule_info i;
    i.struct_size = sizeof(i);
    detail::check(tf_schedule_get_info(lookup(op, N, K, inner_is_outer, false), &i), "FusedSchedule::info");
    refresh();
    return i;
  }

 private:
  struct State {
    int L = 0, M = 0;
    std::vector<int> Ap, Ai;
    tf_inspect_opts base{};
    std::map<std::tuple<int, int, int>, std::shared_ptr<tf_schedule>> built;
    tf_schedule *last_used = nullptr;  // owned by `built`
  };
  std::shared_ptr<State> st_;
};

}  // namespace def

// The README spells the operand types both ways.
using CSRMatrix = def::CSRMatrix;
using Matrix = def::Matrix;

namespace fusion {

// README.md:25.  Records A's sparsity pattern; tiles are cut on first executor call.
inline def::FusedSchedule inspector(def::CSRMatrix A, int NumThreads) {
  (void)NumThreads;
  tf_inspect_opts base{};
  return def::FusedSchedule(A, base);
}
// Same, with explicit schedule parameters (LDS budget, tile rows, recomputation limit).
inline def::FusedSchedule inspector(def::CSRMatrix A, int NumThreads, const tf_inspect_opts &opts) {
  (void)NumThreads;
  return def::FusedSchedule(A, opts);
}

namespace detail_exec {
struct StagedCsr {
  const tf_csr *h = nullptr;
  tf_csr *tmp = nullptr;
  explicit StagedCsr(const def::CSRMatrix &a) {
    if (a.onDevice()) { h = a.device(); return; }
    detail::check(tf_csr_upload(a.M, a.N, a.Ap, a.Ai, a.Ax, &tmp), "executor (upload sparse operand)");
    h = tmp;
  }
  ~StagedCsr() { tf_csr_free(tmp); }
};
struct StagedDense {
  tf_dense *h = nullptr;
  tf_dense *tmp = nullptr;
  explicit StagedDense(const def::Matrix &m) {
    if (m.onDevice()) { h = m.device(); return; }
    detail::check(tf_dense_upload(m.M, m.N, m.Data, &tmp), "executor (upload dense operand)");
    h = tmp;
  }
  ~StagedDense() { tf_dense_free(tmp); }
};
}  // namespace detail_exec

// README.md:30.  D += A * (B * C), A and B sparse.
inline void spMMSpMMExecutor(def::CSRMatrix A, def::CSRMatrix B, def::Matrix C, def::Matrix D,
                             def::FusedSchedule schedule, int NumThreads) {
  (void)NumThreads;
  const bool same_arrays = (B.Ap == A.Ap && B.Ai == A.Ai && B.Ax == A.Ax && B.M == A.M && B.N == A.N);
  tf_schedule *s = schedule.get(TF_OP_SPMM_SPMM, C.N, 0, same_arrays);
  detail_exec::StagedCsr a(A);
  const bool same = same_arrays && (!B.onDevice() || B.device() == A.device());
  detail_exec::StagedCsr b(same ? A : B);
  const tf_csr *bh = same ? a.h : b.h;
  detail_exec::StagedDense c(C), d(D);
  detail::check(tf_spmm_spmm(a.h, bh, c.h, d.h, s, TF_ACCUMULATE, nullptr), "spMMSpMMExecutor");
  if (d.tmp) detail::check(tf_dense_download(d.tmp, D.Data), "spMMSpMMExecutor (download D)");
  else detail::check(tf_device_synchronize(), "spMMSpMMExecutor");
}

// README.md:31.  D += A * (B * C), A sparse, B (M x K) and C (K x N) dense.
inline void geMMSpMMExecutor(def::CSRMatrix A, def::Matrix B, def::Matrix C, def::Matrix D,
                             def::FusedSchedule schedule, int NumThreads) {
  (void)NumThreads;
  tf_schedule *s = schedule.get(TF_OP_GEMM_SPMM, C.N, B.N);
  detail_exec::StagedCsr a(A);
  detail_exec::StagedDense b(B), c(C), d(D);
  detail::check(tf_gemm_spmm(a.h, b.h, c.h, d.h, s, TF_ACCUMULATE, nullptr), "geMMSpMMExecutor");
  if (d.tmp) detail::check(tf_dense_download(d.tmp, D.Data), "geMMSpMMExecutor (download D)");
  else detail::check(tf_device_synchronize(), "geMMSpMMExecutor");
}

}  // namespace fusion
}  // namespace swiftware

#endif  // TILE_FUSION_H
