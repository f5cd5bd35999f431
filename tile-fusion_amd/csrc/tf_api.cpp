// C ABI of libtilefusion_hip: error channel, device objects, executors.
// Compiled by hipcc together with tf_inspector.cpp and tf_kernels.hip.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <new>

#include "tf_internal.h"

// ---- handles ---------------------------------------------------------------------

struct tf_csr {
  int M = 0, N = 0, nnz = 0;
  int *p = nullptr, *i = nullptr;
  float *x = nullptr;
  bool owns = false;
  // > 0 for an uploaded matrix: its device arrays never change, so work derived from its values
  // (the regrouped values of column-partitioned long rows) is done once per schedule
  unsigned long long serial = 0;
  uint64_t hash = 0;  // tf_pattern_hash of the host arrays it was uploaded from (0: unknown, wrapped)
};

struct tf_dense {
  int M = 0, N = 0;
  float *d = nullptr;
  bool owns = false;
};

namespace tf {

struct DeviceSchedule {
  int device = -1;
  TileDesc *tiles = nullptr;
  int *fused_ids = nullptr;
  int *win = nullptr;
  int *rem_rows = nullptr;
  int *zero_rows = nullptr;
  int *plain_rows = nullptr;
  int *step_begin = nullptr;  // streamed GeMM-SpMM: per launched tile, first entry in step_ptr
  int *step_ptr = nullptr;
  int *fused_rec = nullptr;
  LongChunk *long_chunks = nullptr;
  LongRow *long_rows = nullptr;
  LongRow *seg_groups = nullptr;
  float *inter = nullptr;    // M x N intermediate, only if some tile writes back
  float *partial = nullptr;  // n_long_chunks (or segments) x N
  int *seg_ptr = nullptr, *ent_src = nullptr, *ent_pos = nullptr, *seg_col = nullptr, *lrow_seg = nullptr;  // column-partitioned long rows
  float *seg_val = nullptr;  // A's values in the order of the regrouped entries
  unsigned long long seg_val_serial = 0;  // the uploaded matrix they were taken from (0: none)
  // the short remainder rows stored in the order of the row list: row pointers, columns, where each
  // value comes from in A's array, and the values themselves (of the uploaded matrix rem_val_serial)
  int *rem_ptr = nullptr, *rem_col = nullptr, *rem_src = nullptr;
  float *rem_val = nullptr;
  unsigned long long rem_val_serial = 0;
  Tile2 *l2_tiles = nullptr; // two-layer tiles
  float *hidden = nullptr;   // tf_gcn_two_layers: the first layer's output, L x K of this (second-layer) schedule
  size_t hidden_floats = 0;
  float *Bpad = nullptr;     // M x K' and K' x N copies of B and C, zero-padded, when K is not a multiple of 8
  float *Cpad = nullptr;
  float *Cpanel = nullptr;   // K' x N and L x N: one column panel of C (zero-padded) and of D, when the caller's width is
  float *Dpanel = nullptr;   // not one the kernels take (user_N != N)
  // marching runs: the schedule's lists, and the ELL rows with the operands' values filled in
  int *m_runs = nullptr, *m_row_ptr = nullptr, *m_load_ptr = nullptr, *m_load = nullptr, *m_row_out = nullptr;
  int *m_ell_off = nullptr, *m_ell_src = nullptr, *m_ell = nullptr;
  float *m_trash = nullptr;  // a row in global memory that takes the stores of lane groups without a row
  unsigned long long m_serial_a = 0, m_serial_b = 0;  // the uploaded matrices the values were taken from (0: none)
  // A second stream of the same priority for kernels that may run beside the caller's stream (the
  // hot long-row segments beside the rest of the GEMM), with the events that fork it off and join it.
  hipStream_t side = nullptr;
  hipEvent_t fork = nullptr, join = nullptr;
  // per-launch timing, when tf_schedule_set_profiling switched it on
  int prof_n = 0;
  const char *prof_name[TF_PROFILE_MAX] = {};
  hipEvent_t prof_ev[TF_PROFILE_MAX][2] = {};
};

// launchers in tf_kernels.hip
hipError_t launch_fused_spmm_spmm(const TileDesc *, int, const int *, const int *, const int *,
                                  const float *, const float *, const int *, const int *,
                                  const float *, float *, float *, int, int, int, hipStream_t);
hipError_t launch_fused_spmm_spmm_window(const TileDesc *, const int *, int, const int *, const int *,
                                         const int *, const float *, const float *, float *, int, int,
                                         int, int, hipStream_t);
hipError_t launch_fused_spmm_spmm_window64(const TileDesc *, const int *, int, const int *, const int *,
                                           const float *, int, const float *, const int *, const int *,
                                           const float *, int, float *, int, int, int, int, hipStream_t);
hipError_t launch_spmm_rows(const int *, int, const int *, const int *, const float *, const float *,
                            float *, int, int, int, int, hipStream_t, int compact = 0, int coalesced_pairs = 0, int flagged = 0);
hipError_t launch_gather_values(const int *, const float *, float *, int, hipStream_t);
hipError_t launch_march_fill(const int *, const int *, const float *, const float *, int *, size_t, hipStream_t);
hipError_t launch_fused_spmm_spmm_march(const int *, int, const int *, const int *, const int *, const int *, const int *,
                                        const float *, float *, float *, int, int, int, int, int, int, int, hipStream_t);
hipError_t launch_scatter_values(const int *, const int *, const float *, float *, int, hipStream_t);
hipError_t launch_seg_reduce(const LongRow *, int, const int *, const float *, float *, int, int, hipStream_t);
hipError_t launch_long_rows(const LongChunk *, int, const LongRow *, int, const int *, const float *,
                            const float *, float *, float *, int, int, hipStream_t);
hipError_t launch_fused_gemm_spmm(const TileDesc *, int, const int *, const float *, const float *,
                                  int, int, const int *, const int *, const float *, float *,
                                  float *, int, int, int, int, int, hipStream_t);
hipError_t launch_fused_gemm_spmm_stream(const TileDesc *, int, const int *, const int *, const int *,
                                         const float *, const float *, int, int, int, const int *,
                                         const float *, float *, float *, int, int, hipStream_t, int relu_in = 0);
hipError_t launch_gemm(const float *, const float *, float *, const int *, int, int, int, int, hipStream_t, int y_by_position = 0);
hipError_t launch_fill(float *, size_t, float, hipStream_t);
hipError_t launch_pad(const float *, int, int, float *, int, int, hipStream_t);
hipError_t launch_copy_cols(const float *, int, int, int, int, float *, int, int, int, int, int, hipStream_t);
hipError_t launch_relu(float *, size_t, hipStream_t);
hipError_t launch_fused_gcn2(const Tile2 *, int, const float *, const float *, const float *, int, int, int, const int *, const int *,
                             const float *, float *, int, int, int, hipStream_t);
hipError_t launch_zero_rows(const int *, int, float *, int, hipStream_t);
hipError_t launch_xcd_probe(int *, int, hipStream_t);
hipError_t launch_issue_probe(float *, int, int, int, int, hipStream_t);

// An intermediate larger than the 256 MB last-level cache is gone from it before its readers
// come: such rows leave through streaming stores.
inline int inter_streams(const tf_schedule *s) {
  return (size_t)s->M * s->opts.N * sizeof(float) > ((size_t)256 << 20) ? 1 : 0;
}

static thread_local char g_err[512] = "";

tf_status fail(tf_status code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

static tf_status hip_fail(hipError_t e, const char *what) {
  return fail(e == hipErrorOutOfMemory ? TF_ENOMEM : TF_EHIP, "%s: %s", what, hipGetErrorString(e));
}

#define TF_HIP(call)                                         \
  do {                                                       \
    hipError_t e_ = (call);                                  \
    if (e_ != hipSuccess) return tf::hip_fail(e_, #call);    \
  } while (0)

int default_compute_units() {
  int dev = 0, cu = 0;
  if (hipGetDevice(&dev) == hipSuccess &&
      hipDeviceGetAttribute(&cu, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && cu > 0)
    return cu;
  (void)hipGetLastError();
  return 256;
}

void release_device_schedule(DeviceSchedule *d) {
  if (!d) return;
  (void)hipFree(d->tiles); (void)hipFree(d->fused_ids); (void)hipFree(d->win); (void)hipFree(d->rem_rows); (void)hipFree(d->zero_rows); (void)hipFree(d->plain_rows);
  (void)hipFree(d->long_chunks); (void)hipFree(d->long_rows); (void)hipFree(d->seg_groups);
  (void)hipFree(d->seg_ptr); (void)hipFree(d->ent_src); (void)hipFree(d->ent_pos); (void)hipFree(d->seg_col); (void)hipFree(d->lrow_seg); (void)hipFree(d->seg_val);
  (void)hipFree(d->step_begin); (void)hipFree(d->step_ptr); (void)hipFree(d->fused_rec);
  (void)hipFree(d->inter); (void)hipFree(d->partial); (void)hipFree(d->Bpad); (void)hipFree(d->Cpad); (void)hipFree(d->Cpanel); (void)hipFree(d->Dpanel); (void)hipFree(d->hidden); (void)hipFree(d->l2_tiles);
  (void)hipFree(d->rem_ptr); (void)hipFree(d->rem_col); (void)hipFree(d->rem_src); (void)hipFree(d->rem_val);
  (void)hipFree(d->m_runs); (void)hipFree(d->m_row_ptr); (void)hipFree(d->m_load_ptr); (void)hipFree(d->m_load);
  (void)hipFree(d->m_row_out); (void)hipFree(d->m_ell_off); (void)hipFree(d->m_ell_src); (void)hipFree(d->m_ell); (void)hipFree(d->m_trash);
  if (d->side) (void)hipStreamDestroy(d->side);
  if (d->fork) (void)hipEventDestroy(d->fork);
  if (d->join) (void)hipEventDestroy(d->join);
  for (auto &pair : d->prof_ev)
    for (hipEvent_t e : pair)
      if (e) (void)hipEventDestroy(e);
  delete d;
}

template <class T> static tf_status upload_vec(const std::vector<T> &v, T **out) {
  *out = nullptr;
  if (v.empty()) return TF_OK;
  TF_HIP(hipMalloc(reinterpret_cast<void **>(out), v.size() * sizeof(T)));
  TF_HIP(hipMemcpy(*out, v.data(), v.size() * sizeof(T), hipMemcpyHostToDevice));
  return TF_OK;
}

// Device copies of the schedule arrays and the workspace, made on first use.
static tf_status ensure_device(tf_schedule *s) {
  static std::mutex mu;
  std::lock_guard<std::mutex> lock(mu);
  int dev = 0;
  TF_HIP(hipGetDevice(&dev));
  if (s->dev) {
    if (s->dev->device != dev)
      return fail(TF_ESCHEDULE, "schedule was uploaded to device %d, current device is %d", s->dev->device, dev);
    return TF_OK;
  }
  auto *d = new (std::nothrow) DeviceSchedule();
  if (!d) return fail(TF_ENOMEM, "out of host memory");
  d->device = dev;
  tf_status rc = TF_OK;
  if (s->march) {  // nothing but the run lists is needed on the device
    rc = upload_vec(s->march_runs, &d->m_runs);
    if (!rc) rc = upload_vec(s->march_row_ptr, &d->m_row_ptr);
    if (!rc) rc = upload_vec(s->march_load_ptr, &d->m_load_ptr);
    if (!rc) rc = upload_vec(s->march_load, &d->m_load);
    if (!rc) rc = upload_vec(s->march_row_out, &d->m_row_out);
    if (!rc) rc = upload_vec(s->march_ell_off, &d->m_ell_off);
    if (!rc) rc = upload_vec(s->march_ell_src, &d->m_ell_src);
    if (!rc) {
      hipError_t e = hipMalloc(reinterpret_cast<void **>(&d->m_ell), s->march_ell_off.size() * 2 * sizeof(int));
      if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&d->m_trash), 64 * sizeof(float));
      if (e == hipSuccess) e = hipMemset(d->m_trash, 0, 64 * sizeof(float));
      if (e != hipSuccess) rc = hip_fail(e, "hipMalloc(ELL rows)");
    }
    if (rc) { release_device_schedule(d); return rc; }
    s->dev = d;
    return TF_OK;
  }
  rc = upload_vec(s->launch_tiles, &d->tiles);
  if (!rc) rc = upload_vec(s->l2_tiles, &d->l2_tiles);
  if (!rc) rc = upload_vec(s->fused_ids, &d->fused_ids);
  if (!rc) rc = upload_vec(s->win, &d->win);
  if (!rc) rc = upload_vec(s->rem_rows, &d->rem_rows);
  if (!rc) rc = upload_vec(s->zero_rows, &d->zero_rows);
  if (!rc) rc = upload_vec(s->plain_rows, &d->plain_rows);
  if (!rc) rc = upload_vec(s->launch_step, &d->step_begin);
  if (!rc) rc = upload_vec(s->step_ptr, &d->step_ptr);
  if (!rc) rc = upload_vec(s->fused_rec, &d->fused_rec);
  if (!rc && !s->rem_ptr.empty()) {
    rc = upload_vec(s->rem_ptr, &d->rem_ptr);
    if (!rc) rc = upload_vec(s->rem_col, &d->rem_col);
    if (!rc) rc = upload_vec(s->rem_src, &d->rem_src);
    if (!rc) {
      hipError_t e = hipMalloc(reinterpret_cast<void **>(&d->rem_val), std::max<size_t>(s->rem_src.size(), 1) * sizeof(float));
      if (e != hipSuccess) rc = hip_fail(e, "hipMalloc(reordered rows)");
    }
  }
  if (!rc) rc = upload_vec(s->long_chunks, &d->long_chunks);
  if (!rc) rc = upload_vec(s->long_rows, &d->long_rows);
  if (!rc && s->long_part) {
    rc = upload_vec(s->seg_ptr, &d->seg_ptr);
    if (!rc) rc = upload_vec(s->ent_src, &d->ent_src);
    if (!rc) rc = upload_vec(s->ent_pos, &d->ent_pos);
    if (!rc) rc = upload_vec(s->seg_col, &d->seg_col);
    if (!rc) rc = upload_vec(s->lrow_seg, &d->lrow_seg);
    if (!rc) rc = upload_vec(s->seg_groups, &d->seg_groups);
    if (!rc) {
      hipError_t e = hipMalloc(reinterpret_cast<void **>(&d->seg_val), std::max<size_t>(s->seg_src.size(), 1) * sizeof(float));
      if (e == hipSuccess)
        e = hipMalloc(reinterpret_cast<void **>(&d->partial), (s->seg_ptr.size() - 1 + s->seg_groups.size()) * (size_t)s->opts.N * sizeof(float));
      if (e != hipSuccess) rc = hip_fail(e, "hipMalloc(long-row segments)");
    }
  }
  if (!rc && s->n_writeback_rows > 0) {
    hipError_t e = hipMalloc(reinterpret_cast<void **>(&d->inter), (size_t)s->M * s->opts.N * sizeof(float));
    if (e != hipSuccess) rc = hip_fail(e, "hipMalloc(intermediate)");
  }
  if (!rc && s->opts.op == TF_OP_GEMM_SPMM && s->user_N != s->opts.N) {
    hipError_t e = hipMalloc(reinterpret_cast<void **>(&d->Cpanel), (size_t)s->opts.K * s->opts.N * sizeof(float));
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&d->Dpanel), (size_t)s->L * s->opts.N * sizeof(float));
    if (e != hipSuccess) rc = hip_fail(e, "hipMalloc(column panels)");
  }
  if (!rc && s->opts.op == TF_OP_GEMM_SPMM && s->user_K != s->opts.K) {
    hipError_t e = hipMalloc(reinterpret_cast<void **>(&d->Bpad), (size_t)s->M * s->opts.K * sizeof(float));
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&d->Cpad), (size_t)s->opts.K * s->opts.N * sizeof(float));
    if (e != hipSuccess) rc = hip_fail(e, "hipMalloc(padded operands)");
  }
  if (!rc && !s->long_chunks.empty()) {
    hipError_t e = hipMalloc(reinterpret_cast<void **>(&d->partial), s->long_chunks.size() * (size_t)s->opts.N * sizeof(float));
    if (e != hipSuccess) rc = hip_fail(e, "hipMalloc(partials)");
  }
  if (!rc && s->long_part && s->plain_hot > 0) {
    hipError_t e = hipStreamCreateWithFlags(&d->side, hipStreamNonBlocking);
    if (e == hipSuccess) e = hipEventCreateWithFlags(&d->fork, hipEventDisableTiming);
    if (e == hipSuccess) e = hipEventCreateWithFlags(&d->join, hipEventDisableTiming);
    if (e != hipSuccess) rc = hip_fail(e, "hipStreamCreate(side stream)");
  }
  if (rc) { release_device_schedule(d); return rc; }
  s->dev = d;
  return TF_OK;
}

// Timing of one launch (or group of launches) of an executor call: events around it on its stream.
static hipError_t prof_begin(tf_schedule *s, const char *name, hipStream_t st) {
  DeviceSchedule *d = s->dev;
  if (!s->profiling || d->prof_n >= TF_PROFILE_MAX) return hipSuccess;
  const int n = d->prof_n;
  for (int q = 0; q < 2; ++q)
    if (!d->prof_ev[n][q]) {
      hipError_t e = hipEventCreate(&d->prof_ev[n][q]);
      if (e != hipSuccess) return e;
    }
  d->prof_name[n] = name;
  return hipEventRecord(d->prof_ev[n][0], st);
}
static hipError_t prof_end(tf_schedule *s, hipStream_t st) {
  DeviceSchedule *d = s->dev;
  if (!s->profiling || d->prof_n >= TF_PROFILE_MAX) return hipSuccess;
  return hipEventRecord(d->prof_ev[d->prof_n++][1], st);
}
#define TF_PHASE(sched, name, st, call)        \
  do {                                         \
    TF_HIP(tf::prof_begin(sched, name, st));   \
    TF_HIP(call);                              \
    TF_HIP(tf::prof_end(sched, st));           \
  } while (0)

static bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// The hot segments of column-partitioned long rows: segments of partition p are worked on by the
// workgroups that land on XCD p.  The values in the order of the regrouped entries -- what the
// reference's reordered adjacency (createReorderedAdj, GCN_Single_Layer_SP_Demo_Utils.h:618-653)
// is to its executors -- are built on the first call with an uploaded matrix and kept; a wrapped
// matrix can change between calls, so its values are regrouped every time.
// ensure_segment_values fills the values of ALL segments, hot and cold, so it must run on a stream
// that both the hot and the cold launch are ordered after: the caller's, before a second stream forks.
static tf_status ensure_segment_values(const tf_csr *A, tf_schedule *s, hipStream_t st) {
  DeviceSchedule *d = s->dev;
  const bool have_values = A->serial != 0 && d->seg_val_serial == A->serial;
  if (!have_values)
    TF_PHASE(s, "scatter_values_kernel", st, launch_scatter_values(d->ent_src, d->ent_pos, A->x, d->seg_val, (int)s->seg_src.size(), st));
  d->seg_val_serial = A->serial;
  return TF_OK;
}
static tf_status run_hot_segments(tf_schedule *s, hipStream_t st) {
  DeviceSchedule *d = s->dev;
  TF_PHASE(s, "spmm_rows_kernel (hot long-row segments)", st,
           launch_spmm_rows(nullptr, 8 * s->seg_per_xcd, d->seg_ptr, d->seg_col, d->seg_val, d->inter, d->partial, s->opts.N, 0, -1, 1, st, /*compact=*/0, /*coalesced_pairs=*/1));
  return TF_OK;
}

// Second-op rows that no tile fused: served from the intermediate in HBM.  hot_on_side: the hot
// long-row segments were launched on the side stream already and are joined here.
static tf_status run_remainder(const tf_csr *A, tf_dense *D, tf_schedule *s, int accumulate, bool hot_on_side, hipStream_t st) {
  DeviceSchedule *d = s->dev;
  const int N = s->opts.N;
  if (!s->zero_rows.empty() && !accumulate)  // (D += 0 needs nothing)
    TF_PHASE(s, "zero_rows_kernel (rows without entries)", st, launch_zero_rows(d->zero_rows, (int)s->zero_rows.size(), D->d, N, st));
  if (!s->rem_rows.empty() && !s->rem_ptr.empty()) {
    // The rows in the order of the list, entries side by side -- the reference's reordered adjacency
    // (createReorderedAdj, GCN_Single_Layer_SP_Demo_Utils.h:618-653; executor at
    // GCN_Layer_MKL_Forward_Utils.h:294-373).  The values are copied on the first call with an uploaded
    // matrix, whose device arrays never change, and on every call with a wrapped one.
    if (!(A->serial != 0 && d->rem_val_serial == A->serial))
      TF_PHASE(s, "gather_values_kernel", st, launch_gather_values(d->rem_src, A->x, d->rem_val, (int)s->rem_src.size(), st));
    d->rem_val_serial = A->serial;
    TF_PHASE(s, "spmm_rows_kernel (short remainder rows)", st,
             launch_spmm_rows(d->rem_rows, (int)s->rem_rows.size(), d->rem_ptr, d->rem_col, d->rem_val, d->inter, D->d, N, accumulate,
                              s->xcd_chunk_rows, /*streaming=*/1, st, /*compact=*/1, /*coalesced_pairs=*/0, s->rem_flagged ? 1 : 0));
  } else if (!s->rem_rows.empty()) {
    // identity list: no indirection needed
    TF_PHASE(s, "spmm_rows_kernel (short remainder rows)", st,
             launch_spmm_rows(s->rem_identity ? nullptr : d->rem_rows, (int)s->rem_rows.size(), A->p, A->i,
                              A->x, d->inter, D->d, N, accumulate, s->xcd_chunk_rows, /*streaming=*/1, st));
  }
  if (s->long_part) {
    const int n_hot = 8 * s->seg_per_xcd, n_seg = (int)s->seg_ptr.size() - 1;
    if (!hot_on_side) {
      if (tf_status rc = ensure_segment_values(A, s, st)) return rc;
      if (tf_status rc = run_hot_segments(s, st)) return rc;
    }
    TF_PHASE(s, "spmm_rows_kernel (cold long-row segments)", st,
             launch_spmm_rows(nullptr, n_seg - n_hot, d->seg_ptr + n_hot, d->seg_col, d->seg_val, d->inter,
                              d->partial + (size_t)n_hot * N, N, 0, 0, 1, st));
    if (hot_on_side) TF_HIP(hipStreamWaitEvent(st, d->join, 0));
    // groups of segments of the rows with many (into their own slots of `partial`), then the rows
    if (!s->seg_groups.empty())
      TF_PHASE(s, "long_seg_reduce_kernel (groups)", st,
               launch_seg_reduce(d->seg_groups, (int)s->seg_groups.size(), d->lrow_seg, d->partial, d->partial, N, 0, st));
    TF_PHASE(s, "long_seg_reduce_kernel (rows)", st,
             launch_seg_reduce(d->long_rows, (int)s->long_rows.size(), d->lrow_seg, d->partial, D->d, N, accumulate, st));
  }
  if (!s->long_chunks.empty())
    TF_PHASE(s, "spmm_long_chunk_kernel + long_row_reduce_kernel", st,
             launch_long_rows(d->long_chunks, (int)s->long_chunks.size(), d->long_rows,
                              (int)s->long_rows.size(), A->i, A->x, d->inter, d->partial, D->d, N,
                              accumulate, st));
  return TF_OK;
}

}  // namespace tf

using tf::fail;

// The fixed scratch array of tf_spmm_spmm_noalloc (further down) and its per-device address.
namespace {

constexpr size_t kScratchFloats = (size_t)8 << 20;  // 32 MiB: e.g. 65,536 intermediate rows of 128 columns
static __device__ __align__(256) float scratch[kScratchFloats];

constexpr int kMaxDevices = 64;
float *g_scratch_ptr[kMaxDevices] = {};
std::mutex g_scratch_mu;

// The device address of the current device's copy of `scratch`, looked up once per device.
// (In host code the array's name is only a handle for this lookup, never an address.)
tf_status scratch_of_current_device(float **out) {
  int dev = 0;
  TF_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return fail(TF_EUNSUPPORTED, "device ordinal %d is beyond the %d this library keeps scratch addresses for", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    void *p = nullptr;
    TF_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) return fail(TF_EHIP, "hipGetSymbolAddress returned a null address for the scratch array");
    g_scratch_ptr[dev] = static_cast<float *>(p);
  }
  *out = g_scratch_ptr[dev];
  return TF_OK;
}

// tf_gemm's buffers for shapes off the MFMA kernel's fast path: padded X, a panel of W, a panel of Y.
struct GemmWorkspace {
  float *buf[3] = {nullptr, nullptr, nullptr};
  size_t floats[3] = {0, 0, 0};
};
GemmWorkspace g_gemm_ws[kMaxDevices];

}  // namespace


// ---- errors, device, streams -----------------------------------------------------

extern "C" const char *tf_last_error_string(void) { return tf::g_err; }
extern "C" const char *tf_version(void) { return "0.1"; }

extern "C" tf_status tf_device_init(int device, tf_device_info *info) {
  int count = 0;
  hipError_t e = hipGetDeviceCount(&count);
  if (e != hipSuccess || count <= 0) {
    (void)hipGetLastError();
    return fail(TF_EHIP, "no HIP device available (%s)", e == hipSuccess ? "count is 0" : hipGetErrorString(e));
  }
  if (device < 0 || device >= count) return fail(TF_EINVAL, "device %d out of range (have %d)", device, count);
  TF_HIP(hipSetDevice(device));
  {
    float *unused = nullptr;
    if (tf_status rc = scratch_of_current_device(&unused)) return rc;
  }
  if (info) {
    if (info->struct_size < TF_SIZE_THROUGH(tf_device_info, xcd_round_robin))  // before any work is done for it
      return fail(TF_EINVAL, "tf_device_init: info->struct_size is %zu, the struct's first version has %zu bytes (set it to sizeof(tf_device_info))",
                  info->struct_size, TF_SIZE_THROUGH(tf_device_info, xcd_round_robin));
    hipDeviceProp_t p;
    TF_HIP(hipGetDeviceProperties(&p, device));
    tf_device_info full;
    std::memset(&full, 0, sizeof(full));
    tf_device_info *const caller = info;
    info = &full;
    info->device = device;
    info->compute_units = p.multiProcessorCount;
    info->xcds = 8;
    info->lds_bytes_per_block = (int)p.sharedMemPerBlock;
    int optin = 0;
    if (hipDeviceGetAttribute(&optin, hipDeviceAttributeSharedMemPerBlockOptin, device) == hipSuccess && optin > info->lds_bytes_per_block)
      info->lds_bytes_per_block = optin;
    (void)hipGetLastError();
    info->wavefront = p.warpSize;
    info->clock_khz = p.clockRate;
    info->hbm_bytes = p.totalGlobalMem;
    std::snprintf(info->arch, sizeof(info->arch), "%s", p.gcnArchName);
    // Workgroup b of a launch is expected on XCD b mod 8: checked once here, on 64 workgroups.
    info->xcd_round_robin = -1;
    int *probe = nullptr, host[64];
    if (hipMalloc(reinterpret_cast<void **>(&probe), sizeof(host)) == hipSuccess) {
      if (tf::launch_xcd_probe(probe, 64, nullptr) == hipSuccess &&
          hipMemcpy(host, probe, sizeof(host), hipMemcpyDeviceToHost) == hipSuccess) {
        bool ok = true;
        for (int b = 0; b < 64 && ok; ++b) ok = host[b] == host[b % info->xcds];
        for (int a = 0; a < info->xcds && ok; ++a)
          for (int b = a + 1; b < info->xcds && ok; ++b) ok = host[a] != host[b];
        info->xcd_round_robin = ok ? 1 : 0;
      }
      (void)hipFree(probe);
    }
    (void)hipGetLastError();
    return tf::emit_out("tf_device_init", caller, full, TF_SIZE_THROUGH(tf_device_info, xcd_round_robin));
  }
  return TF_OK;
}

extern "C" tf_status tf_device_synchronize(void) {
  TF_HIP(hipDeviceSynchronize());
  return TF_OK;
}

extern "C" tf_status tf_calibrate_issue(int role_older, int role_younger, int iters, float *ms) {
  if (!ms || iters <= 0 || iters > (1 << 20) || role_older < 0 || role_older > 3 || role_younger < 0 || role_younger > 3)
    return fail(TF_EINVAL, "tf_calibrate_issue: roles are 0 .. 3, iters 1 .. 2^20");
  float *out = nullptr;
  TF_HIP(hipMalloc(reinterpret_cast<void **>(&out), 512 * sizeof(float)));
  hipEvent_t e0 = nullptr, e1 = nullptr;
  hipError_t err = hipEventCreate(&e0);
  if (err == hipSuccess) err = hipEventCreate(&e1);
  const int cus = tf::default_compute_units(), reps = 5;
  if (err == hipSuccess) err = tf::launch_issue_probe(out, cus, iters, role_older, role_younger, nullptr);  // warm-up
  if (err == hipSuccess) err = hipEventRecord(e0, nullptr);
  for (int r = 0; r < reps && err == hipSuccess; ++r) err = tf::launch_issue_probe(out, cus, iters, role_older, role_younger, nullptr);
  if (err == hipSuccess) err = hipEventRecord(e1, nullptr);
  if (err == hipSuccess) err = hipEventSynchronize(e1);
  float t = 0.f;
  if (err == hipSuccess) err = hipEventElapsedTime(&t, e0, e1);
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  (void)hipFree(out);
  TF_HIP(err);
  *ms = t / reps;
  return TF_OK;
}

extern "C" tf_status tf_stream_create(void **stream) {
  if (!stream) return fail(TF_EINVAL, "tf_stream_create: null");
  hipStream_t s;
  TF_HIP(hipStreamCreate(&s));
  *stream = s;
  return TF_OK;
}
extern "C" tf_status tf_stream_destroy(void *stream) {
  if (stream) TF_HIP(hipStreamDestroy(static_cast<hipStream_t>(stream)));
  return TF_OK;
}
extern "C" tf_status tf_stream_synchronize(void *stream) {
  TF_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
  return TF_OK;
}
extern "C" tf_status tf_event_create(void **event) {
  if (!event) return fail(TF_EINVAL, "tf_event_create: null");
  hipEvent_t e;
  TF_HIP(hipEventCreate(&e));
  *event = e;
  return TF_OK;
}
extern "C" tf_status tf_event_destroy(void *event) {
  if (event) TF_HIP(hipEventDestroy(static_cast<hipEvent_t>(event)));
  return TF_OK;
}
extern "C" tf_status tf_event_record(void *event, void *stream) {
  TF_HIP(hipEventRecord(static_cast<hipEvent_t>(event), static_cast<hipStream_t>(stream)));
  return TF_OK;
}
extern "C" tf_status tf_event_synchronize(void *event) {
  TF_HIP(hipEventSynchronize(static_cast<hipEvent_t>(event)));
  return TF_OK;
}
extern "C" tf_status tf_event_elapsed_ms(void *start, void *stop, float *ms) {
  if (!ms) return fail(TF_EINVAL, "tf_event_elapsed_ms: null");
  TF_HIP(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
  return TF_OK;
}

// ---- operands ----------------------------------------------------------------------

extern "C" tf_status tf_csr_upload(int M, int N, const int *Ap, const int *Ai, const float *Ax,
                                   tf_csr **out) {
  if (!out) return fail(TF_EINVAL, "tf_csr_upload: out is null");
  *out = nullptr;
  if (M <= 0 || N <= 0 || !Ap) return fail(TF_EINVAL, "tf_csr_upload: bad M/N/Ap");
  if (Ap[0] != 0) return fail(TF_EINVAL, "tf_csr_upload: Ap[0] != 0");
  for (int r = 0; r < M; ++r)
    if (Ap[r + 1] < Ap[r]) return fail(TF_EINVAL, "tf_csr_upload: Ap not monotone at row %d", r);
  const int nnz = Ap[M];
  if (nnz > 0 && (!Ai || !Ax)) return fail(TF_EINVAL, "tf_csr_upload: Ai/Ax null");
  for (int k = 0; k < nnz; ++k)
    if (Ai[k] < 0 || Ai[k] >= N) return fail(TF_EINVAL, "tf_csr_upload: column %d out of range at entry %d", Ai[k], k);
  auto *a = new (std::nothrow) tf_csr();
  if (!a) return fail(TF_ENOMEM, "out of host memory");
  a->M = M; a->N = N; a->nnz = nnz; a->owns = true;
  static std::atomic<unsigned long long> next_serial{1};
  a->serial = next_serial.fetch_add(1);
  a->hash = tf_pattern_hash(M, Ap, Ai);
  hipError_t e = hipMalloc(reinterpret_cast<void **>(&a->p), (size_t)(M + 1) * sizeof(int));
  if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&a->i), (size_t)std::max(nnz, 1) * sizeof(int));
  if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&a->x), (size_t)std::max(nnz, 1) * sizeof(float));
  if (e == hipSuccess) e = hipMemcpy(a->p, Ap, (size_t)(M + 1) * sizeof(int), hipMemcpyHostToDevice);
  if (e == hipSuccess && nnz > 0) e = hipMemcpy(a->i, Ai, (size_t)nnz * sizeof(int), hipMemcpyHostToDevice);
  if (e == hipSuccess && nnz > 0) e = hipMemcpy(a->x, Ax, (size_t)nnz * sizeof(float), hipMemcpyHostToDevice);
  if (e != hipSuccess) { tf_csr_free(a); return tf::hip_fail(e, "tf_csr_upload"); }
  *out = a;
  return TF_OK;
}

extern "C" tf_status tf_csr_wrap_device(int M, int N, int nnz, const int *dAp, const int *dAi,
                                        const float *dAx, tf_csr **out) {
  if (!out) return fail(TF_EINVAL, "tf_csr_wrap_device: out is null");
  *out = nullptr;
  if (M <= 0 || N <= 0 || nnz < 0 || !dAp || (nnz > 0 && (!dAi || !dAx)))
    return fail(TF_EINVAL, "tf_csr_wrap_device: bad argument");
  auto *a = new (std::nothrow) tf_csr();
  if (!a) return fail(TF_ENOMEM, "out of host memory");
  a->M = M; a->N = N; a->nnz = nnz; a->owns = false;
  a->p = const_cast<int *>(dAp); a->i = const_cast<int *>(dAi); a->x = const_cast<float *>(dAx);
  *out = a;
  return TF_OK;
}

extern "C" tf_status tf_csr_set_pattern_hash(tf_csr *a, uint64_t hash) {
  if (!a) return fail(TF_EINVAL, "tf_csr_set_pattern_hash: null argument");
  a->hash = hash;
  return TF_OK;
}

extern "C" void tf_csr_free(tf_csr *a) {
  if (!a) return;
  if (a->owns) { (void)hipFree(a->p); (void)hipFree(a->i); (void)hipFree(a->x); }
  delete a;
}

extern "C" tf_status tf_dense_alloc(int M, int N, tf_dense **out) {
  if (!out) return fail(TF_EINVAL, "tf_dense_alloc: out is null");
  *out = nullptr;
  if (M <= 0 || N <= 0) return fail(TF_EINVAL, "tf_dense_alloc: bad shape %d x %d", M, N);
  auto *d = new (std::nothrow) tf_dense();
  if (!d) return fail(TF_ENOMEM, "out of host memory");
  d->M = M; d->N = N; d->owns = true;
  hipError_t e = hipMalloc(reinterpret_cast<void **>(&d->d), (size_t)M * N * sizeof(float));
  if (e != hipSuccess) { delete d; return tf::hip_fail(e, "tf_dense_alloc"); }
  *out = d;
  return TF_OK;
}

extern "C" tf_status tf_dense_upload(int M, int N, const float *host, tf_dense **out) {
  if (!host) return fail(TF_EINVAL, "tf_dense_upload: host is null");
  tf_status rc = tf_dense_alloc(M, N, out);
  if (rc) return rc;
  hipError_t e = hipMemcpy((*out)->d, host, (size_t)M * N * sizeof(float), hipMemcpyHostToDevice);
  if (e != hipSuccess) { tf_dense_free(*out); *out = nullptr; return tf::hip_fail(e, "tf_dense_upload"); }
  return TF_OK;
}

extern "C" tf_status tf_dense_wrap_device(int M, int N, float *dptr, tf_dense **out) {
  if (!out) return fail(TF_EINVAL, "tf_dense_wrap_device: out is null");
  *out = nullptr;
  if (M <= 0 || N <= 0 || !dptr) return fail(TF_EINVAL, "tf_dense_wrap_device: bad argument");
  if (!tf::aligned16(dptr)) return fail(TF_EINVAL, "tf_dense_wrap_device: pointer must be 16-byte aligned");
  auto *d = new (std::nothrow) tf_dense();
  if (!d) return fail(TF_ENOMEM, "out of host memory");
  d->M = M; d->N = N; d->d = dptr; d->owns = false;
  *out = d;
  return TF_OK;
}

extern "C" tf_status tf_dense_download(const tf_dense *d, float *host) {
  if (!d || !host) return fail(TF_EINVAL, "tf_dense_download: null argument");
  TF_HIP(hipMemcpy(host, d->d, (size_t)d->M * d->N * sizeof(float), hipMemcpyDeviceToHost));
  return TF_OK;
}

extern "C" tf_status tf_dense_fill(tf_dense *d, float value, void *stream) {
  if (!d) return fail(TF_EINVAL, "tf_dense_fill: null argument");
  TF_HIP(tf::launch_fill(d->d, (size_t)d->M * d->N, value, static_cast<hipStream_t>(stream)));
  return TF_OK;
}

extern "C" tf_status tf_dense_copy(tf_dense *dst, const tf_dense *src, void *stream) {
  if (!dst || !src) return fail(TF_EINVAL, "tf_dense_copy: null argument");
  if (dst->M != src->M || dst->N != src->N)
    return fail(TF_EINVAL, "tf_dense_copy: shapes differ (%d x %d and %d x %d)", dst->M, dst->N, src->M, src->N);
  TF_HIP(hipMemcpyAsync(dst->d, src->d, (size_t)src->M * src->N * sizeof(float), hipMemcpyDeviceToDevice,
                        static_cast<hipStream_t>(stream)));
  return TF_OK;
}

extern "C" float *tf_dense_device_ptr(const tf_dense *d) { return d ? d->d : nullptr; }

extern "C" void tf_dense_free(tf_dense *d) {
  if (!d) return;
  if (d->owns) (void)hipFree(d->d);
  delete d;
}

// ---- executors -----------------------------------------------------------------------

static tf_status check_common(const char *who, const tf_csr *A, const tf_dense *C, const tf_dense *D,
                              const tf_schedule *s, int op) {
  if (!A || !C || !D || !s) return fail(TF_EINVAL, "%s: null argument", who);
  if (s->opts.op != op) return fail(TF_ESCHEDULE, "%s: schedule was built for the other operation", who);
  if (A->M != s->L || A->N != s->M || A->nnz != s->nnz)
    return fail(TF_ESCHEDULE, "%s: schedule was built for a %d x %d pattern with %lld entries, A is %d x %d with %d",
                who, s->L, s->M, s->nnz, A->M, A->N, A->nnz);
  if (A->hash && A->hash != s->pattern_hash)
    return fail(TF_ESCHEDULE, "%s: A has the shape and entry count the schedule was built for, but another sparsity pattern", who);
  if (C->N != s->user_N || D->N != s->user_N)
    return fail(TF_ESCHEDULE, "%s: schedule was built for N = %d, C has %d and D has %d columns", who, s->user_N, C->N, D->N);
  if (D->M != A->M) return fail(TF_EINVAL, "%s: D has %d rows, A has %d", who, D->M, A->M);
  return TF_OK;
}

extern "C" tf_status tf_spmm_spmm(const tf_csr *A, const tf_csr *B, const tf_dense *C, tf_dense *D,
                                  tf_schedule *s, unsigned flags, void *stream) {
  tf_status rc = check_common("tf_spmm_spmm", A, C, D, s, TF_OP_SPMM_SPMM);
  if (rc) return rc;
  if (!B) return fail(TF_EINVAL, "tf_spmm_spmm: B is null");
  if (B->M != A->N) return fail(TF_EINVAL, "tf_spmm_spmm: B has %d rows, A has %d columns", B->M, A->N);
  if (C->M != B->N) return fail(TF_EINVAL, "tf_spmm_spmm: C has %d rows, B has %d columns", C->M, B->N);
  rc = tf::ensure_device(s);
  if (rc) return rc;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int acc = (flags & TF_ACCUMULATE) ? 1 : 0;
  tf::DeviceSchedule *d = s->dev;
  d->prof_n = 0;
  const int n_launch = (int)s->launch_tiles.size();
  if (s->march) {
    if (B->nnz != s->inner_nnz || B->N != s->opts.inner_cols || (B->hash && B->hash != s->inner_hash))
      return fail(TF_ESCHEDULE, "tf_spmm_spmm: the schedule's runs were built on another inner pattern than B's");
    // The values in the order of the runs' ELL rows (the reference's reordered adjacency,
    // createReorderedAdj, GCN_Single_Layer_SP_Demo_Utils.h:618-653): filled in on the first call with
    // uploaded matrices, whose device arrays never change, and on every call with wrapped ones.
    const bool have = A->serial != 0 && B->serial != 0 && d->m_serial_a == A->serial && d->m_serial_b == B->serial;
    if (!have)
      TF_PHASE(s, "march_fill_kernel", st, tf::launch_march_fill(d->m_ell_off, d->m_ell_src, A->x, B->x, d->m_ell, s->march_ell_off.size(), st));
    d->m_serial_a = A->serial;
    d->m_serial_b = B->serial;
    TF_PHASE(s, "fused_spmm_spmm_march_kernel", st,
             tf::launch_fused_spmm_spmm_march(d->m_runs, (int)s->march_runs.size() / 2, d->m_row_ptr, d->m_load_ptr, d->m_load,
                                              d->m_row_out, d->m_ell, C->d, D->d, d->m_trash, s->opts.N, s->lds_bytes, s->march_tpg,
                                              s->march_dpg, s->march_lpg, s->march_width, acc, st));
    return TF_OK;
  }
  if (s->windowed) {
    if (B->nnz != s->inner_nnz || B->N != s->opts.inner_cols)
      return fail(TF_ESCHEDULE, "tf_spmm_spmm: schedule was built for an inner pattern with %lld entries and %d columns, B has %d and %d",
                  s->inner_nnz, s->opts.inner_cols, B->nnz, B->N);
    // the windowed kernels turn B's columns into LDS offsets inside the tile's window of C: another
    // pattern would read outside it
    if (B->hash && B->hash != s->inner_hash)
      return fail(TF_ESCHEDULE, "tf_spmm_spmm: B has the shape and entry count of the inner pattern the schedule was built on, but another sparsity pattern");
    // The windowed kernel walks one staged CSR chunk for both products: B must be A.
    const bool same = (B == A) || (B->p == A->p && B->i == A->i && B->x == A->x);
    // (the kernel fetches entries four at a time and clamps the last fetch to nnz - 4: both arrays need four)
    if (s->win_wide && A->nnz >= 4 && B->nnz >= 4) {  // reads B's entries for the first product and A's for the second, in place
      TF_PHASE(s, "fused_spmm_spmm_window64_kernel", st,
               tf::launch_fused_spmm_spmm_window64(d->tiles, d->win, n_launch, B->p, B->i, B->x,
                                                   B->nnz, C->d, A->p, A->i, A->x, A->nnz, D->d, s->opts.N,
                                                   s->lds_bytes, acc, s->opts.compute_units, st));
      return TF_OK;
    }
    if (same) {
      TF_PHASE(s, "fused_spmm_spmm_window_kernel", st,
               tf::launch_fused_spmm_spmm_window(d->tiles, d->win, n_launch, d->fused_ids, A->p,
                                                 A->i, A->x, C->d, D->d, s->opts.N, s->opts.strip_cols,
                                                 s->lds_bytes, acc, st));
      return TF_OK;
    }
    if (s->lds_bytes_general > 163840)
      return fail(TF_ESCHEDULE, "tf_spmm_spmm: this schedule needs B to be the same matrix as A");
  }
  if (n_launch > 0)
    TF_PHASE(s, "fused_spmm_spmm_kernel", st,
             tf::launch_fused_spmm_spmm(d->tiles, n_launch, d->fused_ids, B->p, B->i, B->x,
                                        C->d, A->p, A->i, A->x, D->d, d->inter, s->opts.N,
                                        s->windowed ? s->lds_bytes_general : s->lds_bytes, acc, st));
  if (!s->plain_rows.empty()) {  // intermediate rows of tiles that fuse nothing
    const bool all = (int)s->plain_rows.size() == s->M;
    TF_PHASE(s, "spmm_rows_kernel (intermediate rows)", st,
             tf::launch_spmm_rows(all ? nullptr : d->plain_rows, (int)s->plain_rows.size(), B->p, B->i, B->x,
                                  C->d, d->inter, s->opts.N, 0, s->xcd_chunk_rows, tf::inter_streams(s), st));
  }
  return tf::run_remainder(A, D, s, acc, false, st);
}

// One pass of a GeMM-SpMM schedule: D (L x opts.N, dense) = A * (Bd * Cd) with Bd L' x opts.K and Cd opts.K x opts.N
// as the kernels take them.
// relu_in: Bd holds a layer's output before its activation; only for schedules that relu_on_load_ok() accepts.
static tf_status gemm_spmm_pass(const tf_csr *A, const float *Bd, const float *Cd, tf_dense *D, tf_schedule *s, int acc,
                                unsigned flags, hipStream_t st, int relu_in = 0) {
  tf::DeviceSchedule *d = s->dev;
  const int n_launch = (int)s->launch_tiles.size();
  if (n_launch > 0) {
    if (s->gemm_stream)
      TF_PHASE(s, "fused_gemm_spmm_stream_kernel", st,
               tf::launch_fused_gemm_spmm_stream(d->tiles, n_launch, d->step_begin, d->step_ptr,
                                                 d->fused_rec, Bd, Cd, s->opts.K, s->opts.N, s->ring_rows,
                                                 A->i, A->x, D->d, d->inter, s->lds_bytes, acc, st, relu_in));
    else
      TF_PHASE(s, s->gemm_regw ? "fused_gemm_spmm_regw_kernel" : "fused_gemm_spmm_kernel", st,
               tf::launch_fused_gemm_spmm(d->tiles, n_launch, d->fused_ids, Bd, Cd,
                                          s->opts.K, s->gemm_kc, A->p, A->i, A->x, D->d, d->inter,
                                          s->opts.N, s->lds_bytes, acc, s->opts.compute_units, s->gemm_regw ? 1 : 0, st));
  }
  // Column-partitioned long rows read the most-read ("hot") intermediate rows only through their
  // hot segments.  Those rows are produced first; on request (TF_SECOND_STREAM) the hot segments
  // then run on a second stream beside the rest of the GEMM and are joined before the rows' sums.
  const bool overlap = d->side && s->plain_hot > 0 && (flags & TF_SECOND_STREAM);
  if (!s->plain_rows.empty()) {  // intermediate rows of tiles that fuse nothing
    const int n_plain = (int)s->plain_rows.size();
    const int placed = s->t_pos.empty() ? 0 : 1;  // the intermediate's rows stored in the order of the list
    const bool all = n_plain == s->M && s->plain_hot == 0 && !placed;
    if (overlap) {
      TF_PHASE(s, "gemm_rows_kernel (hot rows)", st,
               tf::launch_gemm(Bd, Cd, d->inter, d->plain_rows, s->plain_hot, s->opts.K, s->opts.N, s->opts.compute_units, st, placed));
      // the regrouped values (of the hot and of the cold segments) before the fork: the cold segments run on
      // this stream and are not ordered after anything the side stream does until the join
      if (tf_status rc2 = tf::ensure_segment_values(A, s, st)) return rc2;
      TF_HIP(hipEventRecord(d->fork, st));
      TF_HIP(hipStreamWaitEvent(d->side, d->fork, 0));
      if (tf_status rc2 = tf::run_hot_segments(s, d->side)) return rc2;
      TF_HIP(hipEventRecord(d->join, d->side));
      if (n_plain > s->plain_hot)
        TF_PHASE(s, "gemm_rows_kernel (other rows)", st,
                 tf::launch_gemm(Bd, Cd, d->inter + (placed ? (size_t)s->plain_hot * s->opts.N : 0), d->plain_rows + s->plain_hot,
                                 n_plain - s->plain_hot, s->opts.K, s->opts.N, s->opts.compute_units, st, placed));
    } else {
      TF_PHASE(s, "gemm_rows_kernel", st,
               tf::launch_gemm(Bd, Cd, d->inter, all ? nullptr : d->plain_rows, n_plain, s->opts.K, s->opts.N, s->opts.compute_units, st, placed));
    }
  }
  return tf::run_remainder(A, D, s, acc, overlap && !s->plain_rows.empty(), st);
}


// A schedule whose every intermediate row is produced by the streamed kernel straight from B (no padded copy, no
// column panels, no rows left to the row GEMM) can apply an activation to B as it is read.
static bool relu_on_load_ok(const tf_schedule *s) {
  return s->gemm_stream && s->plain_rows.empty() && s->user_K == s->opts.K && s->user_N == s->opts.N && !s->launch_tiles.empty();
}

static tf_status gemm_spmm_impl(const tf_csr *A, const tf_dense *B, const tf_dense *C, tf_dense *D,
                                tf_schedule *s, unsigned flags, void *stream, int relu_in) {
  tf_status rc = check_common("tf_gemm_spmm", A, C, D, s, TF_OP_GEMM_SPMM);
  if (rc) return rc;
  if (!B) return fail(TF_EINVAL, "tf_gemm_spmm: B is null");
  if (B->M != A->N) return fail(TF_EINVAL, "tf_gemm_spmm: B has %d rows, A has %d columns", B->M, A->N);
  if (B->N != s->user_K || C->M != s->user_K)
    return fail(TF_ESCHEDULE, "tf_gemm_spmm: schedule was built for K = %d, B has %d columns and C has %d rows", s->user_K, B->N, C->M);
  rc = tf::ensure_device(s);
  if (rc) return rc;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int acc = (flags & TF_ACCUMULATE) ? 1 : 0;
  tf::DeviceSchedule *d = s->dev;
  d->prof_n = 0;
  const float *Bd = B->d, *Cd = C->d;
  const bool panels = s->user_N != s->opts.N;
  if (s->user_K != s->opts.K) {  // zero-padded copies with K rounded up to 8 (the kernels' k step)
    TF_PHASE(s, "pad_kernel (B)", st, tf::launch_pad(B->d, B->M, B->N, d->Bpad, B->M, s->opts.K, st));
    Bd = d->Bpad;
    if (!panels) {
      TF_PHASE(s, "pad_kernel (C)", st, tf::launch_pad(C->d, C->M, C->N, d->Cpad, s->opts.K, C->N, st));
      Cd = d->Cpad;
    }
  }
  if (relu_in && !relu_on_load_ok(s)) return fail(TF_EINVAL, "tf_gemm_spmm: internal error, activation on load with a schedule that cannot apply it");
  if (!panels) return gemm_spmm_pass(A, Bd, Cd, D, s, acc, flags, st, relu_in);
  // A width the MFMA kernels do not take: one pass per column panel of opts.N columns.  The panel of C is
  // copied out (zero columns past N, zero rows past K), the pass writes a dense L x opts.N panel of D,
  // and its columns are copied (or added, with TF_ACCUMULATE) into the caller's D.
  tf_dense panel = *D;
  panel.d = d->Dpanel;
  panel.N = s->opts.N;
  panel.owns = false;
  for (int q = 0; q < s->n_panels; ++q) {
    const int c0 = q * s->opts.N, w = std::min(s->opts.N, s->user_N - c0);
    TF_PHASE(s, "copy_cols_kernel (panel of C)", st,
             tf::launch_copy_cols(C->d, C->M, C->N, c0, w, d->Cpanel, s->opts.K, s->opts.N, 0, s->opts.N, 0, st));
    if (tf_status rc2 = gemm_spmm_pass(A, Bd, d->Cpanel, &panel, s, 0, flags, st)) return rc2;
    TF_PHASE(s, "copy_cols_kernel (panel of D)", st,
             tf::launch_copy_cols(d->Dpanel, D->M, s->opts.N, 0, w, D->d, D->M, D->N, c0, w, acc, st));
  }
  return TF_OK;
}

extern "C" tf_status tf_gemm_spmm(const tf_csr *A, const tf_dense *B, const tf_dense *C, tf_dense *D,
                                  tf_schedule *s, unsigned flags, void *stream) {
  return gemm_spmm_impl(A, B, C, D, s, flags, stream, 0);
}

extern "C" tf_status tf_gcn_two_layers(const tf_csr *A, const tf_dense *X, const tf_dense *W1, const tf_dense *W2, tf_dense *D,
                                       tf_schedule *s1, tf_schedule *s2, tf_dense *hidden, unsigned flags, void *stream) {
  if (!A || !X || !W1 || !W2 || !D || !s1 || !s2) return fail(TF_EINVAL, "tf_gcn_two_layers: null argument");
  if (A->M != A->N) return fail(TF_EINVAL, "tf_gcn_two_layers: A must be square (it is %d x %d)", A->M, A->N);
  const int H = W1->N;
  if (W2->M != H) return fail(TF_EINVAL, "tf_gcn_two_layers: W1 has %d columns, W2 has %d rows", H, W2->M);
  if (hidden && (hidden->M != A->M || hidden->N != H))
    return fail(TF_EINVAL, "tf_gcn_two_layers: hidden is %d x %d, expected %d x %d", hidden->M, hidden->N, A->M, H);
  // every check of shape and schedule before anything is allocated or run
  if (s1->opts.op != TF_OP_GEMM_SPMM || s2->opts.op != TF_OP_GEMM_SPMM)
    return fail(TF_ESCHEDULE, "tf_gcn_two_layers: both schedules must be built for TF_OP_GEMM_SPMM");
  if (s1->L != A->M || s1->M != A->N || s2->L != A->M || s2->M != A->N)
    return fail(TF_ESCHEDULE, "tf_gcn_two_layers: the schedules were built for %d x %d and %d x %d patterns, A is %d x %d", s1->L, s1->M, s2->L, s2->M, A->M, A->N);
  if (s1->user_N != H) return fail(TF_ESCHEDULE, "tf_gcn_two_layers: the first schedule was built for N = %d, W1 has %d columns", s1->user_N, H);
  if (s2->user_K != H) return fail(TF_ESCHEDULE, "tf_gcn_two_layers: the second schedule was built for K = %d, the hidden layer has %d columns", s2->user_K, H);
  if (X->M != A->N || X->N != s1->user_K || W1->M != s1->user_K)
    return fail(TF_ESCHEDULE, "tf_gcn_two_layers: the first schedule was built for K = %d, X is %d x %d and W1 has %d rows", s1->user_K, X->M, X->N, W1->M);
  if (W2->N != s2->user_N || D->N != s2->user_N || D->M != A->M)
    return fail(TF_ESCHEDULE, "tf_gcn_two_layers: the second schedule was built for N = %d, W2 has %d columns and D is %d x %d", s2->user_N, W2->N, D->M, D->N);
  // On request (TF_FUSE_LAYERS): one launch with the hidden layer in LDS, every tile of the second schedule's two-layer
  // tiles carrying its rows through both layers (fused_gcn2_kernel).  Not the default: a tile recomputes its
  // neighbours' halo rows in both GEMMs and runs its four phases one after the other, which on the banded 262,144-row
  // pattern (K = H = N = 128) takes 0.63 ms against 0.31 ms for the two streamed launches of the composed path.
  const bool fuse_ok = !hidden && !s2->l2_tiles.empty() && s2->user_N == s2->opts.N && s1->user_K == s1->opts.K && s1->user_K <= 256;
  if ((flags & TF_FUSE_LAYERS) && !fuse_ok)
    return fail(TF_EUNSUPPORTED, "tf_gcn_two_layers: TF_FUSE_LAYERS needs a second schedule with two-layer tiles (tf_schedule_info.two_layer_tiles: "
                "a banded pattern, widths of 32, 64 or 128), K a multiple of 8 up to 256 and no `hidden` argument");
  if (flags & TF_FUSE_LAYERS) {
    if (A->nnz != s2->nnz || (A->hash && A->hash != s2->pattern_hash))
      return fail(TF_ESCHEDULE, "tf_gcn_two_layers: the second schedule was built for another sparsity pattern than A's");
    if (tf_status rc = tf::ensure_device(s2)) return rc;
    tf::DeviceSchedule *d = s2->dev;
    d->prof_n = 0;
    hipStream_t st = static_cast<hipStream_t>(stream);
    TF_PHASE(s2, "fused_gcn2_kernel", st,
             tf::launch_fused_gcn2(d->l2_tiles, (int)s2->l2_tiles.size(), X->d, W1->d, W2->d, s1->user_K, H, s2->user_N, A->p, A->i, A->x,
                                   D->d, s2->l2_lds_bytes, (flags & TF_RELU) ? 1 : 0, (flags & TF_ACCUMULATE) ? 1 : 0, st));
    return TF_OK;
  }
  tf_dense h;
  h.M = A->M; h.N = H; h.owns = false;
  if (hidden) {
    h.d = hidden->d;
  } else {
    if (tf_status rc = tf::ensure_device(s2)) return rc;
    static std::mutex mu;  // (two threads may share a schedule object up to here; executor calls themselves are one at a time)
    std::lock_guard<std::mutex> lock(mu);
    const size_t need = (size_t)s2->L * s2->user_K;  // the hidden layer of THIS schedule: L x K
    if (!s2->dev->hidden) {
      TF_HIP(hipMalloc(reinterpret_cast<void **>(&s2->dev->hidden), need * sizeof(float)));
      s2->dev->hidden_floats = need;
    }
    if (s2->dev->hidden_floats != need)
      return fail(TF_ESCHEDULE, "tf_gcn_two_layers: the second schedule's hidden-layer buffer holds %zu floats, %zu are needed", s2->dev->hidden_floats, need);
    h.d = s2->dev->hidden;
  }
  // first layer (its schedule is checked against X and W1 there), activation, second layer.  The activation is a
  // launch of its own over the hidden layer -- unless that layer stays inside the library and the second schedule
  // streams all its rows: then the second layer's producers apply it to the hidden rows as they read them
  // (262,144-row band, K = H = N = 128: the pass over the hidden layer took 41 of the call's 343 us).
  if (tf_status rc = tf_gemm_spmm(A, X, W1, &h, s1, flags & TF_SECOND_STREAM, stream)) return rc;
  const bool relu = (flags & TF_RELU) != 0, on_load = relu && !hidden && relu_on_load_ok(s2);
  if (relu && !on_load) TF_HIP(tf::launch_relu(h.d, (size_t)h.M * h.N, static_cast<hipStream_t>(stream)));
  return gemm_spmm_impl(A, &h, W2, D, s2, flags & (TF_ACCUMULATE | TF_SECOND_STREAM), stream, on_load ? 1 : 0);
}

// ---- benchmark aid: per-launch times of the last executor call -------------------------

extern "C" tf_status tf_schedule_set_profiling(tf_schedule *s, int enable) {
  if (!s) return fail(TF_EINVAL, "tf_schedule_set_profiling: null argument");
  s->profiling = enable != 0;
  return TF_OK;
}

extern "C" tf_status tf_schedule_get_profile(tf_schedule *s, tf_profile *out) {
  if (!s || !out) return fail(TF_EINVAL, "tf_schedule_get_profile: null argument");
  tf_profile full;
  std::memset(&full, 0, sizeof(full));
  if (s->dev && s->profiling) {
    tf::DeviceSchedule *d = s->dev;
    for (int q = 0; q < d->prof_n; ++q) {
      TF_HIP(hipEventSynchronize(d->prof_ev[q][1]));
      TF_HIP(hipEventElapsedTime(&full.ms[q], d->prof_ev[q][0], d->prof_ev[q][1]));
      full.name[q] = d->prof_name[q];
    }
    full.n = d->prof_n;
  }
  return tf::emit_out("tf_schedule_get_profile", out, full, TF_SIZE_THROUGH(tf_profile, ms));
}

// ---- an executor that allocates nothing ----------------------------------------------------
//
// For callers that cannot call hipMalloc (code under HIP graph capture, serving loops, harnesses
// that forbid it): D = A*(B*C) as two row-kernel passes with the intermediate in a fixed array in
// device memory instead of a schedule's workspace.  Every GPU the library runs on holds its own
// copy of the array from the moment the library is loaded there until the process ends.

extern "C" size_t tf_noalloc_scratch_bytes(void) { return kScratchFloats * sizeof(float); }

extern "C" tf_status tf_spmm_spmm_noalloc(const tf_csr *A, const tf_csr *B, const tf_dense *C, tf_dense *D,
                                          unsigned flags, void *stream) {
  if (!A || !B || !C || !D) return fail(TF_EINVAL, "tf_spmm_spmm_noalloc: null argument");
  if (B->M != A->N) return fail(TF_EINVAL, "tf_spmm_spmm_noalloc: B has %d rows, A has %d columns", B->M, A->N);
  if (C->M != B->N) return fail(TF_EINVAL, "tf_spmm_spmm_noalloc: C has %d rows, B has %d columns", C->M, B->N);
  if (D->M != A->M || D->N != C->N)
    return fail(TF_EINVAL, "tf_spmm_spmm_noalloc: D is %d x %d, A has %d rows and C has %d columns", D->M, D->N, A->M, C->N);
  const size_t need = (size_t)B->M * C->N;
  if (need > kScratchFloats)
    return fail(TF_EUNSUPPORTED, "tf_spmm_spmm_noalloc: the intermediate (%d x %d floats, %zu bytes) exceeds the fixed scratch of %zu bytes; "
                "use tf_spmm_spmm, whose schedule allocates its workspace", B->M, C->N, need * sizeof(float), kScratchFloats * sizeof(float));
  float *T = nullptr;
  if (tf_status rc = scratch_of_current_device(&T)) return rc;
  hipStream_t st = static_cast<hipStream_t>(stream);
  // every intermediate row is overwritten (rows without entries with zeros), so nothing of the
  // previous call's contents is read
  TF_HIP(tf::launch_spmm_rows(nullptr, B->M, B->p, B->i, B->x, C->d, T, C->N, 0, 0, /*streaming=*/0, st));
  TF_HIP(tf::launch_spmm_rows(nullptr, A->M, A->p, A->i, A->x, T, D->d, C->N, (flags & TF_ACCUMULATE) ? 1 : 0, 0, /*streaming=*/1, st));
  return TF_OK;
}

extern "C" tf_status tf_spmm(const tf_csr *A, const tf_dense *X, tf_dense *Y, unsigned flags, void *stream) {
  if (!A || !X || !Y) return fail(TF_EINVAL, "tf_spmm: null argument");
  if (X->M != A->N || Y->M != A->M || X->N != Y->N)
    return fail(TF_EINVAL, "tf_spmm: shapes A %d x %d, X %d x %d, Y %d x %d", A->M, A->N, X->M, X->N, Y->M, Y->N);
  TF_HIP(tf::launch_spmm_rows(nullptr, A->M, A->p, A->i, A->x, X->d, Y->d, X->N,
                              (flags & TF_ACCUMULATE) ? 1 : 0, 0, /*streaming=*/1, static_cast<hipStream_t>(stream)));
  return TF_OK;
}

extern "C" tf_status tf_gemm(const tf_dense *X, const tf_dense *W, tf_dense *Y, void *stream) {
  if (!X || !W || !Y) return fail(TF_EINVAL, "tf_gemm: null argument");
  if (X->N != W->M || Y->M != X->M || Y->N != W->N)
    return fail(TF_EINVAL, "tf_gemm: shapes X %d x %d, W %d x %d, Y %d x %d", X->M, X->N, W->M, W->N, Y->M, Y->N);
  const int K = X->N, N = W->N, M = X->M;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (K <= 0 || N <= 0 || M <= 0) return fail(TF_EINVAL, "tf_gemm: empty operand");
  if (K % 8 == 0 && N % 32 == 0 && N <= 256) {
    TF_HIP(tf::launch_gemm(X->d, W->d, Y->d, nullptr, M, K, N, tf::default_compute_units(), st));
    return TF_OK;
  }
  // Shapes the MFMA kernel does not take: K padded to 8 with zeros and N cut into equal panels of 32 .. 256 columns,
  // in a workspace this library keeps per device.  It only ever grows: a call whose buffers fit allocates
  // nothing and does not wait for the stream; a call that needs more frees and allocates (which waits for
  // the device) and is refused while `st` is being captured into a graph.
  const int Kp = (K + 7) / 8 * 8, n_panels = (N + 255) / 256, Wd = ((N + n_panels - 1) / n_panels + 31) / 32 * 32;
  const size_t need[3] = {Kp != K ? (size_t)M * Kp : 0, (size_t)Kp * Wd, (size_t)M * Wd};
  int dev = 0;
  TF_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return fail(TF_EUNSUPPORTED, "tf_gemm: device ordinal %d is beyond the %d this library keeps workspaces for", dev, kMaxDevices);
  static std::mutex mu;
  std::lock_guard<std::mutex> lock(mu);
  GemmWorkspace &ws = g_gemm_ws[dev];
  for (int q = 0; q < 3; ++q) {
    if (need[q] <= ws.floats[q]) continue;
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &cap) == hipSuccess && cap != hipStreamCaptureStatusNone)
      return fail(TF_EUNSUPPORTED, "tf_gemm: this shape needs a larger workspace than the library holds, which cannot be allocated while the "
                  "stream is being captured; call it once with this shape outside the capture first");
    (void)hipGetLastError();
    (void)hipFree(ws.buf[q]);  // (waits for work that may still use it)
    ws.buf[q] = nullptr;
    ws.floats[q] = 0;
    hipError_t e = hipMalloc(reinterpret_cast<void **>(&ws.buf[q]), need[q] * sizeof(float));
    if (e != hipSuccess) return tf::hip_fail(e, "hipMalloc(tf_gemm workspace)");
    ws.floats[q] = need[q];
  }
  float *Xp = need[0] ? ws.buf[0] : nullptr, *Wp = ws.buf[1], *Yp = ws.buf[2];
  if (Xp) TF_HIP(tf::launch_pad(X->d, M, K, Xp, M, Kp, st));
  for (int q = 0; q < n_panels; ++q) {
    const int c0 = q * Wd, w = std::min(Wd, N - c0);
    TF_HIP(tf::launch_copy_cols(W->d, K, N, c0, w, Wp, Kp, Wd, 0, Wd, 0, st));
    TF_HIP(tf::launch_gemm(Xp ? Xp : X->d, Wp, Yp, nullptr, M, Kp, Wd, tf::default_compute_units(), st));
    TF_HIP(tf::launch_copy_cols(Yp, M, Wd, 0, w, Y->d, M, N, c0, w, 0, st));
  }
  return TF_OK;
}
