// Device-side helpers shared by the kernel files of libtilefusion_hip (gfx950): the lane-group row
// products every sparse kernel is built from, vectors of floats, streaming loads and stores, the
// workgroup-to-XCD mapping and the LDS-only barrier.
#pragma once
#include <hip/hip_runtime.h>
#include <climits>

#include "tf_internal.h"

namespace tf {

#ifndef TF_BLOCK
#define TF_BLOCK 256
#endif
constexpr int kBlock = TF_BLOCK;  // threads per workgroup of the lane-group kernels
constexpr int kXcds = 8;     // workgroup ids are dealt round-robin over the 8 XCDs

template <int V> struct alignas(4 * V) fvec { float v[V]; };

template <int V> __device__ __forceinline__ fvec<V> vzero() {
  fvec<V> r;
#pragma unroll
  for (int i = 0; i < V; ++i) r.v[i] = 0.f;
  return r;
}
template <int V> __device__ __forceinline__ void vfma(float a, const fvec<V> &x, fvec<V> &acc) {
#pragma unroll
  for (int i = 0; i < V; ++i) acc.v[i] = __builtin_fmaf(a, x.v[i], acc.v[i]);
}
template <int V> __device__ __forceinline__ void vadd(const fvec<V> &x, fvec<V> &acc) {
#pragma unroll
  for (int i = 0; i < V; ++i) acc.v[i] += x.v[i];
}
// Output that this library does not read again leaves through a streaming (nontemporal) store.
template <int V> __device__ __forceinline__ void store_streaming(float *dst, const fvec<V> &v) {
  typedef float fv __attribute__((ext_vector_type(V)));
  fv x;
#pragma unroll
  for (int u = 0; u < V; ++u) x[u] = v.v[u];
  __builtin_nontemporal_store(x, reinterpret_cast<fv *>(dst));
}
template <> __device__ __forceinline__ void store_streaming<1>(float *dst, const fvec<1> &v) {
  __builtin_nontemporal_store(v.v[0], dst);
}
// ... and input that is read once, whole cache lines per instruction, comes through a streaming load.
__device__ __forceinline__ fvec<4> load_streaming4(const float *src) {
  typedef float f4 __attribute__((ext_vector_type(4)));
  const f4 x = __builtin_nontemporal_load(reinterpret_cast<const f4 *>(src));
  fvec<4> r;
  r.v[0] = x[0]; r.v[1] = x[1]; r.v[2] = x[2]; r.v[3] = x[3];
  return r;
}

// A plain load of four floats as one value (assigning *(fvec<4> *) to a member of a struct in registers
// can stay a copy through private memory).
__device__ __forceinline__ fvec<4> load4(const float *src) {
  typedef float f4 __attribute__((ext_vector_type(4)));
  const f4 x = *reinterpret_cast<const f4 *>(src);
  fvec<4> r;
  r.v[0] = x[0]; r.v[1] = x[1]; r.v[2] = x[2]; r.v[3] = x[3];
  return r;
}

// Consecutive workgroup ids land on different XCDs (each with its own 4 MB L2).  Work items
// are cut into chunks of `bpc` consecutive items and chunk c goes to XCD c % 8, so that an
// XCD walks whole chunks in order.  With bpc = all items / 8 every XCD gets one contiguous
// run (neighbouring tiles share halo rows in one L2); with bpc = (a far stencil stride) / 8
// every XCD keeps the same slab of every plane, so the plane above and below a row are
// still in its L2 when they are needed again.  bpc <= 0 switches the remapping off.
__device__ __forceinline__ int xcd_contiguous(int bid, int bpc) {
  if (bpc <= 0) return bid;
  const int xcd = bid % kXcds, s = bid / kXcds;
  return ((s / bpc) * kXcds + xcd) * bpc + (s % bpc);
}

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every
// global load and store of the wavefront, which would cut off the loads a kernel issues
// ahead of time for a later phase; kernels that prefetch across barriers use this instead.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

template <int V> struct GlobalRows {
  const float *__restrict__ base;
  int ld;    // row stride in floats
  int coff;  // this lane's first column
  __device__ __forceinline__ fvec<V> load(int row) const {
    return *reinterpret_cast<const fvec<V> *>(base + (size_t)row * ld + coff);
  }
  // A column index whose top bit is set names a row the schedule expects no second reader to find in L2
  // ("cold"): it is fetched with a streaming load, so that it does not push a row with readers out.
  __device__ __forceinline__ fvec<V> load_flagged(int c) const {
    const float *p = base + (size_t)(c & INT_MAX) * ld + coff;
    fvec<V> r;
    if (c < 0) {
      if constexpr (V == 1) {
        r.v[0] = __builtin_nontemporal_load(p);
      } else {
        typedef float fv __attribute__((ext_vector_type(V)));
        const fv x = __builtin_nontemporal_load(reinterpret_cast<const fv *>(p));
#pragma unroll
        for (int u = 0; u < V; ++u) r.v[u] = x[u];
      }
    } else {
      r = *reinterpret_cast<const fvec<V> *>(p);
    }
    return r;
  }
};
template <int V> struct LdsRows {
  const float *base;  // slab; row r of the intermediate is at (r - first) * ld
  int ld, coff, first;
  __device__ __forceinline__ fvec<V> load(int row) const {
    return *reinterpret_cast<const fvec<V> *>(base + (row - first) * ld + coff);
  }
};

// acc += sum over stored entries k in [kb, ke) of val[k] * src.row(idx[k]), CSR order.
// All LPR lanes of the group must call this together (it shuffles inside the group).
// The group loads up to LPR (column, value) pairs with one coalesced load, then takes them
// eight (or four) at a time: all gathers of a batch are issued before its first fma, and a
// short last batch re-reads the last entry in its unused slots and skips their fma, so a
// short row costs one gather round trip instead of one per entry.
template <int V, int LPR, int B, class Src, bool FLAG = false>
__device__ __forceinline__ void row_dot_batch(int c, float a, int t, int cnt, bool col_ok, const Src &src,
                                              fvec<V> &acc) {
  int cc[B];
  float aa[B];
#pragma unroll
  for (int u = 0; u < B; ++u) {
    const int sl = min(t + u, cnt - 1);
    cc[u] = __shfl(c, sl, LPR);
    aa[u] = __shfl(a, sl, LPR);
  }
  if (col_ok) {
    fvec<V> x[B];
#pragma unroll
    for (int u = 0; u < B; ++u) {
      if constexpr (FLAG) x[u] = (t + u < cnt) ? src.load_flagged(cc[u]) : vzero<V>();
      else x[u] = (t + u < cnt) ? src.load(cc[u]) : vzero<V>();
    }
#pragma unroll
    for (int u = 0; u < B; ++u) {
      fvec<V> next = acc;
      vfma<V>(aa[u], x[u], next);
      if (t + u < cnt) acc = next;
    }
  }
}

// The same for cnt <= LPR entries already in registers: lane g of the group holds entry g.
template <int V, int LPR, class Src, bool FLAG = false>
__device__ __forceinline__ void row_dot_loaded(int c, float a, int cnt, bool col_ok, const Src &src,
                                               fvec<V> &acc) {
  int t = 0;
  if constexpr (LPR >= 8)
    for (; t + 8 <= cnt; t += 8) row_dot_batch<V, LPR, 8, Src, FLAG>(c, a, t, cnt, col_ok, src, acc);
  if (t + 4 <= cnt) { row_dot_batch<V, LPR, 4, Src, FLAG>(c, a, t, cnt, col_ok, src, acc); t += 4; }
  if (t < cnt) row_dot_batch<V, LPR, 4, Src, FLAG>(c, a, t, cnt, col_ok, src, acc);
}

template <int V, int LPR, class Src, bool FLAG = false>
__device__ __forceinline__ void row_dot(const int *__restrict__ idx, const float *__restrict__ val,
                                        int kb, int ke, int glane, bool col_ok, const Src &src,
                                        fvec<V> &acc) {
  for (int k0 = kb; k0 < ke; k0 += LPR) {
    const int k = k0 + glane;
    int c = 0;
    float a = 0.f;
    if (k < ke) { c = idx[k]; a = val[k]; }
    row_dot_loaded<V, LPR, Src, FLAG>(c, a, min(LPR, ke - k0), col_ok, src, acc);
  }
}

// The same sum with every lane reading the row's (column, value) pairs itself: the lanes of a
// group read the same address, which costs one request per group and no cross-lane traffic.
// Eight pairs, then their eight gathers, then the fmas; slots past the row's end load nothing.
// (Requesting the next eight pairs behind the current gathers, so that they arrive together, takes
// 112 registers instead of 60 and halves the wavefronts in flight: the R-MAT step went from 2.24 to
// 2.88 ms.  Wavefronts in flight are worth more to these launches than a shorter chain of dependent
// loads per row.)
template <int V, int LPR, class Src, bool FLAG = false>
__device__ __forceinline__ void row_dot_direct(const int *__restrict__ idx, const float *__restrict__ val,
                                               int kb, int ke, bool col_ok, const Src &src, fvec<V> &acc) {
  for (int k0 = kb; k0 < ke; k0 += 8) {
    int cc[8];
    float aa[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      cc[u] = 0;
      aa[u] = 0.f;
      if (k0 + u < ke) { cc[u] = idx[k0 + u]; aa[u] = val[k0 + u]; }
    }
    if (col_ok) {
      fvec<V> x[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        if constexpr (FLAG) x[u] = (k0 + u < ke) ? src.load_flagged(cc[u]) : vzero<V>();
        else x[u] = (k0 + u < ke) ? src.load(cc[u]) : vzero<V>();
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        fvec<V> next = acc;
        vfma<V>(aa[u], x[u], next);
        if (k0 + u < ke) acc = next;
      }
    }
  }
}
}  // namespace tf
